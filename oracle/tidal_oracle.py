"""CPU oracle for TidalDecode's decode-attention path.  TEST INFRASTRUCTURE ONLY.

This file restates, in plain torch-CPU / numpy fp32, what the reference computes on the decode
path, so that the HIP kernels can be checked against it.  Only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` may import it; the
product (``tidaldecode_amd``) never does.

Reference lines each function follows (paths relative to the reference checkout):

* ``attn_logits``, ``select_layer``, ``sparse_layer``  src/tidal_build/modify_llama.py:82-83,103-133
* ``TidalSchedule``                                     src/tidal_build/modify_llama.py:84,116 and
                                                        src/models/llama_tidaldecoding.py:983-985,1019
* ``rope_hf``                                           src/models/llama_tidaldecoding.py:248-279
* ``rope_closed_form``                                  kernels/src/include/cpu_reference.h:36-53
* ``k_elem_offset``/``v_elem_offset``                   kernels/include/decode/decode_page.cuh:191-234
* ``paged_append``                                      kernels/src/include/cpu_reference.h:294-327
* ``paged_selected_attention``                          kernels/src/include/cpu_reference.h:161-292
                                                        (selected pages + forced last page)
* ``stable_topk``/``head_sum_scores``                   the benchmark configuration's rule (softmax
                                                        summed over heads, ties to the lower index);
                                                        per-head mode is modify_llama.py:118

Pinning (tests/test_oracle.py): dense attention against
``torch.nn.functional.scaled_dot_product_attention`` and a pure-Python brute force; top-k against
``torch.topk`` as sets, closed-form special cases (k=1 argmax, k=N everything) and a brute-force
tie case; sparse attention against the gather form, permutation invariance, k=N and k=1 special
cases; RoPE against transformers' ``apply_rotary_pos_emb`` / ``LlamaRotaryEmbedding`` and its
algebraic invariants; paged addressing by append -> gather round trips under page permutations
and against the C restatement in ``oracle/cpu_reference.c``.  No function here is
"parity unpinned".
"""
import math
from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch


# --------------------------------------------------------------------------------------------
# dense math of the patched attention forward
# --------------------------------------------------------------------------------------------
def repeat_kv(x: torch.Tensor, n_rep: int) -> torch.Tensor:
    """[N, H_kv, D] -> [N, H_kv * n_rep, D]; query head h reads KV head h // n_rep
    (modify_llama.py:82-83, transformers' repeat_kv)."""
    if n_rep == 1:
        return x
    n, h, d = x.shape
    return x[:, :, None, :].expand(n, h, n_rep, d).reshape(n, h * n_rep, d)


def attn_logits(q: torch.Tensor, k: torch.Tensor) -> torch.Tensor:
    """q [H_q, D], k [N, H_kv, D] -> logits [H_q, N] = q K^T / sqrt(D) (modify_llama.py:105-107)."""
    q = q.float()
    k = repeat_kv(k.float(), q.shape[0] // k.shape[1])
    return torch.einsum("hd,nhd->hn", q, k) / math.sqrt(q.shape[-1])


def softmax_pv(logits: torch.Tensor, v: torch.Tensor) -> torch.Tensor:
    """fp32 softmax then P @ V (modify_llama.py:130-133).  logits [H_q, N], v [N, H_kv, D]."""
    p = torch.softmax(logits.float(), dim=-1)
    v = repeat_kv(v.float(), logits.shape[0] // v.shape[1])
    return torch.einsum("hn,nhd->hd", p, v)


def full_attention(q, k, v) -> torch.Tensor:
    """Dense decode attention of one query token, [H_q, D]."""
    return softmax_pv(attn_logits(q, k), v)


def stable_topk(scores: torch.Tensor, k: int) -> torch.Tensor:
    """Row-wise indices of the k largest scores; ties go to the lower index; each row is
    returned sorted by ascending index.  int64 [R, k]."""
    k = min(int(k), scores.shape[-1])
    order = torch.sort(scores.float(), dim=-1, descending=True, stable=True).indices[..., :k]
    return torch.sort(order, dim=-1).values


def page_score_bound(q: torch.Tensor, k: torch.Tensor, page_size: int) -> torch.Tensor:
    """Page-level upper bound of the logits from per-page element-wise key max / min (the
    estimator of the reference's ancestor: compute_max_possible,
    kernels/include/decode/decode_attn.cuh:142-172; test loop kernels/src/test/test_max_possible.cu:81-100):
    bound[h, p] = sum_d max(q[h, d] * max_p[d], q[h, d] * min_p[d]), unscaled.
    q [H_q, D], k [N, H_kv, D]; pages are the full and partial groups of page_size tokens.
    Returns [H_q, ceil(N / page_size)]."""
    q, k = q.float(), k.float()
    n, hkv, d = k.shape
    hq = q.shape[0]
    n_pages = (n + page_size - 1) // page_size
    pad = n_pages * page_size - n
    inf = torch.full((pad, hkv, d), float("inf"))
    mx = torch.cat([k, -inf]).view(n_pages, page_size, hkv, d).max(1).values  # [pages, H_kv, D]
    mn = torch.cat([k, inf]).view(n_pages, page_size, hkv, d).min(1).values
    mx = mx.repeat_interleave(hq // hkv, 1)                                    # [pages, H_q, D]
    mn = mn.repeat_interleave(hq // hkv, 1)
    return torch.maximum(q[None] * mx, q[None] * mn).sum(-1).t().contiguous()  # [H_q, pages]


def head_sum_scores(logits: torch.Tensor, rows: int = 1) -> torch.Tensor:
    """Softmax probabilities summed over the query heads of each of `rows` equal groups:
    [H_q, N] -> [rows, N] (rows=1: all heads; rows=H_kv: per KV head)."""
    p = torch.softmax(logits.float(), dim=-1)
    h, n = p.shape
    return p.reshape(rows, h // rows, n).sum(dim=1)


def select_layer(q, k, v, top_k: int, mode: str = "per_head"
                 ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Token-selection layer (modify_llama.py:112-120,130-133): attends to every token and picks
    the token budget.  Returns (o [H_q, D], indices [rows, budget] ascending, logits [H_q, N]).

    mode "per_head": one row per query head, top-k of the logits (the reference's torch.topk on
    attn_weights; softmax is monotone per head so logits and probabilities select the same set).
    mode "head_sum" / "group_sum": one shared row / one row per KV head, top-k of the summed
    softmax probabilities.
    """
    logits = attn_logits(q, k)
    budget = min(logits.shape[-1], int(top_k))  # modify_llama.py:112-113
    if mode == "per_head":
        idx = stable_topk(logits, budget)
    elif mode == "head_sum":
        idx = stable_topk(head_sum_scores(logits, 1), budget)
    elif mode == "group_sum":
        idx = stable_topk(head_sum_scores(logits, k.shape[1]), budget)
    else:
        raise KeyError(mode)
    return softmax_pv(logits, v), idx, logits


def mask_from_indices(idx: torch.Tensor, num_q_heads: int, n: int) -> torch.Tensor:
    """pos_dict of the reference: zeros.scatter_(-1, idx, 1.0) (modify_llama.py:119-120),
    broadcast to query heads when idx has fewer rows."""
    rows = idx.shape[0]
    m = torch.zeros(rows, n).scatter_(-1, idx.long(), 1.0)
    return m.repeat_interleave(num_q_heads // rows, dim=0)


def sparse_layer(q, k, v, mask: torch.Tensor) -> torch.Tensor:
    """Sparse layer (modify_llama.py:121-133): dense logits, masked_fill(mask == 0, finfo.min),
    fp32 softmax, P @ V."""
    logits = attn_logits(q, k)
    logits = logits.masked_fill(mask == 0, torch.finfo(logits.dtype).min)
    return softmax_pv(logits, v)


def sparse_layer_gather(q, k, v, idx: torch.Tensor) -> torch.Tensor:
    """Same result by attending only to the gathered rows; idx [rows, budget] with rows in
    {H_q, H_kv, 1}."""
    hq, d = q.shape
    hkv = k.shape[1]
    rows = idx.shape[0]
    out = torch.empty(hq, d)
    for h in range(hq):
        r = h * rows // hq
        sel = idx[r].long()
        kh = k[sel, h // (hq // hkv)].float()
        vh = v[sel, h // (hq // hkv)].float()
        p = torch.softmax(kh @ q[h].float() / math.sqrt(d), dim=-1)
        out[h] = p @ vh
    return out


class TidalSchedule:
    """Which layer does what during decode (modify_llama.py:84,116; the mask set by a selection
    layer is handed from layer to layer and reset every forward,
    llama_tidaldecoding.py:983-985,1019)."""

    def __init__(self, num_layers: int, sparse_layer_start: int = 2, correction_layer: int = 13):
        self.num_layers = num_layers
        self.sparse_layer_start = sparse_layer_start
        self.correction_layer = correction_layer

    def kind(self, layer: int) -> str:
        if layer < self.sparse_layer_start:
            return "full"
        if layer == self.sparse_layer_start or layer == self.correction_layer:
            return "select"
        return "sparse"


def decode_step_layers(qs: Sequence[torch.Tensor], ks: Sequence[torch.Tensor],
                       vs: Sequence[torch.Tensor], schedule: TidalSchedule, top_k: int,
                       mode: str = "per_head") -> Tuple[List[torch.Tensor], List[Optional[torch.Tensor]]]:
    """One decode step over all layers with independent per-layer q, K, V: returns the attention
    outputs and the index list that was in force at each layer (None for full layers)."""
    outs, used = [], []
    idx = None  # pos_dict = None at the start of every forward
    for layer in range(schedule.num_layers):
        q, k, v = qs[layer], ks[layer], vs[layer]
        kind = schedule.kind(layer)
        if kind == "full":
            outs.append(full_attention(q, k, v))
            used.append(None)
        elif kind == "select":
            o, idx, _ = select_layer(q, k, v, top_k, mode)
            outs.append(o)
            used.append(idx)
        else:
            if idx is None:
                raise ValueError("pos dict should be set up in sparse attn layers")
            outs.append(sparse_layer(q, k, v, mask_from_indices(idx, q.shape[0], k.shape[0])))
            used.append(idx)
    return outs, used


# --------------------------------------------------------------------------------------------
# RoPE
# --------------------------------------------------------------------------------------------
def rope_closed_form(x: np.ndarray, positions: np.ndarray, theta: float = 1e4,
                     scale: float = 1.0) -> np.ndarray:
    """Rotate-half RoPE in float64: x [N, H, D], positions [N].  For j < D/2 and
    a = pos / scale * theta^(-2j/D):  y[j] = x[j] cos a - x[j+D/2] sin a,
    y[j+D/2] = x[j+D/2] cos a + x[j] sin a   (cpu_reference.h:36-53)."""
    x = np.asarray(x, dtype=np.float64)
    n, h, d = x.shape
    half = d // 2
    j = np.arange(half, dtype=np.float64)
    ang = (np.asarray(positions, dtype=np.float64)[:, None] / scale) * theta ** (-2.0 * j / d)
    cs, sn = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    lo, hi = x[..., :half], x[..., half:]
    return np.concatenate([lo * cs - hi * sn, hi * cs + lo * sn], axis=-1)


def rope_hf(x: torch.Tensor, positions: torch.Tensor, theta: float = 1e4) -> torch.Tensor:
    """The fp32 pipeline of the patched model (llama_tidaldecoding.py:248-279): inv_freq and the
    position product in fp32, cos/sin of that, x*cos + rotate_half(x)*sin.  x [N, H, D] fp32."""
    d = x.shape[-1]
    inv_freq = 1.0 / (theta ** (torch.arange(0, d, 2, dtype=torch.int64).float() / d))
    freqs = positions.float()[:, None] * inv_freq[None, :]
    emb = torch.cat((freqs, freqs), dim=-1)
    cos, sin = emb.cos()[:, None, :], emb.sin()[:, None, :]
    x1, x2 = x[..., : d // 2], x[..., d // 2:]
    return x * cos + torch.cat((-x2, x1), dim=-1) * sin


# --------------------------------------------------------------------------------------------
# paged pool
# --------------------------------------------------------------------------------------------
NHD, HND = 0, 1


def k_elem_offset(page, head, entry, feat, num_heads, page_size, head_dim, layout=NHD):
    """decode_page.cuh:191-201"""
    if layout == HND:
        return ((page * 2 * num_heads + head) * page_size + entry) * head_dim + feat
    return ((page * 2 * page_size + entry) * num_heads + head) * head_dim + feat


def v_elem_offset(page, head, entry, feat, num_heads, page_size, head_dim, layout=NHD):
    """decode_page.cuh:223-234"""
    if layout == HND:
        return (((page * 2 + 1) * num_heads + head) * page_size + entry) * head_dim + feat
    return (((page * 2 + 1) * page_size + entry) * num_heads + head) * head_dim + feat


def pool_shape(max_pages, page_size, num_heads, head_dim, layout=NHD):
    if layout == HND:
        return (max_pages, 2, num_heads, page_size, head_dim)
    return (max_pages, 2, page_size, num_heads, head_dim)


def paged_append(pool: np.ndarray, page_indices: Sequence[int], seq_len_after: int,
                 k_new: np.ndarray, v_new: np.ndarray, layout=NHD) -> None:
    """Write the last k_new.shape[0] tokens of a sequence of seq_len_after tokens
    (cpu_reference.h:294-327).  k_new, v_new [n, H, D]; pool is modified in place."""
    n = k_new.shape[0]
    page_size = pool.shape[3] if layout == HND else pool.shape[2]
    start = seq_len_after - n
    for j in range(n):
        pos = start + j
        page = page_indices[pos // page_size]
        entry = pos % page_size
        if layout == HND:
            pool[page, 0, :, entry, :] = k_new[j]
            pool[page, 1, :, entry, :] = v_new[j]
        else:
            pool[page, 0, entry, :, :] = k_new[j]
            pool[page, 1, entry, :, :] = v_new[j]


def paged_rows(pool: np.ndarray, slots: np.ndarray, head: int, layout=NHD):
    """K and V rows [len(slots), D] of one head at physical slots (page * page_size + entry)."""
    page_size = pool.shape[3] if layout == HND else pool.shape[2]
    pages, entries = slots // page_size, slots % page_size
    if layout == HND:
        return pool[pages, 0, head, entries, :], pool[pages, 1, head, entries, :]
    return pool[pages, 0, entries, head, :], pool[pages, 1, entries, head, :]


def paged_selected_attention(q: np.ndarray, pool: np.ndarray, page_lists: np.ndarray,
                             last_page_idx: int, last_page_len: int, layout=NHD,
                             kind: str = "pages") -> Tuple[np.ndarray, List[np.ndarray]]:
    """Attention of q [H_q, D] over, for the row of each query head, the listed pages (every
    listed page is full) or token slots, followed by the first last_page_len entries of page
    last_page_idx (cpu_reference.h:161-292 with the forced last page of
    decode_page.cuh:326-329).  page_lists [rows, n] with rows in {H_q, H_kv, 1}.
    Returns (o [H_q, D] float32, per-head logits in list order)."""
    page_size = pool.shape[3] if layout == HND else pool.shape[2]
    hkv = pool.shape[2] if layout == HND else pool.shape[3]
    hq, d = q.shape
    rows = page_lists.shape[0]
    out = np.zeros((hq, d), dtype=np.float32)
    all_logits = []
    for h in range(hq):
        row = np.asarray(page_lists[h * rows // hq], dtype=np.int64)
        if kind == "pages":
            slots = (row[:, None] * page_size + np.arange(page_size)[None, :]).reshape(-1)
        else:
            slots = row
        slots = np.concatenate([slots, last_page_idx * page_size + np.arange(last_page_len)])
        kk, vv = paged_rows(pool, slots, h // (hq // hkv), layout)
        s = (kk.astype(np.float32) @ q[h].astype(np.float32)) / np.float32(math.sqrt(d))
        all_logits.append(s)
        if len(s) == 0:
            continue
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h] = p @ vv.astype(np.float32)
    return out, all_logits

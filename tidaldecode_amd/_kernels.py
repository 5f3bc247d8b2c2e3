"""Drop-in for the reference's PyBind module ``tidal._kernels`` (tidal/ops/csrc/bsk_ops.cu:4-20,
declarations tidal/ops/csrc/bsk_ops.h:23-118), backed by ``libtidal_hip.so``.

Same names, positional arguments and error behaviour (``RuntimeError`` on a failed check) as the
reference.  Differences, all additive:

* bf16 next to fp16; grouped-query attention (``num_qo_heads`` a multiple of ``num_kv_heads``);
  batches (``q`` of shape ``[B, H, D]`` with ``indptr`` of length ``B + 1``); token-granular
  index lists for ``page_size > 1`` (``index_kind="slots"``).
* ``forward`` writes ``qk_product`` when a non-empty tensor is passed (the reference's binding
  drops it, tidal/ops/csrc/approx_attn.cu:137) in list order, as natural-log-domain logits
  ``q.k/sqrt(D)``.
* kernels run on torch's current stream (the reference always uses the null stream, which is
  torch's default current stream).
"""
import math
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import (DecodePlan, FreshToken, IndexList, PagedKV, TD_BF16, TD_F16, TD_F32, TD_HND, TD_IDX_PAGES,
                   TD_IDX_SLOTS, TD_NHD, check, lib)

_DTYPES = {torch.float16: TD_F16, torch.bfloat16: TD_BF16, torch.float32: TD_F32}


def _dtype_code(t: torch.dtype, what: str) -> int:
    if t not in _DTYPES:
        raise RuntimeError(f"{what} failed to dispatch with dtype {t}")
    return _DTYPES[t]


def _check_input(x: torch.Tensor, name: str) -> None:
    # CHECK_INPUT of tidal/ops/csrc/pytorch_extension_utils.h:52-58
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if not x.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _check_rows(x: torch.Tensor, name: str) -> None:
    """2-D device tensor whose rows are dense (a column slice of a wider buffer is fine)."""
    if not x.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")
    if x.dim() != 2:
        raise RuntimeError(f"{name} must be a 2D tensor")
    if x.numel() > 0 and x.stride(1) != 1:
        raise RuntimeError(f"{name} must have dense rows")


def _check_dim(d: int, x: torch.Tensor, name: str) -> None:
    if x.dim() != d:
        raise RuntimeError(f"{name} must be a {d}D tensor")


def _check_i32(x: torch.Tensor, name: str) -> None:
    if x.dtype != torch.int32:
        raise RuntimeError(f"{name} must be int32")


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(x: Optional[torch.Tensor]) -> Optional[int]:
    return None if x is None or x.numel() == 0 else x.data_ptr()


def _pool(kv_data: torch.Tensor, layout: int, name: str = "kv_data") -> PagedKV:
    _check_input(kv_data, name)
    _check_dim(5, kv_data, name)
    if kv_data.size(1) != 2:
        raise RuntimeError(f"{name}.size(1) must be 2")
    if layout == TD_HND:
        heads, page = kv_data.size(2), kv_data.size(3)
    elif layout == TD_NHD:
        page, heads = kv_data.size(2), kv_data.size(3)
    else:
        raise RuntimeError(f"Invalid layout {layout}")
    return PagedKV(kv_data.data_ptr(), kv_data.size(0), heads, kv_data.size(4), page, layout,
                   _dtype_code(kv_data.dtype, name))


# ------------------------------------------------------------------------------------------
# free functions
# ------------------------------------------------------------------------------------------
def apply_rope_in_place(q: torch.Tensor, k: torch.Tensor, past_kv_len: int, rope_scale: float,
                        rope_theta: float) -> None:
    """bsk_ops.h:23-27 / page.cu:212-253.  q ``[N, H_q, D]``, k ``[N, H_kv, D]``."""
    _check_input(q, "q")
    _check_input(k, "k")
    _check_dim(3, q, "q")
    _check_dim(3, k, "k")
    if q.size(0) != k.size(0) or q.size(2) != k.size(2) or q.dtype != k.dtype:
        raise RuntimeError("q and k must agree in tokens, head_dim and dtype")
    check(lib.td_rope_in_place(q.data_ptr(), k.data_ptr(), q.size(0), q.size(1), k.size(1),
                               q.size(2), int(past_kv_len), float(rope_scale), float(rope_theta),
                               _dtype_code(q.dtype, "apply_rope_in_place"), _stream()))


def rms_norm_forward(input: torch.Tensor, weight: torch.Tensor, output: torch.Tensor,
                     epsilon: float) -> None:
    """bsk_ops.h:29-32 / rms_norm.cu:160-212.  input/output ``[..., C]``, weight ``[C]``."""
    _check_input(input, "input")
    _check_input(weight, "weight")
    _check_input(output, "output")
    cols = input.size(-1)
    if weight.numel() != cols or output.shape != input.shape or weight.dtype != input.dtype \
            or output.dtype != input.dtype:
        raise RuntimeError("rms_norm_forward: shape or dtype mismatch")
    check(lib.td_rms_norm(input.data_ptr(), weight.data_ptr(), output.data_ptr(),
                          input.numel() // cols, cols, float(epsilon),
                          _dtype_code(input.dtype, "rms_norm_forward"), _stream()))


def gemv(weight: torch.Tensor, x: torch.Tensor, *, norm_weight: Optional[torch.Tensor] = None,
         eps: float = 1e-5, gated: bool = False, residual: Optional[torch.Tensor] = None,
         pair_gated: bool = False, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Extension for the batch-1 decode driver: ``y = weight @ f(x) (+ residual)`` in one launch.

    ``weight [rows, cols]`` (an ``nn.Linear`` weight, rows may be strided), ``x`` one token.
    ``norm_weight``: ``f(x) = RMSNorm(x, eps) * norm_weight``; ``gated``: ``x`` holds
    ``[gate | up]`` (2 cols) and ``f(x) = silu(gate) * up``; otherwise ``f(x) = x``.
    ``residual`` (may be ``out``) is added to the product.  ``pair_gated``: ``weight`` stacks the
    gate and the up projection and ``out[i] = silu(weight[i] . f(x)) * (weight[i + rows/2] . f(x))``
    (``rows/2`` values).  Returns ``out``."""
    _check_input(x, "x")
    if not weight.is_cuda or weight.dim() != 2 or weight.stride(1) != 1:
        raise RuntimeError("gemv: weight must be a CUDA matrix with contiguous rows")
    rows, cols = weight.shape
    if weight.dtype != x.dtype or x.numel() != (2 * cols if gated else cols):
        raise RuntimeError("gemv: x does not fit the weight")
    if norm_weight is not None and gated:
        raise RuntimeError("gemv: norm_weight and gated exclude each other")
    if norm_weight is not None:
        _check_input(norm_weight, "norm_weight")
        if norm_weight.numel() != cols or norm_weight.dtype != x.dtype:
            raise RuntimeError("gemv: norm_weight does not fit")
    n_out = rows // 2 if pair_gated else rows
    if pair_gated and (rows % 2 or gated or residual is not None):
        raise RuntimeError("gemv: pair_gated needs an even row count, no gated input, no residual")
    if out is None:
        out = torch.empty(n_out, dtype=x.dtype, device=x.device)
    _check_input(out, "out")
    if out.numel() != n_out or out.dtype != x.dtype:
        raise RuntimeError("gemv: out does not fit")
    if residual is not None:
        _check_input(residual, "residual")
        if residual.numel() != rows or residual.dtype != x.dtype:
            raise RuntimeError("gemv: residual does not fit")
    mode = 1 if norm_weight is not None else (2 if gated else 0)
    check(lib.td_gemv(weight.data_ptr(), weight.stride(0), rows, cols, x.data_ptr(), mode,
                      None if norm_weight is None else norm_weight.data_ptr(), float(eps),
                      None if residual is None else residual.data_ptr(), int(pair_gated),
                      out.data_ptr(), _dtype_code(x.dtype, "gemv"), _stream()))
    return out


def topk_filtering(estimated_value: torch.Tensor, estimated_indices: Optional[torch.Tensor],
                   d_out: Optional[torch.Tensor], indices_out: torch.Tensor,
                   buf: Optional[torch.Tensor], page_budget: int, *,
                   page_table: Optional[torch.Tensor] = None, page_size: int = 1,
                   lengths: Optional[torch.Tensor] = None,
                   upper_bound: Optional[torch.Tensor] = None) -> None:
    """bsk_ops.h:34-39 / topk.cu:7-44.  Row-wise top-``page_budget`` of ``estimated_value``
    ``[H, len]``; ``indices_out[h, j]`` is ``estimated_indices[h, p]`` of the selected position
    ``p``.  ``buf`` is scratch, as in the reference (there: RAFT's): a zero-initialised uint8 /
    any-dtype device tensor of at least ``topk_workspace_bytes(H)`` bytes through which the
    workgroups of a row of more than 65536 elements share the work; shorter rows never touch it,
    and without it (smaller or ``None``) every workgroup of a long row goes through the whole row.
    The call leaves ``buf`` zeroed where it must be for the next call.

    Deterministic where the reference is not: ties at the threshold go to the lower position
    and each output row is sorted by position.  If ``estimated_indices`` has fewer columns than
    ``estimated_value`` only those leading columns take part (the reference strides both by
    ``estimated_value.size(1)``, kernels/include/topk/decode_select_k.cuh:53-55).

    Extensions: ``estimated_indices=None`` returns positions, or physical token slots when a
    ``page_table`` ``[n_pages]`` is given (``[groups, n_pages]``: one table per ``H / groups``
    consecutive rows, the sequences of a batch); fp32 values.  ``lengths`` (int32 device
    ``[groups]``): rows of group g use only their first ``lengths[g]`` columns and select
    ``min(page_budget, lengths[g])`` of them, leaving the rest of their output row untouched.
    ``upper_bound`` (fp32 device ``[H]``): a value per row that no score of the row exceeds (a
    selection layer's log-sum-exp, the head count for summed probabilities); same result, without
    the pass that finds the row maximum.  NaN entries mean "no bound".
    """
    _check_rows(estimated_value, "estimated_value")
    rows, length = estimated_value.shape
    in_ptr, in_stride = None, 0
    if estimated_indices is not None:
        _check_input(estimated_indices, "estimated_indices")
        _check_dim(2, estimated_indices, "estimated_indices")
        _check_i32(estimated_indices, "estimated_indices")
        if estimated_indices.size(0) != rows:
            raise RuntimeError("estimated_value and estimated_indices differ in rows")
        length = min(length, estimated_indices.size(1))
        in_ptr, in_stride = estimated_indices.data_ptr(), estimated_indices.size(1)
    _check_rows(indices_out, "indices_out")
    _check_i32(indices_out, "indices_out")
    k = int(page_budget)
    if indices_out.dim() != 2 or indices_out.size(0) != rows or indices_out.size(1) != k:
        raise RuntimeError(f"indices_out must be [{rows}, {k}]")
    out_vals = None
    if d_out is not None and d_out.numel() > 0:
        _check_rows(d_out, "d_out")
        if d_out.shape != indices_out.shape or d_out.dtype != estimated_value.dtype or \
                d_out.stride(0) != indices_out.stride(0):
            raise RuntimeError("d_out must match indices_out in shape and estimated_value in dtype")
        out_vals = d_out.data_ptr()
    if k > length:
        raise RuntimeError(f"page_budget {k} exceeds the row length {length}")
    pt_ptr, pt_stride, rows_per_table = None, 0, 0
    if page_table is not None:
        _check_input(page_table, "page_table")
        _check_i32(page_table, "page_table")
        if page_table.dim() == 2:   # one table per group of consecutive rows (a batch of sequences)
            groups = page_table.size(0)
            if groups < 1 or rows % groups != 0:
                raise RuntimeError(f"page_table has {groups} tables for {rows} rows")
            pt_stride, rows_per_table = page_table.stride(0), rows // groups
        elif page_table.dim() != 1:
            raise RuntimeError("page_table must be [n_pages] or [groups, n_pages]")
        if page_table.size(-1) * page_size < length:
            raise RuntimeError("page_table does not cover the row")
        pt_ptr = page_table.data_ptr()
    len_ptr = None
    if lengths is not None:
        _check_input(lengths, "lengths")
        _check_i32(lengths, "lengths")
        groups = lengths.numel()
        if groups < 1 or rows % groups != 0 or (rows_per_table and rows_per_table != rows // groups):
            raise RuntimeError(f"lengths has {groups} entries for {rows} rows")
        rows_per_table = rows // groups
        len_ptr = lengths.data_ptr()
    ws_ptr, ws_bytes = None, 0
    if buf is not None and buf.is_cuda and buf.is_contiguous():
        ws_bytes = buf.numel() * buf.element_size()
        if ws_bytes >= topk_workspace_bytes(rows):
            ws_ptr = buf.data_ptr()
    bound_ptr = None
    if upper_bound is not None:
        _check_input(upper_bound, "upper_bound")
        if upper_bound.dtype != torch.float32 or upper_bound.numel() != rows:
            raise RuntimeError(f"upper_bound must hold {rows} float32 values")
        bound_ptr = upper_bound.data_ptr()
    check(lib.td_topk_bounded(estimated_value.data_ptr(),
                              _dtype_code(estimated_value.dtype, "Top-k filtering"),
                              estimated_value.stride(0), rows, length, k, in_ptr, in_stride,
                              pt_ptr, pt_stride, rows_per_table, len_ptr, int(page_size),
                              bound_ptr, out_vals, indices_out.data_ptr(), indices_out.stride(0),
                              ws_ptr, ws_bytes if ws_ptr else 0, _stream()))


def topk_workspace_bytes(rows: int) -> int:
    """Bytes of zero-initialised scratch ``topk_filtering`` wants in ``buf`` for `rows` rows."""
    return int(lib.td_topk_workspace_bytes(int(rows)))


def estimate_attn_score(q: torch.Tensor, o: torch.Tensor, metadata_data: torch.Tensor,
                        metadata_indices: torch.Tensor, metadata_indptr: Optional[torch.Tensor],
                        metadata_last_page_len: int, metadata_last_page_idx: int,
                        layout: int) -> None:
    """bsk_ops.h:41-48 / estimate.cu:6-88.  Page-level upper bound of the logits (the estimator
    TidalDecode inherited from Quest): ``o[h, e] = sum_d max(q*max_e, q*min_e)`` over the
    metadata entries of ``metadata_indices`` except the newest one; ``q [1, H, D]``,
    ``o [H, entries]``.  ``metadata_indptr`` and ``metadata_last_page_idx`` are accepted for
    signature parity (all pages of ``metadata_indices`` are used, the last one is its last)."""
    _check_input(q, "q")
    _check_dim(3, q, "q")
    _check_input(o, "o")
    _check_dim(2, o, "o")
    _check_input(metadata_indices, "metadata_indices")
    _check_i32(metadata_indices, "metadata_indices")
    pool = _pool(metadata_data, int(layout), "metadata_data")
    if q.size(0) != 1 or q.size(2) != pool.head_dim or q.dtype != metadata_data.dtype \
            or o.dtype != q.dtype or o.size(0) != q.size(1):
        raise RuntimeError("estimate_attn_score: q / o do not fit the metadata pool")
    n_pages = metadata_indices.numel()
    n_entries = (n_pages - 1) * pool.page_size + int(metadata_last_page_len) - 1
    if o.size(1) < n_entries:
        raise RuntimeError(f"estimate_attn_score: o holds {o.size(1)} entries, {n_entries} needed")
    check(lib.td_estimate_score(pool, metadata_indices.data_ptr(), n_pages,
                                int(metadata_last_page_len), q.data_ptr(), q.size(1),
                                o.data_ptr(), o.stride(0), _stream()))


def _append(k, v, kv_data, kv_indices, kv_indptr, kv_last_page_len, metadata_data,
            metadata_indices, metadata_indptr, metadata_last_page_len, layout, decode: bool):
    # checks of tidal/ops/csrc/page.cu:19-55
    for t, n in ((k, "k"), (v, "v"), (kv_indices, "kv_indices")):
        _check_input(t, n)
    _check_dim(3, k, "k")
    _check_dim(3, v, "v")
    _check_dim(1, kv_indices, "kv_indices")
    _check_i32(kv_indices, "kv_indices")
    _check_i32(kv_indptr, "kv_indptr")
    if decode and (k.size(0) != 1 or v.size(0) != 1):
        raise RuntimeError("append_kv_cache_decode expects k.size(0) == v.size(0) == 1")
    if k.shape != v.shape or k.dtype != v.dtype:
        raise RuntimeError("k and v must agree in shape and dtype")
    pool = _pool(kv_data, int(layout))
    if pool.num_kv_heads != k.size(1) or pool.head_dim != k.size(2) or kv_data.dtype != k.dtype:
        raise RuntimeError("kv_data does not match k in heads, head_dim or dtype")
    meta = None
    if metadata_data is not None and metadata_data.numel() > 0:
        meta = _pool(metadata_data, int(layout), "metadata_data")
        _check_input(metadata_indices, "metadata_indices")
        _check_dim(1, metadata_indices, "metadata_indices")
        _check_i32(metadata_indices, "metadata_indices")
        _check_i32(metadata_indptr, "metadata_indptr")
    check(lib.td_append_kv(pool, k.data_ptr(), v.data_ptr(), k.size(0), kv_indices.data_ptr(),
                           kv_indptr.data_ptr(), int(kv_last_page_len), meta,
                           _ptr(metadata_indices) if meta is not None else None,
                           _ptr(metadata_indptr) if meta is not None else None,
                           int(metadata_last_page_len) if meta is not None else 0, _stream()))


def append_kv_cache_prefill(k, v, kv_data, kv_indices, kv_indptr, kv_last_page_len,
                            kv_last_page_idx, metadata_data, metadata_indices, metadata_indptr,
                            metadata_last_page_len, metadata_last_page_idx, layout) -> None:
    """bsk_ops.h:50-63 / page.cu:101-210.  Appends ``k.size(0)`` tokens."""
    _append(k, v, kv_data, kv_indices, kv_indptr, kv_last_page_len, metadata_data,
            metadata_indices, metadata_indptr, metadata_last_page_len, layout, decode=False)


def append_kv_cache_decode(k, v, kv_data, kv_indices, kv_indptr, kv_last_page_len,
                           kv_last_page_idx, metadata_data, metadata_indices, metadata_indptr,
                           metadata_last_page_len, metadata_last_page_idx, layout) -> None:
    """bsk_ops.h:65-78 / page.cu:6-99.  Appends the single new token."""
    _append(k, v, kv_data, kv_indices, kv_indptr, kv_last_page_len, metadata_data,
            metadata_indices, metadata_indptr, metadata_last_page_len, layout, decode=True)


def rope_append_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, kv_data: torch.Tensor,
                       positions: torch.Tensor, dst_slot: torch.Tensor, layout: int,
                       rope_scale: float = 1.0, rope_theta: float = 1e4) -> None:
    """Extension: ``apply_rope_in_place`` + ``append_kv_cache_decode`` in one launch for a batch.
    q ``[B, H_q, D]`` is rotated in place; rotated k and v ``[B, H_kv, D]`` go to physical slot
    ``dst_slot[b]``; ``positions[b]`` is the token's position."""
    for t, n in ((q, "q"), (k, "k"), (v, "v"), (positions, "positions"), (dst_slot, "dst_slot")):
        _check_input(t, n)
    _check_dim(3, q, "q")
    _check_dim(3, k, "k")
    _check_i32(positions, "positions")
    _check_i32(dst_slot, "dst_slot")
    pool = _pool(kv_data, int(layout))
    b = q.size(0)
    if k.shape != v.shape or k.size(0) != b or k.size(1) != pool.num_kv_heads or \
            q.size(2) != pool.head_dim or k.size(2) != pool.head_dim or \
            not (q.dtype == k.dtype == v.dtype == kv_data.dtype):
        raise RuntimeError("rope_append_decode: q/k/v/kv_data disagree in shape or dtype")
    if positions.numel() != b or dst_slot.numel() != b:
        raise RuntimeError("rope_append_decode: positions and dst_slot must hold one entry per sequence")
    check(lib.td_rope_append_decode(pool, q.data_ptr(), k.data_ptr(), v.data_ptr(), b, q.size(1),
                                    positions.data_ptr(), dst_slot.data_ptr(), float(rope_scale),
                                    float(rope_theta), _stream()))


def merge_states(o_parts: torch.Tensor, lse_parts: torch.Tensor,
                 want_lse: bool = True) -> Tuple[torch.Tensor, Optional[torch.Tensor]]:
    """Extension: merge attention states computed over disjoint token subsets.  ``o_parts``
    ``[n_parts, ..., D]`` (fp16 / bf16 / fp32) and ``lse_parts`` ``[n_parts, ...]`` float32, as
    ``forward(..., lse=)`` produces them; returns ``(o [..., D], lse [...])``."""
    _check_input(o_parts, "o_parts")
    _check_input(lse_parts, "lse_parts")
    if lse_parts.dtype != torch.float32 or o_parts.dim() < 2 or \
            tuple(lse_parts.shape) != tuple(o_parts.shape[:-1]):
        raise RuntimeError("lse_parts must be float32 with the shape of o_parts minus its last axis")
    n_parts, d = o_parts.size(0), o_parts.size(-1)
    rows = lse_parts.numel() // n_parts
    o = torch.empty(o_parts.shape[1:], dtype=o_parts.dtype, device=o_parts.device)
    lse = torch.empty(lse_parts.shape[1:], dtype=torch.float32, device=o_parts.device) \
        if want_lse else None
    check(lib.td_merge_states(o_parts.data_ptr(), _dtype_code(o_parts.dtype, "merge_states"),
                              lse_parts.data_ptr(), n_parts, rows, d, o.data_ptr(),
                              None if lse is None else lse.data_ptr(), _stream()))
    return o, lse


def argmax(x: torch.Tensor, out: torch.Tensor) -> None:
    """Extension: ``out[0]`` (int64, device) = index of the largest element of the 1-D ``x``
    (NaN ranks highest, ties to the lower index).  One launch without scratch: graph-safe."""
    _check_input(x, "x")
    _check_input(out, "out")
    if out.dtype != torch.int64 or out.numel() < 1:
        raise RuntimeError("out must be an int64 tensor")
    check(lib.td_argmax(x.data_ptr(), _dtype_code(x.dtype, "argmax"), x.numel(), out.data_ptr(),
                        _stream()))


def step_advance(state: torch.Tensor, page_table: torch.Tensor, page_size: int, budget: int,
                 token: Optional[torch.Tensor] = None,
                 tokens_out: Optional[torch.Tensor] = None) -> None:
    """Extension: the sequence described by ``state`` (int32 device ``[TD_STEP_WORDS]``, see
    ``_lib.TD_STEP_*``) grows by one token; its words are recomputed on the device from the
    sequence's ``page_table`` (int32 ``[n_pages]``, pages reserved ahead).  ``token`` (int64
    ``[1]``) is recorded at ``tokens_out[steps taken]`` first.  Safe inside a captured graph."""
    _check_input(state, "state")
    _check_input(page_table, "page_table")
    _check_i32(state, "state")
    _check_i32(page_table, "page_table")
    if state.numel() < _lib.TD_STEP_WORDS:
        raise RuntimeError(f"state must hold {_lib.TD_STEP_WORDS} int32 words")
    tok_ptr = out_ptr = None
    cap = 0
    if token is not None or tokens_out is not None:
        if token is None or tokens_out is None:
            raise RuntimeError("token and tokens_out go together")
        _check_input(token, "token")
        _check_input(tokens_out, "tokens_out")
        if token.dtype != torch.int64 or tokens_out.dtype != torch.int64 or token.numel() < 1:
            raise RuntimeError("token and tokens_out must be int64")
        tok_ptr, out_ptr, cap = token.data_ptr(), tokens_out.data_ptr(), tokens_out.numel()
    check(lib.td_step_advance(state.data_ptr(), page_table.data_ptr(), page_table.numel(),
                              int(page_size), int(budget), tok_ptr, out_ptr, cap, _stream()))


def step_advance_batch(state: torch.Tensor, batch: int, page_table: torch.Tensor, page_size: int,
                       budget: int) -> None:
    """Extension: ``step_advance`` for ``batch`` sequences in lock step.  ``state`` is int32
    ``[TD_STEP_WORDS, stride]`` (word w of sequence b at ``state[w, b]``), ``page_table`` int32
    ``[>= batch, pages_per_seq]`` with the pages of sequence b in row b."""
    _check_input(state, "state")
    _check_input(page_table, "page_table")
    _check_i32(state, "state")
    _check_i32(page_table, "page_table")
    _check_dim(2, state, "state")
    _check_dim(2, page_table, "page_table")
    if state.size(0) < _lib.TD_STEP_WORDS or page_table.size(0) < batch:
        raise RuntimeError("state must be [TD_STEP_WORDS, stride], page_table [batch, pages]")
    check(lib.td_step_advance_batch(state.data_ptr(), state.size(1), int(batch),
                                    page_table.data_ptr(), page_table.size(1), int(page_size),
                                    int(budget), _stream()))


def rope_table(positions: torch.Tensor, head_dim: int, rope_scale: float = 1.0,
               rope_theta: float = 1e4, cos: Optional[torch.Tensor] = None,
               sin: Optional[torch.Tensor] = None):
    """Extension: cos / sin ``[B, D/2]`` float32 of the rotary angles of ``positions`` ``[B]``
    (int32); one call per decode step feeds every layer's fused ``forward(..., fresh=...)``."""
    _check_input(positions, "positions")
    _check_i32(positions, "positions")
    b = positions.numel()
    if cos is None:
        cos = torch.empty((b, head_dim // 2), dtype=torch.float32, device=positions.device)
    if sin is None:
        sin = torch.empty((b, head_dim // 2), dtype=torch.float32, device=positions.device)
    check(lib.td_rope_table(positions.data_ptr(), b, int(head_dim), float(rope_scale),
                            float(rope_theta), cos.data_ptr(), sin.data_ptr(), _stream()))
    return cos, sin


def prefill_with_paged_kv_cache(q, kv_data, kv_indices, kv_last_page_len, causal, layout,
                                allow_fp16_qk_reduction, rope_scale, rope_theta) -> torch.Tensor:
    """bsk_ops.h:80-88 / batch_prefill.cu:27-117.  Attention of the ``q.size(0)`` newest tokens
    over the paged cache (their K/V already appended), causal or not, on the matrix cores
    (``td_prefill_attn``; head_dim 64, 128 or 256).  ``allow_fp16_qk_reduction``, ``rope_scale``
    and ``rope_theta`` are accepted for signature parity: RoPE is applied before the cache is
    written (RotaryMode::kNone in the reference's call, batch_prefill.cu:95)."""
    _check_input(q, "q")
    _check_dim(3, q, "q")
    _check_input(kv_indices, "kv_indices")
    _check_i32(kv_indices, "kv_indices")
    pool = _pool(kv_data, int(layout))
    n_pages = kv_indices.numel()
    kv_len = (n_pages - 1) * pool.page_size + int(kv_last_page_len)
    if q.size(2) != pool.head_dim or q.dtype != kv_data.dtype:
        raise RuntimeError("prefill_with_paged_kv_cache: q does not fit the cache")
    o = torch.empty_like(q)
    check(lib.td_prefill_attn(pool, kv_indices.data_ptr(), n_pages, kv_len, q.data_ptr(),
                              o.data_ptr(), q.size(0), q.size(1),
                              1.0 / math.sqrt(pool.head_dim), int(bool(causal)), _stream()))
    return o


# ------------------------------------------------------------------------------------------
# decode attention handler
# ------------------------------------------------------------------------------------------
class BatchDecodeWithPagedKVCachePyTorchWrapper:
    """bsk_ops.h:90-118 / approx_attn.cu:27-151.  ``begin_forward`` fixes the head geometry,
    ``forward`` may then be called for any number of layers, ``end_forward`` closes the
    bracket.  The split plan is recomputed (host arithmetic only) whenever the list shape
    changes; the scratch buffer grows on demand and is kept between brackets."""

    def __init__(self, layout: int):
        if layout not in (TD_NHD, TD_HND):
            raise RuntimeError(f"Invalid layout {layout}")
        self._layout = int(layout)
        self._begun = False
        self._geom = None
        self._plans = {}
        self._workspace = None
        self.waves_per_block = 0  # 0 = library default; tuning knob
        self.fused_merge = -1     # -1 = library default
        self.chunk_tokens = 0     # 0 = library default
        self.tile_rows = 0        # 0 = library default
        self.sparse_waves = 0     # short-list kernel: 0 = library default, -1 = never
        self.sparse_rows = 0
        # True: forward() goes through td_decode_attn_noalloc (scratch inside the library image,
        # no workspace tensor) -- for callers that must not allocate
        self.static_scratch = False

    def begin_forward(self, indptr: torch.Tensor, num_qo_heads: int, num_kv_heads: int,
                      head_dim: int, page_size: int, empty_data: torch.Tensor) -> None:
        if indptr is not None:
            _check_dim(1, indptr, "indptr")
            _check_i32(indptr, "indptr")
        _dtype_code(empty_data.dtype, "BatchDecodeWithPagedKVCache")
        if empty_data.dtype == torch.float32:
            raise RuntimeError("BatchDecodeWithPagedKVCache failed to dispatch with dtype "
                               f"{empty_data.dtype}")
        if num_qo_heads % num_kv_heads != 0:
            raise RuntimeError(f"num_qo_heads {num_qo_heads} is not a multiple of num_kv_heads "
                               f"{num_kv_heads}")
        self._geom = (int(num_qo_heads), int(num_kv_heads), int(head_dim), int(page_size),
                      empty_data.dtype)
        self._plans.clear()
        self._begun = True

    def end_forward(self) -> None:
        self._begun = False
        self._plans.clear()

    def _plan(self, batch: int, idx_rows: int, max_items: int, short_list: bool = True) -> DecodePlan:
        """``short_list``: the call has token-slot lists and no score output, the two things the
        planner cannot see that the short-list kernel needs; other calls get a plan shaped for
        the streaming kernel."""
        sparse_waves = self.sparse_waves if short_list else -1
        key = (batch, idx_rows, max_items, self.waves_per_block, self.fused_merge,
               self.chunk_tokens, self.tile_rows, sparse_waves, self.sparse_rows)
        plan = self._plans.get(key)
        if plan is None:
            hq, hkv, d, _, _ = self._geom
            plan = DecodePlan(self.chunk_tokens, 0, self.waves_per_block, self.tile_rows,
                              self.fused_merge, sparse_waves, self.sparse_rows, 0)
            check(lib.td_decode_make_plan(batch, hq, hkv, d, idx_rows, max_items, plan))
            self._plans[key] = plan
        return plan

    def forward(self, q: torch.Tensor, o: torch.Tensor, paged_kv_data: torch.Tensor,
                paged_kv_indices: torch.Tensor, paged_kv_indptr: Optional[torch.Tensor],
                paged_kv_last_page_len, paged_kv_last_page_idx,
                qk_product: Optional[torch.Tensor], rope_scale: float = 1.0,
                rope_theta: float = 1e4, *, index_kind: str = "pages",
                lse: Optional[torch.Tensor] = None, n_list: Optional[int] = None,
                fresh=None, counts: Optional[torch.Tensor] = None) -> None:
        """q, o ``[B, H_q, D]``; ``paged_kv_indices`` ``[rows, budget]`` int32 with rows in
        {H_q, H_kv, 1}; sequence b uses columns ``indptr[b]:indptr[b+1]`` of every row and then
        the first ``last_page_len`` entries of page ``last_page_idx`` (ints, or int32 device
        tensors ``[B]``).  ``index_kind="slots"`` reads the entries as token slots.
        ``n_list`` bounds the per-sequence column count (default: all columns).
        ``counts`` (int32 device ``[B]``): sequence b uses ``counts[b]`` columns from
        ``indptr[b]`` on — segments of a padded table instead of a packed one.
        rope_scale / rope_theta are accepted for signature parity; RoPE is applied before the
        cache is written (RotaryMode::kNone in the reference, approx_attn.cu:52,139).
        ``fresh=(k, v, cos, sin, dst_slot)`` fuses the decode step: q, k ``[B, H, D]`` are then
        UN-rotated, cos/sin ``[B, D/2]`` float32 come from ``rope_table``; the kernel rotates q
        in registers, writes rotated k and v to ``dst_slot`` and attends to them from registers
        (power-of-two pages and pools below 4 GiB only)."""
        if not self._begun:
            raise RuntimeError("Please call BatchDecodeHandler's BeginForward() before calling "
                               "BatchDecodeWithPagedKVCacheWrapper()")
        _check_input(q, "q")
        _check_input(o, "o")
        _check_rows(paged_kv_indices, "paged_kv_indices")
        _check_dim(3, q, "q")
        _check_i32(paged_kv_indices, "paged_kv_indices")
        pool = _pool(paged_kv_data, self._layout, "paged_kv_data")
        hq, hkv, d, page, dtype = self._geom
        batch = q.size(0)
        if q.size(1) != hq or q.size(2) != d or pool.num_kv_heads != hkv or pool.head_dim != d \
                or pool.page_size != page:
            raise RuntimeError("forward: q / paged_kv_data do not match begin_forward's geometry")
        if q.dtype != dtype or paged_kv_data.dtype != dtype or o.dtype != dtype:
            raise RuntimeError(f"BatchDecodeWithPagedKVCache failed to dispatch with dtype {q.dtype}")
        if o.shape != q.shape:
            raise RuntimeError("o must have the shape of q")
        rows, budget = paged_kv_indices.shape
        if rows not in (1, hkv, hq):
            raise RuntimeError(f"paged_kv_indices.size(0) must be 1, {hkv} or {hq}")
        if index_kind not in ("pages", "slots"):
            raise KeyError(f"Invalid index_kind {index_kind}")
        kind = TD_IDX_PAGES if index_kind == "pages" else TD_IDX_SLOTS

        lst = IndexList()
        lst.idx = _ptr(paged_kv_indices)
        lst.idx_rows = rows
        # what a row holds bounds the kernels' reads; a single row has no meaningful stride
        lst.idx_row_stride = paged_kv_indices.stride(0) if rows > 1 else budget
        lst.kind = kind
        if paged_kv_indptr is not None:
            _check_i32(paged_kv_indptr, "paged_kv_indptr")
            if paged_kv_indptr.numel() != batch + 1:
                raise RuntimeError("paged_kv_indptr must hold batch + 1 entries")
            lst.indptr = paged_kv_indptr.data_ptr()
        if counts is not None:
            _check_i32(counts, "counts")
            if paged_kv_indptr is None or counts.numel() != batch:
                raise RuntimeError("counts needs paged_kv_indptr and one entry per sequence")
            lst.count_arr = counts.data_ptr()
        lst.n_list_host = budget if n_list is None else min(int(n_list), budget)
        max_last = 0
        if isinstance(paged_kv_last_page_len, torch.Tensor):
            _check_i32(paged_kv_last_page_len, "paged_kv_last_page_len")
            lst.last_page_len_arr = paged_kv_last_page_len.data_ptr()
            max_last = page
        else:
            lst.last_page_len = int(paged_kv_last_page_len)
            max_last = lst.last_page_len
        if isinstance(paged_kv_last_page_idx, torch.Tensor):
            _check_i32(paged_kv_last_page_idx, "paged_kv_last_page_idx")
            lst.last_page_idx_arr = paged_kv_last_page_idx.data_ptr()
        else:
            lst.last_page_idx = int(paged_kv_last_page_idx)

        max_items = lst.n_list_host * (page if kind == TD_IDX_PAGES else 1) + max_last
        has_scores = qk_product is not None and qk_product.numel() > 0
        plan = self._plan(batch, rows, max_items, kind == TD_IDX_SLOTS and not has_scores)
        if not self.static_scratch and plan.workspace_bytes > 0 and (self._workspace is None or
                                         self._workspace.numel() < plan.workspace_bytes or
                                         self._workspace.device != q.device):
            self._workspace = torch.zeros(int(plan.workspace_bytes), dtype=torch.uint8,
                                          device=q.device)

        scores_ptr, scores_dtype, score_stride = None, TD_F32, 0
        if qk_product is not None and qk_product.numel() > 0:
            _check_input(qk_product, "qk_product")
            if qk_product.numel() % (batch * hq) != 0:
                raise RuntimeError("qk_product must be [B * H_q, stride]")
            score_stride = qk_product.numel() // (batch * hq)
            if score_stride < max_items:
                raise RuntimeError(f"qk_product rows hold {score_stride} entries, the list has "
                                   f"up to {max_items}")
            scores_ptr = qk_product.data_ptr()
            scores_dtype = _dtype_code(qk_product.dtype, "qk_product")
        lse_ptr = None
        if lse is not None:
            _check_input(lse, "lse")
            if lse.dtype != torch.float32 or lse.numel() != batch * hq:
                raise RuntimeError("lse must be float32 [B, H_q]")
            lse_ptr = lse.data_ptr()
        fresh_arg = None
        if fresh is not None:
            fk, fv, fcos, fsin, fslot = fresh
            for t, n in ((fk, "fresh k"), (fv, "fresh v"), (fcos, "fresh cos"), (fsin, "fresh sin"),
                         (fslot, "fresh dst_slot")):
                _check_input(t, n)
            if fk.shape != (batch, hkv, d) or fv.shape != fk.shape or fk.dtype != dtype or \
                    fv.dtype != dtype:
                raise RuntimeError("fresh k / v must be [B, H_kv, D] in the cache dtype")
            if fcos.dtype != torch.float32 or fsin.dtype != torch.float32 or \
                    fcos.numel() != batch * d // 2 or fsin.numel() != batch * d // 2:
                raise RuntimeError("fresh cos / sin must be float32 [B, D/2]")
            _check_i32(fslot, "fresh dst_slot")
            if fslot.numel() != batch:
                raise RuntimeError("fresh dst_slot must hold one entry per sequence")
            fresh_arg = FreshToken(fk.data_ptr(), fv.data_ptr(), fcos.data_ptr(), fsin.data_ptr(),
                                   fslot.data_ptr())
        if self.static_scratch:
            check(lib.td_decode_attn_noalloc(pool, lst, plan, q.data_ptr(), o.data_ptr(), batch, hq,
                                             1.0 / math.sqrt(d), scores_ptr, scores_dtype,
                                             score_stride, lse_ptr, fresh_arg, _stream()))
            return
        ws = self._workspace
        check(lib.td_decode_attn(pool, lst, plan, q.data_ptr(), o.data_ptr(), batch, hq,
                                 1.0 / math.sqrt(d), scores_ptr, scores_dtype, score_stride,
                                 lse_ptr, fresh_arg, ws.data_ptr() if ws is not None else None,
                                 ws.numel() if ws is not None else 0, _stream()))


def last_decode_kernel() -> str:
    """Kernel family that served this thread's last decode-attention call ("short-list",
    "streaming", each possibly with ", 64-bit offsets")."""
    return lib.td_last_decode_kernel().decode()


def gather_probe(wrapper: "BatchDecodeWithPagedKVCachePyTorchWrapper", paged_kv_data: torch.Tensor,
                 slots: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Measurement aid: only the memory side of ``wrapper.forward(..., slots, index_kind="slots")``
    (same grid, same list -> K/V row loads, no arithmetic, no merge).  Returns the word-per-wave
    output tensor, which is of no use except that it keeps the loads alive."""
    _check_rows(slots, "slots")
    _check_i32(slots, "slots")
    pool = _pool(paged_kv_data, wrapper._layout, "paged_kv_data")
    hq, hkv, d, page, dtype = wrapper._geom
    rows, budget = slots.shape
    lst = IndexList()
    lst.idx = _ptr(slots)
    lst.idx_rows = rows
    lst.idx_row_stride = slots.stride(0) if slots.size(0) > 1 else slots.size(1)
    lst.kind = TD_IDX_SLOTS
    lst.n_list_host = budget
    plan = wrapper._plan(1, rows, budget)
    words = hq * int(plan.max_splits) * int(plan.waves_per_block)
    if out is None:
        out = torch.empty(words, dtype=torch.int32, device=slots.device)
    check(lib.td_gather_probe(pool, lst, plan, 1, hq, out.data_ptr(), out.numel() * 4, _stream()))
    return out


def score_reduce(logits: torch.Tensor, lse: torch.Tensor, num_kv_heads: int, n: int,
                 mode: str = "head_sum", out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Extension: sum of softmax probabilities over query heads.  logits float32 ``[H_q, stride]``,
    lse float32 ``[H_q]``; returns float32 ``[1, n]`` (``head_sum``) or ``[H_kv, n]``
    (``group_sum``)."""
    _check_input(logits, "logits")
    _check_input(lse, "lse")
    _check_dim(2, logits, "logits")
    if logits.dtype != torch.float32 or lse.dtype != torch.float32:
        raise RuntimeError("score_reduce expects float32 logits and lse")
    hq = logits.size(0)
    if lse.numel() != hq:
        raise RuntimeError("lse must hold one entry per query head")
    if mode not in ("head_sum", "group_sum"):
        raise KeyError(f"Invalid score reduce mode {mode}")
    rows = 1 if mode == "head_sum" else int(num_kv_heads)
    if out is None:
        out = torch.empty((rows, n), dtype=torch.float32, device=logits.device)
    check(lib.td_score_reduce(logits.data_ptr(), logits.stride(0), lse.data_ptr(), hq,
                              int(num_kv_heads), int(n),
                              _lib.TD_REDUCE_HEAD_SUM if mode == "head_sum"
                              else _lib.TD_REDUCE_GROUP_SUM,
                              out.data_ptr(), out.stride(0), _stream()))
    return out

"""GPU parity at the full sizes of the benchmark configurations: one selection layer, the top-k
selection and one sparse layer through the operator surface, against the CPU oracle.

  cfg1  Llama-2-7B shape: 32/32 heads x 128, bf16, page 16, 32768 (+1) tokens, top_k 2048
  cfg2  GQA 32/8, 102400 tokens, top_k 4096
  cfg4  40/40 heads, 10240 / 32768 / 102400 tokens, top_k 2048

The oracle's sparse layer gathers the selected rows (equal to the reference's masked dense form,
pinned in tests/test_oracle.py), so it finishes in seconds at these sizes.  Index sets are
compared bit-exact from the scores the GPU wrote; attention within 2e-3 (fp16) / 1e-2 (bf16).
The sparse layer runs twice: as a plain attention launch, and as the fused decode step the
benchmark times (RoPE of q and the new key, cache write and attention in one launch) against the
oracle on float64-rotated, storage-rounded q and K.  Size-independent properties on top: a
permuted list gives the same output, and a list naming every token equals full attention.
"""
import pytest
import torch

from _util import ATOL, PagedCase, randn, rotated, tolerance_report, within_ulps

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name,hq,hkv,n,k,mode,dtype", [
    ("cfg1", 32, 32, 32769, 2048, "per_head", torch.bfloat16),
    ("cfg1-head-sum", 32, 32, 32769, 2048, "head_sum", torch.bfloat16),
    ("cfg2", 32, 8, 102400, 4096, "per_head", torch.bfloat16),
    ("cfg2-group", 32, 8, 102400, 4096, "group_sum", torch.float16),
    ("cfg4", 40, 40, 32768, 2048, "per_head", torch.float16),
    ("cfg4-10k", 40, 40, 10240, 2048, "per_head", torch.bfloat16),
    ("cfg4-100k", 40, 40, 102400, 2048, "per_head", torch.bfloat16),
])
def test_selection_topk_sparse_at_full_size(cuda, name, hq, hkv, n, k, mode, dtype):
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    d, page = 128, 16
    case = PagedCase(n, hkv, d, page, dtype, seed=len(name) + n)
    q_sel, q_sp = randn((hq, d), 5, dtype), randn((hq, d), 6, dtype)
    pool = case.pool.to(cuda)
    table = case.page_table.to(torch.int32).to(cuda)

    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    stride = case.n_pages * page
    scores = torch.zeros((hq, stride), dtype=torch.float32, device=cuda)
    lse = torch.zeros((1, hq), dtype=torch.float32, device=cuda)
    o_sel = torch.empty((1, hq, d), dtype=dtype, device=cuda)
    w.forward(q_sel.to(dtype).to(cuda)[None], o_sel, pool, table[:-1][None].contiguous(), None,
              case.last_page_len, int(table[-1]), scores, lse=lse)
    rows = {"per_head": hq, "group_sum": hkv, "head_sum": 1}[mode]
    sel_scores = scores if mode == "per_head" else _kernels.score_reduce(scores, lse.view(-1), hkv, n, mode)
    scratch = torch.zeros(_kernels.topk_workspace_bytes(rows), dtype=torch.uint8, device=cuda)
    slots = torch.empty((rows, k), dtype=torch.int32, device=cuda)
    pos = torch.empty((rows, k), dtype=torch.int32, device=cuda)
    _kernels.topk_filtering(sel_scores[:, :n], None, None, slots, scratch, k, page_table=table,
                            page_size=page)
    _kernels.topk_filtering(sel_scores[:, :n], None, None, pos, scratch, k)  # scratch left clean
    o_sp = torch.empty((1, hq, d), dtype=dtype, device=cuda)
    w.forward(q_sp.to(dtype).to(cuda)[None], o_sp, pool, slots, None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()

    # selection layer: output and logits
    logits = orc.attn_logits(q_sel, case.k)
    assert tolerance_report(o_sel[0], orc.softmax_pv(logits, case.v)) <= ATOL[dtype]
    if mode == "per_head":
        assert (scores[:, :n].cpu() - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item())
    # top-k: bit-exact from the same scores; slots are the positions seen through the page table
    pos_c = pos.cpu().long()
    assert torch.equal(pos_c, orc.stable_topk(sel_scores[:, :n].cpu(), k))
    assert torch.equal(slots.cpu().long(), case.slots_of(pos_c))
    # sparse layer
    want = orc.sparse_layer_gather(q_sp, case.k, case.v, pos_c)
    assert tolerance_report(o_sp[0], want) <= ATOL[dtype]

    # The decode step as the benchmark times it: RoPE of q and of the new key, the cache write and
    # the attention in ONE launch (fresh=...).  The newest token plays the token being decoded: its
    # slot is in the lists of the even rows (taken from registers there) and in none of the odd ones.
    theta = 5e5 if hkv != hq else 1e4
    new_pos = n - 1
    pos_f = pos_c.clone()
    for r in range(rows):
        hit = (pos_f[r] == new_pos).nonzero().flatten()
        if r % 2 == 0 and hit.numel() == 0:
            pos_f[r, -1] = new_pos                       # lists stay sorted: it is the last position
        elif r % 2 == 1 and hit.numel():
            listed = set(pos_f[r].tolist())
            unused = next(x for x in range(n - 1) if x not in listed)
            pos_f[r, hit[0]] = unused
    k_new, v_new = randn((1, hkv, d), 21, dtype), randn((1, hkv, d), 22, dtype)
    k_f, v_f = case.k.clone(), case.v.clone()
    k_f[new_pos] = rotated(k_new, [new_pos], dtype, theta)[0]
    v_f[new_pos] = v_new[0]
    want_f = orc.sparse_layer_gather(rotated(q_sp[None], [new_pos], dtype, theta)[0], k_f, v_f, pos_f)
    assert w._plan(1, rows, k).sparse_waves > 0          # the short-list kernel, as in the benchmark
    pool_f = pool.clone()
    dst = case.slots_of(torch.tensor([new_pos])).to(torch.int32).to(cuda)
    cos, sin = _kernels.rope_table(torch.tensor([new_pos], dtype=torch.int32, device=cuda), d, 1.0, theta)
    o_f = torch.empty((1, hq, d), dtype=dtype, device=cuda)
    w.forward(q_sp.to(dtype).to(cuda)[None], o_f, pool_f, case.slots_of(pos_f).to(torch.int32).to(cuda),
              None, 0, 0, None, index_kind="slots",
              fresh=(k_new.to(dtype).to(cuda), v_new.to(dtype).to(cuda), cos, sin, dst))
    torch.cuda.synchronize()
    assert tolerance_report(o_f[0], want_f) <= ATOL[dtype]
    page_f, entry_f = int(dst[0]) // page, int(dst[0]) % page
    assert within_ulps(pool_f[page_f, 0, entry_f], k_f[new_pos], dtype)     # rotated key, one rounding
    assert torch.equal(pool_f[page_f, 1, entry_f].cpu(), v_new[0].to(dtype))
    pool_f[page_f, :, entry_f] = pool[page_f, :, entry_f]
    assert torch.equal(pool_f, pool)                                        # nothing else was written
    del pool_f

    # a permuted list names the same set: same output up to the summation order
    g = torch.Generator().manual_seed(1)
    perm = torch.stack([torch.randperm(k, generator=g) for _ in range(rows)]).to(cuda)
    o_perm = torch.empty_like(o_sp)
    w.forward(q_sp.to(dtype).to(cuda)[None], o_perm, pool, torch.gather(slots, 1, perm).contiguous(),
              None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()
    assert tolerance_report(o_perm[0], want) <= ATOL[dtype]
    assert tolerance_report(o_perm[0], o_sp[0]) <= ATOL[dtype] / 2


def test_list_of_every_token_equals_full_attention(cuda):
    """k = N at the benchmark length: the sparse path over all 32768 slots (shared list) equals
    the selection-layer path over the page table."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    hq, hkv, d, page, n, dtype = 32, 32, 128, 16, 32768, torch.bfloat16
    case = PagedCase(n, hkv, d, page, dtype, seed=9)
    q = randn((hq, d), 8, dtype)
    pool = case.pool.to(cuda)
    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    qd = q.to(dtype).to(cuda)[None]
    o_full, o_all = torch.empty_like(qd), torch.empty_like(qd)
    table = case.page_table.to(torch.int32).to(cuda)
    w.forward(qd, o_full, pool, table[:-1][None].contiguous(), None, case.last_page_len,
              int(table[-1]), None)
    slots = case.slots_of(torch.arange(n))[None].to(torch.int32).to(cuda)
    w.forward(qd, o_all, pool, slots, None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()
    want = orc.softmax_pv(orc.attn_logits(q, case.k), case.v)
    assert tolerance_report(o_full[0], want) <= ATOL[dtype]
    assert tolerance_report(o_all[0], want) <= ATOL[dtype]


def test_ragged_batch_of_eight_at_full_size(cuda):
    """cfg3: 8 sequences of randint(8192, 65537) tokens (seed 0), fp16, 32 heads x 128, page 16,
    1024 tokens selected per sequence and head — one launch for the batch per piece (selection layer
    with logits, top-k of all 256 rows, sparse layer) through BatchInferenceController.  The pool
    (8.6 GB) is filled on the device; the oracle checks the shortest and the longest sequence from
    their own pages, and every sequence through properties that do not need its K/V on the host:
    lists sorted by position, duplicate-free, inside the sequence, and equal to the oracle's
    selection from the logits the GPU wrote."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd.utils import BatchInferenceController

    dtype, h, d, page, k = torch.float16, 32, 128, 16, 1024
    lens = torch.randint(8192, 65537, (8,), generator=torch.Generator().manual_seed(0)).tolist()
    ctl = BatchInferenceController(1, h, d, page, k, max(lens) + 64, 8, dtype, cuda, page_order_seed=0)
    ctl.add_sequences(lens)
    ctl.pool.buf.normal_()
    ctl.begin_step()
    q = randn((8, h, d), 3, dtype)
    qd = q.to(dtype).to(cuda)
    o_full = ctl.attend_full(qd, 0, True)
    ctl.select()
    o_sparse = ctl.attend_sparse(qd, 0)
    torch.cuda.synchronize()
    order = sorted(range(8), key=lambda b: ctl.seq_lens[b])
    for b in range(8):
        n = ctl.seq_lens[b]
        table = torch.tensor(ctl._pages[b])
        logits_gpu = ctl.qk_product[b * h: (b + 1) * h, :n].cpu()
        slots = ctl.topk_dindices_buffer[:, b * k: (b + 1) * k].cpu().long()
        inv = torch.full((int(table.max()) + 1,), -1, dtype=torch.long)
        inv[table] = torch.arange(table.numel())
        pos = inv[slots // page] * page + slots % page
        assert (inv[slots // page] >= 0).all() and (pos < n).all(), b
        assert (pos[:, 1:] > pos[:, :-1]).all(), b                     # sorted, no duplicates
        assert torch.equal(pos, orc.stable_topk(logits_gpu, k)), b
        assert torch.isinf(ctl.qk_product[b * h: (b + 1) * h, n:]).all(), b
        if b in (order[0], order[-1]):
            pages = ctl.buf_layer(0)[table.to(cuda)]                   # [pages, 2, P, H, D]
            kk = pages[:, 0].reshape(-1, h, d)[:n].float().cpu()
            vv = pages[:, 1].reshape(-1, h, d)[:n].float().cpu()
            logits = orc.attn_logits(q[b], kk)
            assert (logits_gpu - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item()), b
            assert tolerance_report(o_full[b], orc.softmax_pv(logits, vv)) <= ATOL[dtype], b
            assert tolerance_report(o_sparse[b], orc.sparse_layer_gather(q[b], kk, vv, pos)) <= ATOL[dtype], b
    ctl.release()

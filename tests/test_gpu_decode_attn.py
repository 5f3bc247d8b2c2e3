"""GPU parity: decode attention through the C ABI (td_decode_attn) against the CPU oracle.

Tolerance: max-abs 2e-3 for fp16 and 1e-2 for bf16 against the fp32 oracle evaluated on the same,
identically rounded inputs.  The parameter grid follows the reference's own decode test
(kernels/src/test/test_batch_decode.cu:215-267: sequence lengths, page sizes, page budgets, head
dims; per-head page lists drawn from a shuffled iota with the forced last page, :57-76).
"""

import numpy as np
import pytest
import torch

from _util import ATOL, PagedCase, randn, tolerance_report

pytestmark = pytest.mark.gpu


def _wrapper(layout, hq, hkv, d, page, dtype, **knobs):
    from tidaldecode_amd import _kernels

    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(layout)
    for key, val in knobs.items():
        setattr(w, key, val)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    return w


def _oracle_paged(q, case, lists, last_idx, last_len, kind):
    from oracle import tidal_oracle as orc

    o, logits = orc.paged_selected_attention(q.numpy(), case.pool_np, lists.numpy(), last_idx, last_len,
                                             layout=case.layout, kind=kind)
    return torch.from_numpy(o), logits


def _per_head_page_lists(case, hq, budget, seed):
    """first budget-1 entries of a shuffled iota(num_pages-1) per head, as physical pages"""
    g = torch.Generator().manual_seed(seed)
    rows = []
    for _ in range(hq):
        perm = torch.randperm(case.n_pages - 1, generator=g)[: budget - 1]
        rows.append(case.page_table[perm])
    return torch.stack(rows).to(torch.int32)


SEQ_LENS = [63, 127, 213, 1110, 2000, 4099, 8192, 8222, 12345, 28837]


@pytest.mark.parametrize("head_dim", [64, 128])
@pytest.mark.parametrize("seq_len", SEQ_LENS)
def test_reference_grid_page_lists(cuda, seq_len, head_dim):
    """fp16, NHD, 32/32 heads: page sizes x page budgets of the reference's test."""
    h, dtype = 32, torch.float16
    worst = 0.0
    kv = (randn((seq_len, h, head_dim), seq_len, dtype), randn((seq_len, h, head_dim), seq_len + 1, dtype))
    for page_size in [1, 3, 7, 16, 32]:
        case = PagedCase(seq_len, h, head_dim, page_size, dtype, seed=seq_len + page_size, kv=kv)
        pool = case.pool.to(cuda)
        q = randn((h, head_dim), seq_len * 31 + page_size, dtype)
        for budget in [16, 32, 64, 128]:
            budget = min(budget, case.n_pages)
            if budget < 2:
                continue
            lists = _per_head_page_lists(case, h, budget, seed=budget)
            last_idx = int(case.page_table[-1])
            want, _ = _oracle_paged(q, case, lists, last_idx, case.last_page_len, "pages")
            w = _wrapper(0, h, h, head_dim, page_size, dtype)
            qd = q.to(dtype).to(cuda).unsqueeze(0)
            od = torch.full_like(qd, float("nan"))
            # the reference passes a [H, budget] buffer of which the first budget-1 columns count
            idx_buf = torch.zeros((h, budget), dtype=torch.int32)
            idx_buf[:, : budget - 1] = lists
            indptr = torch.tensor([0, budget - 1], dtype=torch.int32, device=cuda)
            w.forward(qd, od, pool, idx_buf.to(cuda), indptr, case.last_page_len, last_idx, None)
            torch.cuda.synchronize()
            err = tolerance_report(od[0], want)
            worst = max(worst, err)
            assert err <= ATOL[dtype], (seq_len, head_dim, page_size, budget, err)
    print(f"seq_len={seq_len} D={head_dim} worst max-abs {worst:.2e}")


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", [0, 1])
def test_c_restatement_of_reference_checker(cuda, dtype, layout):
    """Same comparison against the C restatement of cpu_reference::selected_single_mha, which
    works on a contiguous cache with logical page numbers."""
    from oracle import cref

    h, d, n, page_size, budget = 32, 128, 2000, 16, 32
    case = PagedCase(n, h, d, page_size, dtype, layout=layout, seed=5)
    q = randn((h, d), 99, dtype)
    g = torch.Generator().manual_seed(1)
    logical = torch.stack([torch.randperm(case.n_pages - 1, generator=g)[: budget - 1]
                           for _ in range(h)])
    sel = torch.cat([logical, torch.full((h, 1), case.n_pages - 1)], dim=1).to(torch.int32)
    kc, vc = case.k.numpy(), case.v.numpy()
    if layout == 1:
        kc, vc = kc.transpose(1, 0, 2).copy(), vc.transpose(1, 0, 2).copy()
    want = torch.from_numpy(cref.selected_single_mha(q.numpy(), kc, vc, sel.numpy(),
                                                     case.last_page_len, page_size, layout))
    phys = case.page_table[logical].to(torch.int32)
    w = _wrapper(layout, h, h, d, page_size, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    od = torch.empty_like(qd)
    w.forward(qd, od, case.pool.to(cuda), phys.to(cuda), None, case.last_page_len,
              int(case.page_table[-1]), None)
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,rows", [(32, 32, 32), (32, 32, 1), (32, 8, 32), (32, 8, 8),
                                         (32, 8, 1), (16, 8, 8), (64, 8, 8), (40, 40, 40),
                                         # group sizes without a shared-row kernel (3, 5, 7, 16)
                                         (24, 8, 8), (24, 8, 24), (20, 4, 4), (28, 4, 1),
                                         (28, 4, 4), (32, 2, 2)])
def test_token_slot_lists(cuda, dtype, hq, hkv, rows):
    """Token-granular lists (slots) with page size 16: per query head, per KV head, shared."""
    from oracle import tidal_oracle as orc

    d, n, page_size, k = 128, 3000, 16, 257
    case = PagedCase(n, hkv, d, page_size, dtype, seed=hq + hkv + rows)
    q = randn((hq, d), 17, dtype)
    g = torch.Generator().manual_seed(3)
    pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(rows)])
    want = orc.sparse_layer_gather(q, case.k, case.v, pos)
    # the reference's own definition: dense logits with masked_fill(finfo.min)
    want2 = orc.sparse_layer(q, case.k, case.v, orc.mask_from_indices(pos, hq, n))
    assert (want - want2).abs().max() < 1e-5
    slots = case.slots_of(pos).to(torch.int32)
    w = _wrapper(0, hq, hkv, d, page_size, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    od = torch.empty_like(qd)
    w.forward(qd, od, case.pool.to(cuda), slots.to(cuda), None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv", [(32, 32), (32, 8), (28, 4)])
@pytest.mark.parametrize("n", [1, 15, 16, 17, 1000, 4099, 33000])
def test_full_attention_with_scores(cuda, dtype, hq, hkv, n):
    """Selection-layer mode: the whole page table in order (shared row), logits and lse out.
    Pinned twice: the oracle's dense attention and torch's scaled_dot_product_attention."""
    from oracle import tidal_oracle as orc

    d, page_size = 128, 16
    case = PagedCase(n, hkv, d, page_size, dtype, seed=n)
    q = randn((hq, d), n + 1, dtype)
    logits = orc.attn_logits(q, case.k)
    want = orc.softmax_pv(logits, case.v)
    kk = orc.repeat_kv(case.k, hq // hkv).permute(1, 0, 2)[None]
    vv = orc.repeat_kv(case.v, hq // hkv).permute(1, 0, 2)[None]
    sdpa = torch.nn.functional.scaled_dot_product_attention(q[None, :, None, :], kk, vv)[0, :, 0]
    assert (want - sdpa).abs().max() < 1e-5
    w = _wrapper(0, hq, hkv, d, page_size, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    od = torch.empty_like(qd)
    stride = case.n_pages * page_size
    scores = torch.full((hq, stride), float("nan"), dtype=torch.float32, device=cuda)
    lse = torch.empty((1, hq), dtype=torch.float32, device=cuda)
    table = case.page_table[:-1].to(torch.int32).unsqueeze(0)
    pool_d = case.pool.to(cuda)
    w.forward(qd, od, pool_d, table.to(cuda), None, case.last_page_len,
              int(case.page_table[-1]), scores, lse=lse)
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype]
    got_logits = scores[:, :n].cpu()
    bound = 2e-4 * max(1.0, logits.abs().max().item())
    err = (got_logits - logits).abs()
    if err.max() > bound:   # say where, and whether a second launch gives the same value
        h, i = divmod(int(err.argmax()), n)
        # where the kernel computed it: workgroup tiles of 8 waves x 16 tokens are dealt to the
        # splits round robin, a wave keeps its logits in a strip of tiles until it is flushed
        plan = w._plan(1, 1, (case.n_pages - 1) * page_size + case.last_page_len, False)
        wg_tokens = plan.waves_per_block * plan.tile_rows * 4
        n_splits = -(-n // plan.chunk_tokens)
        where = (f"split {(i // wg_tokens) % n_splits} of {n_splits}, wave {(i % wg_tokens) // (plan.tile_rows * 4)}, "
                 f"tile {(i // wg_tokens) // n_splits} of that wave, row {i % (plan.tile_rows * 4)} of the tile")
        scores2 = torch.full_like(scores, float("nan"))
        w.forward(qd, od, pool_d, table.to(cuda), None, case.last_page_len,
                  int(case.page_table[-1]), scores2, lse=lse)
        torch.cuda.synchronize()
        # which side is off: the logit once more in float64, from the K row of the CPU inputs and
        # from the K row as it sits in the pool on the GPU
        kvh = h // (hq // hkv)
        k_gpu = pool_d[int(case.page_table[i // page_size]), 0, i % page_size, kvh].double().cpu()
        q64 = q[h].to(dtype).double()
        ref_cpu = float(q64 @ case.k[i, kvh].double()) / d ** 0.5
        ref_gpu_row = float(q64 @ k_gpu) / d ** 0.5
        raise AssertionError(f"logit of head {h}, token {i} ({where}): {got_logits[h, i].item()!r}, oracle "
                             f"{logits[h, i].item()!r}, second launch {scores2[h, i].item()!r}, float64 from "
                             f"the CPU's K row {ref_cpu!r}, from the K row in the GPU pool {ref_gpu_row!r}; "
                             f"{int((err > bound).sum())} entries beyond {bound:.2e}")
    assert torch.isnan(scores[:, n:]).all()  # nothing written past the sequence
    assert (lse[0].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,n", [(32, 32, 4099), (32, 8, 9000), (8, 1, 700)])
def test_logits_in_the_kv_dtype(cuda, dtype, hq, hkv, n):
    """The reference keeps its logits buffer in the model's 16-bit type
    (tidal/utils/controller.py:149-151).  A selection launch that is handed such a buffer stores
    the fp32 logit rounded to that type (within one step of the type of the oracle's logit), the
    attention output is unchanged, and the top-k of the stored rows -- with the launch's
    log-sum-exp as the rows' bound -- is the oracle's stable top-k of exactly those values."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    d, page_size, k = 128, 16, 300
    case = PagedCase(n, hkv, d, page_size, dtype, seed=n + 3)
    q = randn((hq, d), n + 4, dtype)
    logits = orc.attn_logits(q, case.k)
    want = orc.softmax_pv(logits, case.v)
    w = _wrapper(0, hq, hkv, d, page_size, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    od = torch.empty_like(qd)
    stride = case.n_pages * page_size
    scores = torch.full((hq, stride), float("nan"), dtype=dtype, device=cuda)
    lse = torch.empty((1, hq), dtype=torch.float32, device=cuda)
    table = case.page_table[:-1].to(torch.int32).unsqueeze(0)
    w.forward(qd, od, case.pool.to(cuda), table.to(cuda), None, case.last_page_len,
              int(case.page_table[-1]), scores, lse=lse)
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype]
    got = scores[:, :n].cpu()
    assert torch.isnan(scores[:, n:]).all()
    # one step of the 16-bit type at the logit's magnitude: 2^-10 (fp16) / 2^-7 (bf16) relative
    step = (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7) * logits.abs().clamp_min(2.0 ** -14)
    assert ((got.float() - logits).abs() <= step + 2e-4).all()
    assert (lse[0].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3
    # the lse bounds the rounded logits as well?  Rounding up can pass an fp32 bound by half a step:
    # the kernel leaves one bf16 step of room for 16-bit rows (csrc/topk.hip), enough for both types
    out = torch.empty((hq, k), dtype=torch.int32, device=cuda)
    _kernels.topk_filtering(scores[:, :n], None, None, out, None, k, upper_bound=lse.view(-1))
    torch.cuda.synchronize()
    assert torch.equal(out.cpu().long(), orc.stable_topk(got.float(), k))


@pytest.mark.parametrize("k_max", [300, 1800, 5000])
def test_batch_ragged_slots(cuda, k_max):
    """Batch of 8 sequences with different lengths sharing one pool; per-head slot lists with
    per-sequence counts through indptr.  Lists of up to 1800 entries are planned as one workgroup of
    2048 tokens per head and sequence (up to 5000: of 8192), the short ones as four-wave workgroups
    of 128."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page_size = torch.float16, 32, 128, 16
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(300, 5000, (8,), generator=g).tolist()
    ks = [min(int(x), n) for x, n in zip(torch.randint(1, k_max, (8,), generator=g), lens)]
    ks[3] = min(k_max, lens[3])
    total_pages = sum((n + page_size - 1) // page_size for n in lens) + 5
    perm = torch.randperm(total_pages, generator=g)
    pool = torch.full((total_pages, 2, page_size, h, d), 55.0)
    qs, wants, rows, used = [], [], [], 0
    for b, n in enumerate(lens):
        k = randn((n, h, d), 100 + b, dtype)
        v = randn((n, h, d), 200 + b, dtype)
        npg = (n + page_size - 1) // page_size
        table = perm[used: used + npg]
        used += npg
        pad = npg * page_size - n
        pool[table, 0] = torch.cat([k, torch.zeros(pad, h, d)]).view(npg, page_size, h, d)
        pool[table, 1] = torch.cat([v, torch.zeros(pad, h, d)]).view(npg, page_size, h, d)
        q = randn((h, d), 300 + b, dtype)
        pos = torch.stack([torch.randperm(n, generator=g)[: ks[b]] for _ in range(h)])
        wants.append(orc.sparse_layer_gather(q, k, v, pos))
        rows.append((table[pos // page_size] * page_size + pos % page_size).to(torch.int32))
        qs.append(q)
    indptr = torch.tensor([0] + list(np.cumsum(ks)), dtype=torch.int32)
    idx = torch.cat(rows, dim=1).contiguous()
    w = _wrapper(0, h, h, d, page_size, dtype)
    qd = torch.stack(qs).to(dtype).to(cuda)
    od = torch.empty_like(qd)
    zeros = torch.zeros(8, dtype=torch.int32, device=cuda)
    w.forward(qd, od, pool.to(dtype).to(cuda), idx.to(cuda), indptr.to(cuda), zeros, zeros, None,
              index_kind="slots", n_list=max(ks))
    torch.cuda.synchronize()
    for b in range(8):
        assert tolerance_report(od[b], wants[b]) <= ATOL[dtype], b


@pytest.mark.parametrize("hq,hkv,page_size,dtype,lens", [
    (8, 2, 16, torch.float16, None), (4, 4, 16, torch.bfloat16, None), (8, 8, 5, torch.float16, None),
    (16, 2, 8, torch.bfloat16, None),
    # several splits for the long sequences, workgroups without work for the short ones
    (32, 8, 16, torch.float16, [9000, 37, 4100, 2500, 1]),
    (16, 16, 16, torch.bfloat16, [700, 9100, 16, 5000, 3000])])
def test_batch_ragged_page_lists_with_logits(cuda, hq, hkv, page_size, dtype, lens):
    """Selection-layer mode for a batch: every sequence's page table in order through indptr, its
    own last page and last-page length, logits and log-sum-exp per sequence and head."""
    from oracle import tidal_oracle as orc

    d = 128
    lens = lens or [37, 1000, page_size, 333, 1]
    b = len(lens)
    cases = [PagedCase(n, hkv, d, page_size, dtype, seed=60 + i, spare=2) for i, n in enumerate(lens)]
    offs = np.cumsum([0] + [c.max_pages for c in cases])
    pool = torch.cat([c.pool for c in cases]).to(cuda)
    q = randn((b, hq, d), 5, dtype)
    idx = torch.cat([c.page_table[:-1] + int(offs[i]) for i, c in enumerate(cases)]).to(torch.int32)[None]
    counts = [c.n_pages - 1 for c in cases]
    indptr = torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32, device=cuda)
    ll = torch.tensor([c.last_page_len for c in cases], dtype=torch.int32, device=cuda)
    li = torch.tensor([int(c.page_table[-1]) + int(offs[i]) for i, c in enumerate(cases)],
                      dtype=torch.int32, device=cuda)
    stride = max(c.n_pages for c in cases) * page_size + 3
    scores = torch.full((b * hq, stride), float("nan"), dtype=torch.float32, device=cuda)
    lse = torch.empty((b, hq), dtype=torch.float32, device=cuda)
    w = _wrapper(0, hq, hkv, d, page_size, dtype)
    qd = q.to(dtype).to(cuda)
    od = torch.empty_like(qd)
    w.forward(qd, od, pool, idx.to(cuda).contiguous(), indptr, ll, li, scores, lse=lse,
              n_list=max(counts))
    torch.cuda.synchronize()
    for i, c in enumerate(cases):
        logits = orc.attn_logits(q[i], c.k)
        want = orc.softmax_pv(logits, c.v)
        assert tolerance_report(od[i], want) <= ATOL[dtype], i
        got = scores[i * hq: (i + 1) * hq].cpu()
        assert (got[:, : c.n] - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item()), i
        assert torch.isnan(got[:, c.n:]).all(), i
        assert (lse[i].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3, i


@pytest.mark.parametrize("knobs", [dict(waves_per_block=8, fused_merge=1),
                                   dict(waves_per_block=16, fused_merge=1),
                                   dict(waves_per_block=8, fused_merge=0),
                                   dict(waves_per_block=8, fused_merge=1, chunk_tokens=32),
                                   dict(waves_per_block=8, fused_merge=0, chunk_tokens=32),
                                   dict(waves_per_block=16, fused_merge=1, chunk_tokens=100000)])
def test_split_merge_is_an_identity(cuda, knobs):
    """Any partition of the token list (1 ... 64 splits, either merge path) gives the unsplit
    result; repeated calls reuse the ticket counters."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page_size, n, k = torch.bfloat16, 32, 128, 16, 9000, 2048
    case = PagedCase(n, h, d, page_size, dtype, seed=11)
    q = randn((h, d), 12, dtype)
    g = torch.Generator().manual_seed(13)
    pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(h)])
    want = orc.sparse_layer_gather(q, case.k, case.v, pos)
    slots = case.slots_of(pos).to(torch.int32).to(cuda)
    w = _wrapper(0, h, h, d, page_size, dtype, **knobs)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    pool = case.pool.to(cuda)
    for _ in range(3):
        od = torch.full_like(qd, float("nan"))
        w.forward(qd, od, pool, slots, None, 0, 0, None, index_kind="slots")
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want) <= ATOL[dtype]


def test_special_cases(cuda):
    """k = 1 returns the value row; k = N equals full attention; order of the list is irrelevant;
    an empty list with no last page returns zeros."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page_size, n = torch.float16, 32, 128, 16, 777
    case = PagedCase(n, h, d, page_size, dtype, seed=21)
    q = randn((h, d), 22, dtype)
    pool = case.pool.to(cuda)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    w = _wrapper(0, h, h, d, page_size, dtype)

    def run(pos):
        od = torch.full_like(qd, float("nan"))
        slots = case.slots_of(pos).to(torch.int32).to(cuda).contiguous()
        w.forward(qd, od, pool, slots, None, 0, 0, None, index_kind="slots")
        torch.cuda.synchronize()
        return od[0].float().cpu()

    one = torch.randint(0, n, (h, 1), generator=torch.Generator().manual_seed(1))
    got = run(one)
    assert torch.equal(got, case.v[one[:, 0], torch.arange(h)])  # softmax over one token is 1
    everything = torch.arange(n).repeat(h, 1)
    assert (run(everything) - orc.full_attention(q, case.k, case.v)).abs().max() <= ATOL[dtype]
    g = torch.Generator().manual_seed(2)
    pos = torch.stack([torch.randperm(n, generator=g)[:100] for _ in range(h)])
    a = run(pos)
    b = run(pos[:, torch.randperm(100, generator=g)])
    assert (a - b).abs().max() <= 1e-3
    od = torch.full_like(qd, float("nan"))
    empty = torch.zeros((h, 0), dtype=torch.int32, device=cuda)
    w.forward(qd, od, pool, empty, None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()
    assert torch.equal(od.float().cpu(), torch.zeros(1, h, d))


def test_out_of_range_indices_are_clamped_not_faulting(cuda):
    """Indices outside the pool read the pool's last slot instead of faulting."""
    dtype, h, d, page_size, n = torch.float16, 32, 128, 16, 100
    case = PagedCase(n, h, d, page_size, dtype, seed=31)
    w = _wrapper(0, h, h, d, page_size, dtype)
    qd = randn((1, h, d), 1, dtype).to(dtype).to(cuda)
    od = torch.empty_like(qd)
    bad = torch.full((h, 8), 2**30, dtype=torch.int32, device=cuda)
    bad[:, 1] = -5
    w.forward(qd, od, case.pool.to(cuda), bad, None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()
    assert torch.isfinite(od.float()).all()


@pytest.mark.parametrize("index_kind", ["pages", "slots"])
def test_poisoned_device_lengths_leave_the_tickets_clean(cuda, index_kind):
    """Lengths that live on the device are not trusted: a last-page fill beyond the page size is
    read as a full page (both kernels), every workgroup that runs finds its ticket taken care
    of, and the counters are zero again afterwards -- a later call is not disturbed."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page_size, n = torch.float16, 8, 128, 16, 3000
    case = PagedCase(n, h, d, page_size, dtype, seed=41)
    pool = case.pool.to(cuda)
    qd = randn((1, h, d), 1, dtype).to(dtype).to(cuda)
    w = _wrapper(0, h, h, d, page_size, dtype)
    if index_kind == "pages":
        lists = case.page_table[:-1].to(torch.int32).unsqueeze(0).to(cuda)
    else:
        g = torch.Generator().manual_seed(7)
        pos = torch.stack([torch.randperm((case.n_pages - 1) * page_size, generator=g)[:500] for _ in range(h)])
        lists = case.slots_of(pos).to(torch.int32).to(cuda)
    indptr = torch.tensor([0, lists.shape[1]], dtype=torch.int32, device=cuda)
    li = torch.tensor([int(case.page_table[-1])], dtype=torch.int32, device=cuda)
    outs = []
    for fill in (10 ** 6, page_size, -3, 0):
        ll = torch.tensor([fill], dtype=torch.int32, device=cuda)
        o = torch.full_like(qd, float("nan"))
        w.forward(qd, o, pool, lists, indptr, ll, li, None, index_kind=index_kind)
        torch.cuda.synchronize()
        assert torch.isfinite(o.float()).all()
        assert int(w._workspace[: 1 << 20].view(torch.int32).abs().sum()) == 0
        outs.append(o)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[2], outs[3])


def test_error_paths(cuda):
    """forward before begin_forward, unsupported dtype, wrong shapes: RuntimeError, as the
    reference's TORCH_CHECKs / handler raise."""
    from tidaldecode_amd import _kernels

    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    q = torch.zeros((1, 32, 128), dtype=torch.float16, device=cuda)
    pool = torch.zeros((4, 2, 16, 32, 128), dtype=torch.float16, device=cuda)
    idx = torch.zeros((32, 4), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="BeginForward"):
        w.forward(q, q.clone(), pool, idx, None, 1, 0, None)
    with pytest.raises(RuntimeError, match="failed to dispatch"):
        w.begin_forward(None, 32, 32, 128, 16, torch.empty(0, dtype=torch.float32))
    with pytest.raises(RuntimeError, match="multiple"):
        w.begin_forward(None, 32, 5, 128, 16, torch.empty(0, dtype=torch.float16))
    w.begin_forward(None, 32, 32, 128, 16, torch.empty(0, dtype=torch.float16))
    with pytest.raises(RuntimeError):
        w.forward(q, q.clone(), pool, idx.long(), None, 1, 0, None)
    with pytest.raises(RuntimeError):
        w.forward(q, q.clone(), pool, idx, None, 17, 0, None)  # last_page_len > page_size
    with pytest.raises(RuntimeError):
        w.forward(q, q.clone(), pool, idx, None, 1, 4, None)  # last_page_idx outside the pool
    with pytest.raises(RuntimeError):
        w.forward(q.cpu(), q.clone(), pool, idx, None, 1, 0, None)
    w.end_forward()
    with pytest.raises(RuntimeError, match="BeginForward"):
        w.forward(q, q.clone(), pool, idx, None, 1, 0, None)
    w48 = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w48.begin_forward(None, 32, 32, 48, 16, torch.empty(0, dtype=torch.float16))
    q48 = torch.zeros((1, 32, 48), dtype=torch.float16, device=cuda)
    pool48 = torch.zeros((4, 2, 16, 32, 48), dtype=torch.float16, device=cuda)
    with pytest.raises(RuntimeError, match="head_dim"):
        w48.forward(q48, q48.clone(), pool48, idx, None, 1, 0, None)


@pytest.mark.parametrize("seed", range(40))
def test_random_configurations(cuda, seed):
    """Seeded random draws over what the grids above enumerate one axis at a time: head counts and
    group sizes, head_dim, page size, layout, dtype, length, budget, list rows, duplicates-free
    token lists (slots) and the selection-layer mode (whole page table + logits) on the same
    case.  Every draw is checked against the oracle's gathered / dense attention."""
    import random

    from oracle import tidal_oracle as orc

    rnd = random.Random(1000 + seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    d = rnd.choice([64, 128, 128, 256])
    hkv = rnd.choice([1, 2, 4, 8])
    group = rnd.choice([1, 1, 2, 4, 8]) if d == 128 else rnd.choice([1, 2, 4])
    if seed >= 24:   # group sizes that run padded, or as several head rows per KV head
        group = rnd.choice([3, 5, 6, 7, 9, 12, 16])
    hq = hkv * group
    page_size = rnd.choice([1, 2, 4, 8, 16, 16, 32])
    layout = rnd.choice([0, 1])
    n = rnd.choice([1, 7, 16, 33, 250, 1000, 2500, 6000])
    case = PagedCase(n, hkv, d, page_size, dtype, layout=layout, seed=seed + 50)
    q = randn((hq, d), seed + 99, dtype)
    w = _wrapper(layout, hq, hkv, d, page_size, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    pool = case.pool.to(cuda)

    # token lists: per query head, per KV head or shared
    rows = rnd.choice(sorted({1, hkv, hq}))
    k = rnd.randint(1, n)
    g = torch.Generator().manual_seed(seed)
    pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(rows)])
    want = orc.sparse_layer_gather(q, case.k, case.v, pos)
    od = torch.empty_like(qd)
    w.forward(qd, od, pool, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
              index_kind="slots")
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype], ("slots", dtype, d, hq, hkv, page_size, layout, n, k, rows)

    # selection-layer mode on the same cache
    logits = orc.attn_logits(q, case.k)
    want_full = orc.softmax_pv(logits, case.v)
    stride = case.n_pages * page_size
    scores = torch.full((hq, stride), float("nan"), dtype=torch.float32, device=cuda)
    lse = torch.empty((1, hq), dtype=torch.float32, device=cuda)
    table = case.page_table[:-1].to(torch.int32).unsqueeze(0)
    od2 = torch.empty_like(qd)
    w.forward(qd, od2, pool, table.to(cuda), None, case.last_page_len, int(case.page_table[-1]),
              scores, lse=lse)
    torch.cuda.synchronize()
    assert tolerance_report(od2[0], want_full) <= ATOL[dtype], ("pages", dtype, d, hq, hkv, page_size, layout, n)
    assert (scores[:, :n].cpu() - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item())
    assert torch.isnan(scores[:, n:]).all()
    assert (lse[0].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3


@pytest.mark.parametrize("fused_merge", [1, 0])
@pytest.mark.parametrize("hq,hkv,d", [(6, 2, 128), (12, 4, 128), (10, 2, 128), (12, 2, 128), (28, 4, 128),
                                      (7, 1, 128), (32, 2, 128), (24, 2, 128), (32, 1, 128), (18, 2, 128),
                                      # head_dim 64 / 256: shared rows on the vector ALU
                                      (8, 2, 64), (6, 2, 64), (32, 2, 64), (14, 2, 64),
                                      (8, 2, 256), (6, 2, 256), (10, 2, 256), (4, 2, 256)])
def test_padded_query_groups(cuda, hq, hkv, d, fused_merge):
    """Groups of 3, 5, 6 and 7 query heads per KV head run on the 4- and 8-head shared-row kernels
    with padding heads, larger groups (16, 12, 32, 9) as several head rows of 8: outputs, logits and log-sum-exps of the real heads must be those of the
    oracle, nothing may be written for the padding, on one split and on many, with the in-kernel
    and the second-kernel merge."""
    from oracle import tidal_oracle as orc

    page_size, dtype = 16, torch.bfloat16
    for n, k in ((40, 33), (5000, 1500)):
        case = PagedCase(n, hkv, d, page_size, dtype, seed=hq * n)
        q = randn((hq, d), hq + n, dtype)
        w = _wrapper(0, hq, hkv, d, page_size, dtype, fused_merge=fused_merge)
        qd = q.to(dtype).to(cuda).unsqueeze(0)
        pool = case.pool.to(cuda)
        g = torch.Generator().manual_seed(n)
        for rows in (hkv, 1):
            pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(rows)])
            want = orc.sparse_layer_gather(q, case.k, case.v, pos)
            od = torch.full((1, hq + 2, d), 9.0, dtype=dtype, device=cuda)  # two guard rows behind o
            w.forward(qd, od[:, :hq], pool, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
                      index_kind="slots")
            torch.cuda.synchronize()
            assert tolerance_report(od[0, :hq], want) <= ATOL[dtype], (n, rows)
            assert (od[0, hq:] == 9.0).all()
        logits = orc.attn_logits(q, case.k)
        stride = case.n_pages * page_size
        scores = torch.full((hq + 2, stride), float("nan"), dtype=torch.float32, device=cuda)
        lse = torch.full((1, hq + 2), float("nan"), dtype=torch.float32, device=cuda)
        od = torch.empty_like(qd)
        table = case.page_table[:-1].to(torch.int32).unsqueeze(0).to(cuda)
        w.forward(qd, od, pool, table, None, case.last_page_len, int(case.page_table[-1]),
                  scores[:hq], lse=lse[:, :hq])
        torch.cuda.synchronize()
        assert tolerance_report(od[0], orc.softmax_pv(logits, case.v)) <= ATOL[dtype], n
        assert (scores[:hq, :n].cpu() - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item())
        assert torch.isnan(scores[hq:]).all() and torch.isnan(scores[:hq, n:]).all()
        assert (lse[0, :hq].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3
        assert torch.isnan(lse[0, hq:]).all()


@pytest.mark.parametrize("hq,hkv,d", [(4, 4, 128), (8, 2, 128), (4, 2, 128), (8, 1, 128), (2, 2, 64),
                                      (2, 2, 256), (8, 2, 64), (16, 2, 64), (8, 2, 256), (6, 2, 256)])
def test_logits_of_long_wave_runs(cuda, hq, hkv, d):
    """One split for the whole sequence: every wave walks hundreds of tiles, so the logits leave
    the per-wave staging strip several times in mid-loop (and once more, partly filled, at the
    end).  All of them must land at their token, nothing past the sequence."""
    from oracle import tidal_oracle as orc

    dtype, page_size, n = torch.float16, 16, 20011
    case = PagedCase(n, hkv, d, page_size, dtype, seed=hq + d)
    q = randn((hq, d), 5, dtype)
    logits = orc.attn_logits(q, case.k)
    want = orc.softmax_pv(logits, case.v)
    knob_sets = [dict(chunk_tokens=1 << 20)]
    if hq == hkv:  # sixteen-wave workgroups exist for one query head per row
        knob_sets.append(dict(chunk_tokens=1 << 20, waves_per_block=16))
    for knobs in knob_sets:
        w = _wrapper(0, hq, hkv, d, page_size, dtype, **knobs)
        qd = q.to(dtype).to(cuda).unsqueeze(0)
        od = torch.empty_like(qd)
        stride = case.n_pages * page_size
        scores = torch.full((hq, stride), float("nan"), dtype=torch.float32, device=cuda)
        lse = torch.empty((1, hq), dtype=torch.float32, device=cuda)
        table = case.page_table[:-1].to(torch.int32).unsqueeze(0)
        w.forward(qd, od, case.pool.to(cuda), table.to(cuda), None, case.last_page_len,
                  int(case.page_table[-1]), scores, lse=lse)
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want) <= ATOL[dtype], knobs
        assert (scores[:, :n].cpu() - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item())
        assert torch.isnan(scores[:, n:]).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("n_parts", [1, 2, 7, 32])
def test_merge_states_of_any_partition_is_the_unsplit_result(cuda, dtype, n_parts):
    """td_merge_states: the tokens of a sequence are dealt into n_parts random subsets (one left
    empty on purpose when there are several), each attended to on its own with its log-sum-exp;
    merged, they must give the attention over all tokens — against the oracle, and against the
    closed form o = sum o_i e^(lse_i - lse) evaluated on the host from the same parts."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    hq, hkv, d, page_size, n = 8, 2, 128, 16, 3000
    case = PagedCase(n, hkv, d, page_size, dtype, seed=n_parts)
    q = randn((hq, d), 5, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    pool = case.pool.to(cuda)
    g = torch.Generator().manual_seed(n_parts)
    owner = torch.randint(0, max(1, n_parts - 1) if n_parts > 2 else n_parts, (n,), generator=g)
    w = _wrapper(0, hq, hkv, d, page_size, dtype)
    o_parts = torch.full((n_parts, 1, hq, d), float("nan"), dtype=dtype, device=cuda)
    lse_parts = torch.full((n_parts, 1, hq), float("-inf"), dtype=torch.float32, device=cuda)
    for i in range(n_parts):
        pos = (owner == i).nonzero().flatten()
        if pos.numel() == 0:
            continue                      # an empty part: lse stays -inf, o stays NaN
        slots = case.slots_of(pos).to(torch.int32).unsqueeze(0).to(cuda)
        w.forward(qd, o_parts[i], pool, slots, None, 0, 0, None, index_kind="slots",
                  lse=lse_parts[i])
    o, lse = _kernels.merge_states(o_parts, lse_parts)
    torch.cuda.synchronize()
    logits = orc.attn_logits(q, case.k)
    assert tolerance_report(o[0], orc.softmax_pv(logits, case.v)) <= ATOL[dtype]
    assert (lse[0].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3
    # closed form on the host from the same parts
    lp, op = lse_parts.cpu()[:, 0], torch.nan_to_num(o_parts.float().cpu()[:, 0])
    tot = torch.logsumexp(lp, 0)
    want = (op * torch.exp(lp - tot)[..., None]).sum(0)
    eps = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    assert ((o[0].float().cpu() - want).abs() <= eps * want.abs() + 1e-5).all()
    # fp32 parts, no lse wanted
    o32, none = _kernels.merge_states(o_parts.float(), lse_parts, want_lse=False)
    assert none is None and ((o32[0].cpu() - want).abs() <= 1e-5 * want.abs().clamp(min=1.0)).all()
    with pytest.raises(RuntimeError):
        _kernels.merge_states(o_parts, lse_parts[:, :, :4].contiguous())

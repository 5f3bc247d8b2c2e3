"""GPU parity: top-k selection (td_topk) and the cross-head score reduction (td_score_reduce).

The index sets must be BIT-EXACT against the oracle's stable rule (k largest, ties to the lower
position) when both see the same scores.  The oracle's rule itself is pinned in
tests/test_oracle.py (torch.topk as sets, brute force on ties, the independent C qsort).
"""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


_scratch = {}


def _shared_scratch(cuda, rows):
    """One scratch tensor for the whole module: zeroed at allocation only, so every cooperative
    call after the first (rows of more than 65536 elements) relies on the previous call having
    left it clean."""
    from tidaldecode_amd import _kernels

    need = _kernels.topk_workspace_bytes(64)
    assert rows <= 64
    if "buf" not in _scratch:
        _scratch["buf"] = torch.zeros(need, dtype=torch.uint8, device=cuda)
    return _scratch["buf"]


def _gpu_topk(values, k, cuda, in_idx=None, page_table=None, page_size=1, want_vals=True,
              scratch=False, upper_bound=None):
    from tidaldecode_amd import _kernels

    rows = values.shape[0]
    out_idx = torch.full((rows, k), -1, dtype=torch.int32, device=cuda)
    out_val = torch.zeros((rows, k), dtype=values.dtype, device=cuda) if want_vals else None
    _kernels.topk_filtering(values.to(cuda), None if in_idx is None else in_idx.to(cuda), out_val,
                            out_idx, _shared_scratch(cuda, rows) if scratch else None, k,
                            page_table=None if page_table is None else page_table.to(cuda),
                            page_size=page_size,
                            upper_bound=None if upper_bound is None else upper_bound.to(cuda))
    torch.cuda.synchronize()
    return out_idx.cpu(), None if out_val is None else out_val.cpu()


def _check(values, k, cuda):
    from oracle import cref, tidal_oracle as orc

    got, vals = _gpu_topk(values, k, cuda)
    want = orc.stable_topk(values.float(), k)
    assert torch.equal(got.long(), want), "index set differs from the stable oracle"
    want_c = cref.stable_topk(values.float().numpy(), k)
    assert np.array_equal(got.numpy(), want_c)
    expect = torch.gather(values, 1, want)  # values travel with their index (NaN == NaN here)
    assert torch.equal(torch.nan_to_num(vals.float(), nan=1e38), torch.nan_to_num(expect.float(), nan=1e38))
    # with scratch: rows of more than 65536 elements take the three cooperative launches
    got2, vals2 = _gpu_topk(values, k, cuda, scratch=True)
    assert torch.equal(got2, got), "cooperative path differs"
    assert torch.equal(torch.nan_to_num(vals2.float(), nan=1e38), torch.nan_to_num(vals.float(), nan=1e38))
    # with an upper bound per row (the row maximum itself, then looser ones: what a log-sum-exp or
    # a head count is to the scores); rows that hold a NaN say "no bound", as an lse would
    for bound in _bounds(values):
        got3, vals3 = _gpu_topk(values, k, cuda, upper_bound=bound)
        assert torch.equal(got3, got), "selection from a bound differs"
        assert torch.equal(torch.nan_to_num(vals3.float(), nan=1e38), torch.nan_to_num(vals.float(), nan=1e38))
    return got


def _bounds(values):
    v = values.float()
    no_bound = torch.isnan(v).any(dim=1)
    # (not nan_to_num: it also turns +inf into the largest finite value, which is no bound of +inf)
    top = torch.where(torch.isnan(v), torch.full_like(v, float("-inf")), v).amax(dim=1)
    out = []
    for b in (top, top + 0.37 * top.abs() + 3.0, top + 1e-3 * top.abs(), top.abs() * 64 + 1e-30):
        b = b.clone()
        b[no_bound] = float("nan")
        out.append(b.contiguous())
    return out


@pytest.mark.parametrize("rows,n,k", [(32, 4096, 256), (32, 32768, 2048), (1, 32768, 2048),
                                      (8, 102400, 4096), (32, 8192, 64), (3, 1000, 999),
                                      (5, 70, 70), (2, 1, 1), (4, 63, 1), (4, 65, 64),
                                      (2, 1025, 512), (1, 131072, 4096), (2, 262144, 5000), (64, 20000, 300)])
def test_random_scores_fp32(cuda, rows, n, k):
    g = torch.Generator().manual_seed(rows * 1000003 + n + k)
    _check(torch.randn((rows, n), generator=g), k, cuda)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,n,k", [(32, 8192, 256), (32, 4097, 128), (2, 50, 7)])
def test_half_precision_scores_have_many_ties(cuda, dtype, rows, n, k):
    """The reference feeds fp16 scores (tidal/ops/csrc/topk.cu:31-41): thousands of exact ties."""
    g = torch.Generator().manual_seed(n + k)
    _check(torch.randn((rows, n), generator=g).to(dtype), k, cuda)


def test_ties_go_to_the_lower_position(cuda):
    g = torch.Generator().manual_seed(7)
    # 5 distinct values only: the threshold value occurs thousands of times
    v = torch.randint(0, 5, (16, 20000), generator=g).float()
    got = _check(v, 3000, cuda)
    assert (got[:, 1:] > got[:, :-1]).all()  # ascending, no duplicates
    # all equal: the first k positions
    got = _check(torch.full((4, 5000), 1.25), 777, cuda)
    assert torch.equal(got, torch.arange(777, dtype=torch.int32).repeat(4, 1))


@pytest.mark.parametrize("n,k", [(64, 5), (1500, 1500), (32768, 2048), (40000, 1), (65536, 4096)])
def test_rows_of_one_value(cuda, n, k):
    """Every score of a row equal (zeros, a NaN row, -inf, a denormal): the selection has nothing to
    rank and goes from the extremes of the row straight to the emission; the first k positions."""
    first_k = torch.arange(k, dtype=torch.int32)
    for value in (0.0, -0.0, float("nan"), float("-inf"), float("inf"), 1e-42, -7.25):
        rows = torch.full((3, n), value)
        rows[1, 1::2] = -value if value == 0.0 else value      # +0 and -0 are one value
        got = _check(rows, k, cuda)
        assert torch.equal(got, first_k.repeat(3, 1)), value


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
def test_long_rows_with_crowded_threshold_bins(cuda, dtype):
    """Rows whose keys share their leading bits (more candidates than the cooperative kernel keeps
    in LDS), rows of a single value, NaN-heavy rows and a length that is not a slice multiple."""
    g = torch.Generator().manual_seed(11)
    n = 40000 + 77
    tight = (1.0 + torch.rand((3, n), generator=g) * 1e-3).to(dtype)      # one 11-bit bin
    _check(tight, 2048, cuda)
    _check(tight, n - 5, cuda)
    tighter = (1.0 + torch.rand((2, n), generator=g) * 2e-7).to(dtype)    # 2-3 distinct fp32 keys
    _check(tighter, 5000, cuda)
    _check(torch.full((2, n), -3.5).to(dtype), 4097, cuda)
    v = torch.randn((4, n), generator=g)
    v[:, ::3] = float("nan")
    v[1, 1::3] = float("inf")
    v[2, :] = -v[2, :].abs()
    _check(v.to(dtype), 20000, cuda)
    _check(v.to(dtype), 1, cuda)
    _check(v.to(dtype), n, cuda)


@pytest.mark.parametrize("n", [5000, 32768, 30000 + 77, 50000])
def test_score_distributions_that_steer_the_radix_levels(cuda, n):
    """The one-launch kernel maps scores to d = distance below the row maximum and starts its radix
    select 64 binades below that maximum.  Rows that leave the usual road: all negative; fewer
    non-negative scores than k (threshold below zero); a threshold 100 binades below the maximum
    (second pass over the rest of the range); +0 / -0 ties at the threshold; denormals; a threshold
    bin with hundreds of members (radix levels on the gathered list) and with thousands (another
    level over the row before anything is gathered)."""
    g = torch.Generator().manual_seed(n)
    k = max(1, n // 16)
    neg = -10.0 + 2.0 * torch.randn((2, n), generator=g)
    few_pos = -3.0 + torch.randn((2, n), generator=g)
    assert ((few_pos >= 0).sum(1) < k).all()
    wide = torch.rand((2, n), generator=g) * 1e-30
    wide[:, torch.randperm(n, generator=g)[: k // 2]] = 0.5 + 0.5 * torch.rand((2, k // 2), generator=g)
    zeros = -torch.rand((2, n), generator=g)
    idx = torch.randperm(n, generator=g)
    zeros[:, idx[: k // 4]] = torch.rand((2, k // 4), generator=g) + 0.1
    zeros[:, idx[k // 4: 2 * k]] = 0.0
    zeros[:, idx[k // 2: 2 * k: 3]] = -0.0
    den = torch.randn((2, n), generator=g) * 1e-41
    for v in (neg, few_pos, wide, zeros, den):
        _check(v, k, cuda)
    # one bin at 1.0 is 2^16 ulps = 0.0078 wide
    for members in (600, 3000):
        if 2 * members > n:
            continue
        v = torch.rand((2, n), generator=g) * 0.9
        idx = torch.randperm(n, generator=g)
        v[:, idx[:members]] = 1.0 + torch.rand((2, members), generator=g) * 0.007
        v[:, idx[members: members + 300]] = 1.01 + torch.rand((2, 300), generator=g)
        _check(v, 300 + members // 2, cuda)


def test_sorted_and_blocky_long_rows(cuda):
    """Rows whose threshold bin sits in one slice only (sorted input), in the last partial slice, or
    alternates between slices: the per-slice candidate lists and offsets of the several-workgroups
    path must still add up."""
    g = torch.Generator().manual_seed(21)
    n = 100000 + 13
    base = torch.randn((1, n), generator=g)
    asc = torch.sort(base, dim=1).values
    desc = torch.flip(asc, dims=[1])
    blocky = base.clone()
    blocky[:, 8192:16384] += 10.0          # one slice holds everything above the threshold
    tail = base.clone()
    tail[:, -100:] += 20.0                 # the winners start in the last, partial slice
    v = torch.cat([asc, desc, blocky, tail])
    for k in (1, 100, 4096, 8192, 50000):
        _check(v, k, cuda)


def test_payloads_on_long_rows(cuda):
    from oracle import tidal_oracle as orc

    g = torch.Generator().manual_seed(5)
    n, k, page = 50000, 3000, 16
    v = torch.randn((4, n), generator=g)
    want = orc.stable_topk(v, k)
    in_idx = torch.randint(0, 1 << 30, (4, n), generator=g, dtype=torch.int32)
    got, _ = _gpu_topk(v, k, cuda, in_idx=in_idx, scratch=True)
    assert torch.equal(got.long(), torch.gather(in_idx.long(), 1, want))
    table = torch.randperm((n + page - 1) // page, generator=g).int()
    got, _ = _gpu_topk(v, k, cuda, page_table=table, page_size=page, scratch=True, want_vals=False)
    assert torch.equal(got.long(), table.long()[want // page] * page + want % page)


def test_signed_zero_inf_and_nan(cuda):
    v = torch.zeros((2, 300))
    v[0, 10::7] = -0.0          # -0 and +0 are equal: position decides
    v[0, 5] = float("inf")
    v[0, 6] = float("-inf")
    v[0, 200] = float("nan")    # NaN orders above +inf, as in torch.topk / torch.sort
    v[1] = -torch.arange(300).float()
    v[1, 250] = float("nan")
    for k in (1, 2, 50, 299, 300):
        _check(v, k, cuda)


def test_a_bound_below_the_scores_is_harmless(cuda):
    """A bound that is none (below some score of its row) makes the selection unspecified, but the
    call returns and writes nothing but positions of the row: scores above the bound are never
    counted, and the search gives up when it has covered the whole range without finding k
    elements (tests/test_topk_level_loop.py restates that rule)."""
    g = torch.Generator().manual_seed(3)
    for v, bound, k in ((torch.full((2, 64), float("inf")), 3.4028234663852886e38, 5),
                        (torch.randn((4, 5000), generator=g), 0.0, 5000),
                        (torch.randn((4, 5000), generator=g), -5.0, 4999),
                        (torch.randn((3, 40000), generator=g), 1.0, 2048)):
        got, _ = _gpu_topk(v, k, cuda, upper_bound=torch.full((v.shape[0],), bound), want_vals=False)
        assert ((got >= -1) & (got < v.shape[1])).all()


def test_closed_forms(cuda):
    g = torch.Generator().manual_seed(11)
    v = torch.randn((32, 5000), generator=g)
    got, _ = _gpu_topk(v, 1, cuda)
    assert torch.equal(got[:, 0].long(), v.argmax(dim=1))
    got, _ = _gpu_topk(v, 5000, cuda)
    assert torch.equal(got, torch.arange(5000, dtype=torch.int32).repeat(32, 1))
    # every unselected score <= the smallest selected one
    got, vals = _gpu_topk(v, 321, cuda)
    mask = torch.ones_like(v, dtype=torch.bool).scatter_(1, got.long(), False)
    assert (v.masked_fill(~mask, float("-inf")).max(1).values <= vals.min(1).values).all()
    # torch.topk agrees as a set (no ties in continuous data)
    ref = torch.topk(v, 321, dim=-1).indices.sort(-1).values
    assert torch.equal(got.long(), ref)


def test_payloads(cuda):
    """in_idx payload (the reference's meaning: physical page of each position), page-table
    payload (token slots) and plain positions."""
    from oracle import tidal_oracle as orc

    g = torch.Generator().manual_seed(5)
    rows, n, k, page = 8, 3000, 100, 16
    v = torch.randn((rows, n), generator=g)
    want = orc.stable_topk(v, k)
    payload = torch.randint(0, 10**6, (rows, n), generator=g, dtype=torch.int32)
    got, _ = _gpu_topk(v, k, cuda, in_idx=payload)
    assert torch.equal(got, torch.gather(payload, 1, want))
    n_pages = (n + page - 1) // page
    table = torch.randperm(n_pages + 9, generator=g)[:n_pages].to(torch.int32)
    got, _ = _gpu_topk(v, k, cuda, page_table=table, page_size=page)
    assert torch.equal(got.long(), table.long()[want // page] * page + want % page)
    # fewer payload columns than values: only those columns take part
    got, _ = _gpu_topk(v, k, cuda, in_idx=payload[:, :500].contiguous())
    assert torch.equal(got, torch.gather(payload, 1, orc.stable_topk(v[:, :500], k)))


def test_page_table_per_row_group(cuda):
    """A batch of sequences in one call: rows of group g read page table g.  Short rows (one
    workgroup per row) and long rows (several workgroups per row) against the oracle."""
    from oracle import tidal_oracle as orc

    g = torch.Generator().manual_seed(17)
    for groups, per, n, k, page in ((3, 4, 3000, 100, 16), (4, 8, 20000, 2048, 16), (2, 1, 9000, 50, 5)):
        rows = groups * per
        v = torch.randn((rows, n), generator=g)
        n_pages = (n + page - 1) // page
        tables = torch.stack([torch.randperm(n_pages + 7, generator=g)[:n_pages] for _ in range(groups)]).int()
        want_pos = orc.stable_topk(v, k)
        want = torch.stack([tables[r // per].long()[want_pos[r] // page] * page + want_pos[r] % page
                            for r in range(rows)])
        for scratch in (False, True):
            got, _ = _gpu_topk(v, k, cuda, page_table=tables, page_size=page, want_vals=False,
                               scratch=scratch)
            assert torch.equal(got.long(), want), (groups, per, n, scratch)
    from tidaldecode_amd import _kernels
    out = torch.zeros((5, 10), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="tables"):
        _kernels.topk_filtering(torch.zeros((5, 100), device=cuda), None, None, out, None, 10,
                                page_table=torch.zeros((2, 100), dtype=torch.int32, device=cuda))


def test_lengths_per_row_group(cuda):
    """Device-side lengths: rows of group g rank only their first lengths[g] columns (what lies
    behind is larger than everything and must not be chosen) and select min(k, lengths[g]);
    the rest of a short row's output stays as it was."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    g = torch.Generator().manual_seed(23)
    for per, n, k, lens, page in ((4, 3000, 100, [3000, 57, 1, 100, 2999], 16),
                                  (8, 40000, 2048, [40000, 9000, 17, 8193, 30000], 16),
                                  (1, 70000, 500, [70000, 12, 65537], 4)):
        groups = len(lens)
        rows = groups * per
        v = torch.randn((rows, n), generator=g)
        for gi, ln in enumerate(lens):
            v[gi * per: (gi + 1) * per, ln:] = 1e9
        n_pages = (n + page - 1) // page
        tables = torch.stack([torch.randperm(n_pages + 3, generator=g)[:n_pages] for _ in range(groups)]).int()
        lengths = torch.tensor(lens, dtype=torch.int32, device=cuda)
        # a bound of what is ranked: the columns behind a row's length exceed it and do not count
        ranked_top = torch.stack([v[r, :lens[r // per]].max() for r in range(rows)]).to(cuda)
        for scratch, bound in ((False, None), (True, None), (False, ranked_top + 0.5)):
            out = torch.full((rows, k), -1, dtype=torch.int32, device=cuda)
            _kernels.topk_filtering(v.to(cuda), None, None, out, _shared_scratch(cuda, rows) if scratch else None,
                                    k, page_table=tables.to(cuda), page_size=page, lengths=lengths,
                                    upper_bound=bound)
            torch.cuda.synchronize()
            out = out.cpu().long()
            for r in range(rows):
                ln = lens[r // per]
                kr = min(k, ln)
                pos = orc.stable_topk(v[r: r + 1, :ln], kr)[0]
                want = tables[r // per].long()[pos // page] * page + pos % page
                assert torch.equal(out[r, :kr], want), (n, r, scratch, bound is not None)
                assert (out[r, kr:] == -1).all(), (n, r, scratch, bound is not None)
    with pytest.raises(RuntimeError, match="lengths"):
        _kernels.topk_filtering(torch.zeros((5, 100), device=cuda), None, None,
                                torch.zeros((5, 10), dtype=torch.int32, device=cuda), None, 10,
                                lengths=torch.ones(2, dtype=torch.int32, device=cuda))


def test_topk_errors(cuda):
    from tidaldecode_amd import _kernels

    v = torch.zeros((4, 100), device=cuda)
    out = torch.zeros((4, 10), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError):
        _kernels.topk_filtering(v, None, None, out, None, 11)            # out shape != k
    with pytest.raises(RuntimeError):
        _kernels.topk_filtering(v, None, None, out.long(), None, 10)     # not int32
    with pytest.raises(RuntimeError):
        _kernels.topk_filtering(v.double(), None, None, out, None, 10)   # dtype dispatch
    big = torch.zeros((4, 200), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError):
        _kernels.topk_filtering(v, None, None, big, None, 200)           # k > len


@pytest.mark.parametrize("hq,hkv,n", [(32, 32, 4096), (32, 8, 5000), (40, 40, 33), (32, 8, 1),
                                      (3, 1, 100), (64, 2, 777), (17, 17, 64), (20, 4, 65)])
def test_score_reduce(cuda, hq, hkv, n):
    """sum over heads of softmax probabilities, from logits + lse, against the closed form."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    g = torch.Generator().manual_seed(n)
    logits = torch.randn((hq, n + 7), generator=g) * 3
    lse = torch.logsumexp(logits[:, :n], dim=-1)
    for mode, rows in (("head_sum", 1), ("group_sum", hkv)):
        got = _kernels.score_reduce(logits.to(cuda), lse.to(cuda), hkv, n, mode).cpu()
        want = orc.head_sum_scores(logits[:, :n], rows)
        assert got.shape == want.shape
        assert (got - want).abs().max() <= 2e-6 * hq
        # probabilities of each head sum to one
        assert (got.sum() - hq).abs() <= 1e-3 * hq

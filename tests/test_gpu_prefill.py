"""GPU parity: paged prefill attention (td_prefill_attn through prefill_with_paged_kv_cache)
against the CPU oracle's dense causal attention (pinned against torch SDPA in
tests/test_oracle.py).  Tolerance: max-abs 2e-3 (fp16) / 1e-2 (bf16) on identically rounded inputs,
scaled by max(1, |o|): the first rows of a prompt average one or two value rows, so |o| reaches 3-4
there and the rounding of the bf16 result alone is 8e-3 at that magnitude.
The grid follows the reference's prefill test (kernels/src/test/test_batch_prefill.cu: query
lengths against longer caches, page sizes, causal on/off, both layouts)."""
import math

import pytest
import torch

from _util import ATOL, PagedCase, randn

pytestmark = pytest.mark.gpu


def _dense(q, k, v, causal):
    """fp32 reference: q [n_q, Hq, D] are the newest n_q of the kv_len tokens in k, v [kv_len, Hkv, D]"""
    n_q, hq, d = q.shape
    kv_len, hkv, _ = k.shape
    g = hq // hkv
    kk, vv = k.repeat_interleave(g, 1), v.repeat_interleave(g, 1)
    logit = torch.einsum("qhd,khd->hqk", q, kk) / math.sqrt(d)
    if causal:
        qpos = torch.arange(kv_len - n_q, kv_len)[:, None]
        logit = logit.masked_fill(torch.arange(kv_len)[None, :] > qpos, float("-inf"))
    return torch.einsum("hqk,khd->qhd", logit.softmax(-1), vv)


def _run(cuda, case, q, causal, dtype):
    from tidaldecode_amd import _kernels

    o = _kernels.prefill_with_paged_kv_cache(
        q.to(dtype).to(cuda), case.pool.to(cuda), case.page_table.to(torch.int32).to(cuda),
        case.last_page_len, causal, case.layout, False, 1.0, 1e4)
    torch.cuda.synchronize()
    return o


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("kv_len,n_q", [(1, 1), (17, 17), (70, 70), (128, 128), (129, 129),
                                        (1000, 1000), (4099, 4099), (4099, 37), (5000, 1),
                                        (777, 300), (2048, 129)])
def test_causal_prefill_matches_dense_attention(cuda, dtype, kv_len, n_q):
    hq, hkv, d, page = 8, 8, 128, 16
    case = PagedCase(kv_len, hkv, d, page, dtype, seed=kv_len + n_q)
    q = randn((n_q, hq, d), kv_len * 3 + n_q, dtype)
    want = _dense(q, case.k, case.v, True)
    # the oracle's single-query attention on the last row: the same restatement the decode tests use
    from oracle import tidal_oracle as orc

    last = orc.softmax_pv(orc.attn_logits(q[-1], case.k), case.v)
    assert (want[-1] - last).abs().max() < 1e-5
    got = _run(cuda, case, q, True, dtype)
    assert got.shape == (n_q, hq, d)
    assert ((got.float().cpu() - want).abs() <= ATOL[dtype] * want.abs().clamp(min=1.0)).all()


@pytest.mark.parametrize("hq,hkv,d,page,layout,causal", [
    (32, 8, 128, 16, 0, True), (4, 2, 64, 4, 0, True), (4, 4, 64, 16, 1, True),
    (8, 2, 128, 1, 0, True), (8, 8, 128, 8, 1, True), (6, 3, 128, 5, 0, True),
    (8, 8, 128, 16, 0, False), (4, 2, 64, 16, 1, False), (4, 2, 256, 16, 0, True),
    (2, 2, 256, 8, 1, True), (4, 1, 256, 16, 0, False)])
def test_head_layouts_page_sizes_and_non_causal(cuda, hq, hkv, d, page, layout, causal):
    dtype = torch.float16
    kv_len, n_q = 1500, 333
    case = PagedCase(kv_len, hkv, d, page, dtype, layout=layout, seed=hq * d + page)
    q = randn((n_q, hq, d), 11, dtype)
    want = _dense(q, case.k, case.v, causal)
    got = _run(cuda, case, q, causal, dtype)
    assert ((got.float().cpu() - want).abs() <= ATOL[dtype] * want.abs().clamp(min=1.0)).all()


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("head_dim", [64, 128])
@pytest.mark.parametrize("page_size", [1, 8, 16])
@pytest.mark.parametrize("hq,hkv", [(32, 4), (32, 8), (32, 32), (8, 1), (8, 2), (8, 8)])
def test_reference_prefill_grid(cuda, hq, hkv, page_size, head_dim, causal):
    """The reference's prefill test grid (kernels/src/test/test_prefill.cu:408-467): its three
    families of lengths -- a few queries over a short cache (q in [1, 15), kv in [15, 257)), a fresh
    short prompt (q = kv in [1, 64)) and 63 queries over 2047 cached tokens -- with seeded draws."""
    dtype = torch.float16
    g = torch.Generator().manual_seed(hq * 1000 + hkv * 100 + page_size * 10 + head_dim + causal)
    q1 = int(torch.randint(1, 15, (1,), generator=g))
    kv1 = int(torch.randint(15, 257, (1,), generator=g))
    q2 = int(torch.randint(1, 64, (1,), generator=g))
    for n_q, kv_len in ((q1, kv1), (q2, q2), (63, 2047)):
        case = PagedCase(kv_len, hkv, head_dim, page_size, dtype, seed=kv_len + n_q + hkv)
        q = randn((n_q, hq, head_dim), n_q * 7 + kv_len, dtype)
        want = _dense(q, case.k, case.v, causal)
        got = _run(cuda, case, q, causal, dtype)
        assert ((got.float().cpu() - want).abs() <= ATOL[dtype] * want.abs().clamp(min=1.0)).all(), \
            (n_q, kv_len)


def test_prefill_at_benchmark_length(cuda):
    """32768 tokens, Llama-2-7B head shape (4 of the 32 heads, GQA 4/2): checked on sampled rows
    against the oracle's single-query attention over the row's causal prefix."""
    from oracle import tidal_oracle as orc

    dtype, n, hq, hkv, d, page = torch.bfloat16, 32768, 4, 2, 128, 16
    case = PagedCase(n, hkv, d, page, dtype, seed=5)
    q = randn((n, hq, d), 6, dtype)
    got = _run(cuda, case, q, True, dtype).float().cpu()
    for row in (0, 1, 127, 128, 4095, 20000, 32767):
        want = orc.softmax_pv(orc.attn_logits(q[row], case.k[: row + 1]), case.v[: row + 1])
        assert (got[row] - want).abs().max() <= ATOL[dtype] * max(1.0, want.abs().max().item()), row


def test_prefill_errors(cuda):
    from tidaldecode_amd import _kernels

    pool = torch.zeros((4, 2, 16, 2, 128), dtype=torch.float16, device=cuda)
    table = torch.arange(2, dtype=torch.int32, device=cuda)
    q = torch.zeros((40, 4, 128), dtype=torch.float16, device=cuda)
    with pytest.raises(RuntimeError):   # 40 queries, 20 cached tokens
        _kernels.prefill_with_paged_kv_cache(q, pool, table, 4, True, 0, False, 1.0, 1e4)
    with pytest.raises(RuntimeError):   # 3 query heads over 2 KV heads
        _kernels.prefill_with_paged_kv_cache(q[:8, :3].contiguous(), pool, table, 16, True, 0,
                                             False, 1.0, 1e4)
    with pytest.raises(RuntimeError, match="failed to dispatch"):   # head_dim without a kernel
        _kernels.prefill_with_paged_kv_cache(
            torch.zeros((4, 2, 32), dtype=torch.float16, device=cuda),
            torch.zeros((4, 2, 16, 2, 32), dtype=torch.float16, device=cuda), table, 16, True, 0,
            False, 1.0, 1e4)
    with pytest.raises(RuntimeError):   # dtype mismatch
        _kernels.prefill_with_paged_kv_cache(q[:8].bfloat16(), pool, table, 16, True, 0, False,
                                             1.0, 1e4)


@pytest.mark.parametrize("seed", range(16))
def test_random_configurations(cuda, seed):
    """Seeded random draws over head counts (incl. the 8-KV-head placement path and the eight-wave
    workgroups above 128 query rows), head_dim, page size, layout, dtype, causal, cache and query
    lengths."""
    import random

    rnd = random.Random(500 + seed)
    dtype = rnd.choice([torch.float16, torch.bfloat16])
    d = rnd.choice([64, 128, 128, 128, 256])
    hkv = rnd.choice([1, 2, 3, 8])
    hq = hkv * rnd.choice([1, 2, 4])
    page = rnd.choice([1, 3, 4, 8, 16, 16, 32])
    layout = rnd.choice([0, 1])
    causal = rnd.random() < 0.75
    kv_len = rnd.choice([1, 31, 64, 129, 257, 700, 1500, 2100])
    n_q = rnd.randint(1, kv_len)
    case = PagedCase(kv_len, hkv, d, page, dtype, layout=layout, seed=seed + 7)
    q = randn((n_q, hq, d), seed + 31, dtype)
    want = _dense(q, case.k, case.v, causal)
    got = _run(cuda, case, q, causal, dtype)
    ok = (got.float().cpu() - want).abs() <= ATOL[dtype] * want.abs().clamp(min=1.0)
    assert ok.all(), (dtype, d, hq, hkv, page, layout, causal, kv_len, n_q)

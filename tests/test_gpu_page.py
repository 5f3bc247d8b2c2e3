"""GPU parity: RoPE, paged append (with the per-page key max/min metadata), their fusion, RMSNorm.

RoPE tolerance.  The GPU forms the angle in float64 and rounds only sin/cos, so it is compared with
the float64 closed form; the error budget is one rounding of the output dtype plus fp32 evaluation
of x*cos +- y*sin: |err| <= 2^-11 |y| (fp16) / 2^-8 |y| (bf16) + 1e-6.  The reference's two own
fp32 formulas (cpu_reference.h:36-53 and the model's, llama_tidaldecoding.py:248-279) differ from
that closed form by up to position * 2^-23 rad; test_rope_reference_formulas_within_their_own_error
checks both stay inside that bound at the positions the benchmark uses.
Append must be bit-exact (copies); max/min metadata bit-exact against brute force.
"""
import numpy as np
import pytest
import torch

from _util import ATOL, PagedCase, randn

pytestmark = pytest.mark.gpu

ULP = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}


def _rope_tol(want, dtype):
    return ULP[dtype] * want.abs() * 1.01 + 2e-6


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("d", [64, 128, 256])
@pytest.mark.parametrize("past,n_tok,theta,scale", [(0, 1, 1e4, 1.0), (4095, 1, 1e4, 1.0),
                                                    (32767, 1, 1e4, 1.0), (102399, 1, 5e5, 1.0),
                                                    (0, 300, 1e4, 1.0), (1000, 17, 5e5, 4.0)])
def test_rope_in_place_against_closed_form(cuda, dtype, d, past, n_tok, theta, scale):
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    hq, hkv = 32, 8
    q = randn((n_tok, hq, d), past + d, dtype)
    k = randn((n_tok, hkv, d), past + d + 1, dtype)
    pos = np.arange(past, past + n_tok)
    want_q = torch.from_numpy(orc.rope_closed_form(q.numpy(), pos, theta, scale))
    want_k = torch.from_numpy(orc.rope_closed_form(k.numpy(), pos, theta, scale))
    qd, kd = q.to(dtype).to(cuda), k.to(dtype).to(cuda)
    _kernels.apply_rope_in_place(qd, kd, past, scale, theta)
    torch.cuda.synchronize()
    assert ((qd.double().cpu() - want_q).abs() <= _rope_tol(want_q, dtype)).all()
    assert ((kd.double().cpu() - want_k).abs() <= _rope_tol(want_k, dtype)).all()


def test_rope_invariants(cuda):
    """position 0 is the identity; pair norms are preserved; q_m . k_n depends on m - n only."""
    from tidaldecode_amd import _kernels

    dtype, d = torch.float16, 128
    q = randn((1, 4, d), 1, dtype).to(dtype).to(cuda)
    k = randn((1, 4, d), 2, dtype).to(dtype).to(cuda)
    q0, k0 = q.clone(), k.clone()
    _kernels.apply_rope_in_place(q, k, 0, 1.0, 1e4)
    assert torch.equal(q, q0) and torch.equal(k, k0)
    dots = []
    for m, n in ((10, 3), (1010, 1003), (30010, 30003)):
        qa, kb = q0.clone(), k0.clone()
        dummy = torch.zeros_like(k0)
        _kernels.apply_rope_in_place(qa, dummy, m, 1.0, 1e4)
        dummy = torch.zeros_like(q0)
        _kernels.apply_rope_in_place(dummy, kb, n, 1.0, 1e4)
        dots.append((qa.float() * kb.float()).sum(-1))
        pair = lambda x: x.float()[..., : d // 2] ** 2 + x.float()[..., d // 2:] ** 2
        assert (pair(qa) - pair(q0)).abs().max() < 2e-2
    assert (dots[0] - dots[1]).abs().max() < 0.1 and (dots[0] - dots[2]).abs().max() < 0.1


def _append_case(cuda, dtype, layout, page_size, seq_before, n_new, d=128, h=8, with_meta=True):
    """Append n_new tokens to a sequence holding seq_before tokens; returns device pools + oracle."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    seq_after = seq_before + n_new
    case = PagedCase(seq_after, h, d, page_size, dtype, layout=layout, seed=seq_after + page_size)
    # pool as it was before the append: oracle-append of the first seq_before tokens into garbage
    shape = orc.pool_shape(case.max_pages, page_size, h, d, layout)
    before = np.full(shape, 33.0, dtype=np.float32)
    if seq_before:
        orc.paged_append(before, case.page_table.tolist(), seq_before, case.k[:seq_before].numpy(),
                         case.v[:seq_before].numpy(), layout)
    want = before.copy()
    orc.paged_append(want, case.page_table.tolist(), seq_after, case.k[seq_before:].numpy(),
                     case.v[seq_before:].numpy(), layout)
    pool = torch.from_numpy(before).to(dtype).to(cuda)
    indices = case.page_table.to(torch.int32).to(cuda)
    indptr = torch.tensor([0, case.n_pages], dtype=torch.int32, device=cuda)
    # metadata pool: one entry per KV page, same page size; state before = brute force over the
    # tokens already present
    n_meta_pages = (case.n_pages + page_size - 1) // page_size
    meta_table = torch.randperm(n_meta_pages + 2, generator=torch.Generator().manual_seed(1))[:n_meta_pages]
    meta_shape = orc.pool_shape(n_meta_pages + 2, page_size, h, d, layout)
    meta_before = np.full(meta_shape, 9.0, dtype=np.float32)
    meta_want = None
    if with_meta:
        def brute(upto):
            m = np.full(meta_shape, 9.0, dtype=np.float32)
            for pg in range((upto + page_size - 1) // page_size):
                rows = case.k[pg * page_size: min(upto, (pg + 1) * page_size)].numpy()
                mp, me = int(meta_table[pg // page_size]), pg % page_size
                if layout == 1:
                    m[mp, 0, :, me, :], m[mp, 1, :, me, :] = rows.max(0), rows.min(0)
                else:
                    m[mp, 0, me, :, :], m[mp, 1, me, :, :] = rows.max(0), rows.min(0)
            return m
        meta_before = brute(seq_before)
        meta_want = brute(seq_after)
    meta = torch.from_numpy(meta_before).to(dtype).to(cuda)
    fn = _kernels.append_kv_cache_decode if n_new == 1 else _kernels.append_kv_cache_prefill
    kd = case.k[seq_before:].to(dtype).to(cuda).contiguous()
    vd = case.v[seq_before:].to(dtype).to(cuda).contiguous()
    fn(kd, vd, pool, indices, indptr, case.last_page_len, int(case.page_table[-1]),
       meta if with_meta else torch.empty(0, device=cuda), meta_table.to(torch.int32).to(cuda),
       torch.tensor([0, n_meta_pages], dtype=torch.int32, device=cuda),
       (case.n_pages - 1) % page_size + 1, int(meta_table[-1]), layout)
    torch.cuda.synchronize()
    return pool.float().cpu().numpy(), want, meta.float().cpu().numpy(), meta_want


@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("page_size", [1, 3, 7, 16, 31])
def test_append_decode_and_prefill_bit_exact(cuda, layout, page_size):
    """page sizes and lengths of the reference's page test (kernels/src/test/test_page.cu:620-684)"""
    for dtype in (torch.float16, torch.bfloat16):
        for seq_before, n_new in ((0, 17), (16, 1), (0, 1), (30, 1), (31, 1), (5, 250), (100, 4000 // 16),
                                  (4099, 1)):
            got, want, mgot, mwant = _append_case(cuda, dtype, layout, page_size, seq_before, n_new)
            assert np.array_equal(got, want), (layout, page_size, dtype, seq_before, n_new)
            assert np.array_equal(mgot, mwant), ("metadata", layout, page_size, dtype, seq_before, n_new)


def test_multi_turn_append_round_trip(cuda):
    """alternate prefill (<= 256 tokens) and decode appends, then gather through the page table
    equals the contiguous K, V (test_page.cu multi-turn case)."""
    from tidaldecode_amd import _kernels

    dtype, h, d, page_size = torch.float16, 8, 128, 7
    g = torch.Generator().manual_seed(3)
    chunks = []
    for i in range(10):
        chunks.append(int(torch.randint(1, 257, (1,), generator=g)) if i % 2 == 0 else 1)
    total = sum(chunks)
    case = PagedCase(total, h, d, page_size, dtype, seed=77)
    pool = torch.full(case.pool.shape, 5.0, dtype=dtype, device=cuda)
    empty = torch.empty(0, device=cuda)
    done = 0
    for n_new in chunks:
        done += n_new
        n_pages = (done + page_size - 1) // page_size
        idx = case.page_table[:n_pages].to(torch.int32).to(cuda)
        indptr = torch.tensor([0, n_pages], dtype=torch.int32, device=cuda)
        kd = case.k[done - n_new: done].to(dtype).to(cuda).contiguous()
        vd = case.v[done - n_new: done].to(dtype).to(cuda).contiguous()
        fn = _kernels.append_kv_cache_decode if n_new == 1 else _kernels.append_kv_cache_prefill
        fn(kd, vd, pool, idx, indptr, (done - 1) % page_size + 1, int(idx[-1]), empty, idx, indptr,
           1, 0, 0)
    torch.cuda.synchronize()
    pages = pool[case.page_table.to(cuda)]
    kk = pages[:, 0].reshape(-1, h, d)[:total].float().cpu()
    vv = pages[:, 1].reshape(-1, h, d)[:total].float().cpu()
    assert torch.equal(kk, case.k) and torch.equal(vv, case.v)


def test_fused_rope_append_keeps_a_bad_slot_inside_the_pool(cuda):
    """A destination slot beyond the pool is written into the pool's last page (the clamp the
    attention launch applies as well) and nowhere else."""
    from tidaldecode_amd import _kernels

    dtype, hq, hkv, d, page_size, pages = torch.float16, 8, 8, 128, 16, 4
    pool = torch.full((pages, 2, page_size, hkv, d), 3.0, dtype=dtype, device=cuda)
    q = randn((1, hq, d), 1, dtype).to(dtype).to(cuda)
    k = randn((1, hkv, d), 2, dtype).to(dtype).to(cuda)
    v = randn((1, hkv, d), 3, dtype).to(dtype).to(cuda)
    pos = torch.zeros(1, dtype=torch.int32, device=cuda)           # position 0: the rotation is the identity
    bad = torch.tensor([1000 * page_size + 5], dtype=torch.int32, device=cuda)
    _kernels.rope_append_decode(q, k, v, pool, pos, bad, 0, 1.0, 1e4)
    torch.cuda.synchronize()
    assert (pool[: pages - 1] == 3.0).all()
    assert torch.equal(pool[pages - 1, 0, 5], k[0]) and torch.equal(pool[pages - 1, 1, 5], v[0])
    untouched = torch.ones(page_size, dtype=torch.bool)
    untouched[5] = False
    assert (pool[pages - 1][:, untouched] == 3.0).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", [0, 1])
def test_fused_rope_append_equals_the_two_calls(cuda, dtype, layout):
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    b, hq, hkv, d, page_size, pages = 5, 32, 8, 128, 16, 40
    theta, scale = 5e5, 1.0
    q = randn((b, hq, d), 1, dtype)
    k = randn((b, hkv, d), 2, dtype)
    v = randn((b, hkv, d), 3, dtype)
    positions = torch.tensor([0, 15, 16, 333, 100000], dtype=torch.int32)
    slots = torch.tensor([7 * 16 + 0, 2 * 16 + 15, 39 * 16 + 0, 11 * 16 + 13, 0 * 16 + 1], dtype=torch.int32)
    shape = orc.pool_shape(pages, page_size, hkv, d, layout)
    pool = torch.full(shape, 3.0, dtype=dtype, device=cuda)
    qd = q.to(dtype).to(cuda)
    _kernels.rope_append_decode(qd, k.to(dtype).to(cuda), v.to(dtype).to(cuda), pool,
                                positions.to(cuda), slots.to(cuda), layout, scale, theta)
    torch.cuda.synchronize()
    want_pool = np.full(shape, 3.0, dtype=np.float32)
    for i in range(b):
        qi, ki = q[i:i + 1].to(dtype).to(cuda), k[i:i + 1].to(dtype).to(cuda)
        _kernels.apply_rope_in_place(qi, ki, int(positions[i]), scale, theta)
        assert torch.equal(qi[0], qd[i])
        page, entry = int(slots[i]) // page_size, int(slots[i]) % page_size
        if layout == 1:
            want_pool[page, 0, :, entry, :] = ki[0].float().cpu().numpy()
            want_pool[page, 1, :, entry, :] = v[i].numpy()
        else:
            want_pool[page, 0, entry, :, :] = ki[0].float().cpu().numpy()
            want_pool[page, 1, entry, :, :] = v[i].numpy()
    assert np.array_equal(pool.float().cpu().numpy(), want_pool)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,cols", [(1, 4096), (7, 5120), (300, 128), (2, 33), (1, 8), (5, 2056),
                                       (3, 8192), (2, 16384), (2, 16392), (3, 20000)])
def test_rms_norm(cuda, dtype, rows, cols):
    from tidaldecode_amd import _kernels

    x = randn((1, rows, cols), rows + cols, dtype)
    w = randn((cols,), cols, dtype)
    want = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + 1e-5) * w
    out = torch.empty((1, rows, cols), dtype=dtype, device=cuda)
    _kernels.rms_norm_forward(x.to(dtype).to(cuda), w.to(dtype).to(cuda), out, 1e-5)
    torch.cuda.synchronize()
    assert ((out.float().cpu() - want).abs() <= ULP[dtype] * 1.01 * want.abs() + 1e-6).all()
    # the same rows at an address that is not 16-byte aligned (2-byte access path)
    flat = torch.zeros(rows * cols + 8, dtype=dtype, device=cuda)
    flat[4:4 + rows * cols] = x.to(dtype).to(cuda).flatten()
    out2 = torch.empty_like(out)
    _kernels.rms_norm_forward(flat[4:4 + rows * cols].view(1, rows, cols), w.to(dtype).to(cuda), out2,
                              1e-5)
    torch.cuda.synchronize()
    assert ((out2.float().cpu() - want).abs() <= ULP[dtype] * 1.01 * want.abs() + 1e-6).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,d,page,layout", [(32, 32, 128, 16, "NHD"), (8, 2, 64, 4, "HND"),
                                                  (4, 4, 256, 7, "NHD"), (32, 8, 128, 32, "NHD")])
def test_page_score_estimator(cuda, dtype, hq, hkv, d, page, layout):
    """decode_estimate over the metadata the append kernels keep (prefill append, then decode
    appends) against the oracle's bound on the same rounded keys; sequence lengths of the
    reference's estimator test (kernels/src/test/test_max_possible.cu:158)."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import utils as ops
    from tidaldecode_amd.utils import InferenceController

    for n in (65, 213, 1110):
        c = InferenceController(1, hq, d, page, 64, 4096, dtype, cuda, num_kv_heads=hkv,
                                kv_layout=layout, with_metadata=True, page_order_seed=2)
        gk = torch.Generator().manual_seed(n)
        k = torch.randn((n + 3, hkv, d), generator=gk).to(dtype)
        v = torch.randn((n + 3, hkv, d), generator=gk).to(dtype)
        c.prepare_metadata(n)
        c.begin_forward(n)
        ops.append_kv(k[:n].to(cuda), v[:n].to(cuda), c, 0)
        c.end_forward()
        for i in range(n, n + 3):
            c.prepare_metadata(1)
            c.begin_forward(1)
            ops.append_kv(k[i:i + 1].to(cuda), v[i:i + 1].to(cuda), c, 0)
            c.end_forward()
        q = torch.randn((1, hq, d), generator=gk).to(dtype)
        got = ops.decode_estimate(q.to(cuda), c, 0)
        torch.cuda.synchronize()
        want = orc.page_score_bound(q[0].float(), k.float(), page)
        n_pages = (n + 3 + page - 1) // page
        assert got.shape == (hq, n_pages - 1)            # the page being filled is left out
        want = want[:, : n_pages - 1]
        tol = (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7) * want.abs().clamp(min=1.0) + 1e-3
        assert ((got.float().cpu() - want).abs() <= tol).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,page,n,budget", [(32, 32, 16, 4099, 300), (8, 2, 4, 1110, 40)])
def test_selection_step_with_logits_in_the_kv_dtype(cuda, dtype, hq, hkv, page, n, budget):
    """InferenceController(logits_dtype=<KV dtype>): the reference's buffer type
    (tidal/utils/controller.py:149-151).  decode_sparse_attn over the whole cache stores the logits
    rounded to that type, decode_topk ranks the stored values (bit-exact against the oracle's
    stable top-k of the same values, through the page table), and a sparse layer over the chosen
    slots matches the oracle's attention over those tokens."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import utils as ops
    from tidaldecode_amd.utils import InferenceController

    d = 128
    with pytest.raises(ValueError, match="logits_dtype"):
        InferenceController(1, hq, d, page, budget, n + 64, dtype, cuda, logits_dtype=torch.float64)
    c = InferenceController(1, hq, d, page, budget, n + 64, dtype, cuda, num_kv_heads=hkv,
                            page_order_seed=4, logits_dtype=dtype)
    assert c.qk_product.dtype == dtype
    g = torch.Generator().manual_seed(n + budget)
    k = torch.randn((n, hkv, d), generator=g).to(dtype)
    v = torch.randn((n, hkv, d), generator=g).to(dtype)
    q = torch.randn((1, hq, d), generator=g).to(dtype)
    c.prepare_metadata(n - 1)
    c.begin_forward(n - 1)
    ops.append_kv(k[:n - 1].to(cuda), v[:n - 1].to(cuda), c, 0)
    c.end_forward()
    c.prepare_metadata(1)
    c.begin_forward(1)
    ops.append_kv(k[n - 1:].to(cuda), v[n - 1:].to(cuda), c, 0)
    o = ops.decode_sparse_attn(q.to(cuda), c, 0, c.kv_indices_without_last, True)
    ops.decode_topk(c)
    o2 = ops.decode_sparse_attn(q.to(cuda), c, 0, c.topk_dindices_buffer, False)
    torch.cuda.synchronize()
    logits = orc.attn_logits(q[0], k)
    assert (o[0].float().cpu() - orc.softmax_pv(logits, v)).abs().max() <= ATOL[dtype]
    stored = c.qk_product[:, :n].float().cpu()
    step = (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7) * logits.abs().clamp_min(2.0 ** -14)
    assert ((stored - logits).abs() <= step + 2e-4).all()
    pos = orc.stable_topk(stored, budget)
    table = c.kv_cache.indices_device.cpu().long()
    got = c.topk_dindices_buffer[:, :budget].cpu().long()
    assert torch.equal(got, table[pos // page] * page + pos % page)
    assert (o2[0].float().cpu() - orc.sparse_layer_gather(q[0], k, v, pos)).abs().max() <= ATOL[dtype]
    c.clean_states()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,page,n,budget", [(32, 32, 16, 4099, 32), (8, 2, 4, 1110, 40),
                                                  (4, 4, 16, 213, 5)])
def test_quest_style_step(cuda, dtype, hq, hkv, page, n, budget):
    """The page-selection step of the reference's ancestor built from the library's pieces, as
    bench.py times it: decode_estimate (upper bound of the logits per page) -> topk_filtering over
    the bounds with the physical page of each position as payload -> attention over the chosen
    pages plus the page being filled.  The chosen pages are bit-exact against the oracle's stable
    top-k of the oracle's bound on the same rounded scores, the attention output against the
    oracle's attention over the tokens of those pages."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels
    from tidaldecode_amd import utils as ops
    from tidaldecode_amd.utils import InferenceController

    d = 128
    c = InferenceController(1, hq, d, page, 64, n + 64, dtype, cuda, num_kv_heads=hkv,
                            with_metadata=True, page_order_seed=3)
    g = torch.Generator().manual_seed(n + budget)
    k = torch.randn((n, hkv, d), generator=g).to(dtype)
    v = torch.randn((n, hkv, d), generator=g).to(dtype)
    q = torch.randn((1, hq, d), generator=g).to(dtype)
    c.prepare_metadata(n - 1)
    c.begin_forward(n - 1)
    ops.append_kv(k[:n - 1].to(cuda), v[:n - 1].to(cuda), c, 0)
    c.end_forward()
    c.prepare_metadata(1)
    c.begin_forward(1)
    ops.append_kv(k[n - 1:].to(cuda), v[n - 1:].to(cuda), c, 0)
    est = ops.decode_estimate(q.to(cuda), c, 0)                       # [hq, n_pages - 1]
    n_pages = (n + page - 1) // page
    assert est.shape == (hq, n_pages - 1) and budget <= n_pages - 1
    page_ids = c.kv_indices_without_last.expand(hq, -1).contiguous()
    chosen = torch.full((hq, budget), -1, dtype=torch.int32, device=cuda)
    _kernels.topk_filtering(est, page_ids, None, chosen, c.topk_buf, budget)
    o = torch.empty_like(q, device=cuda)
    c._decode_handler.forward(q.to(cuda), o, c.kv_cache.buf_layer(0), chosen, None,
                              c.kv_cache.last_page_len, c.kv_last_page_idx, None, index_kind="pages")
    torch.cuda.synchronize()
    # the bound itself (fp32 oracle on the rounded keys), then the selection on the GPU's own scores
    bound = orc.page_score_bound(q[0].float(), k.float(), page)[:, : n_pages - 1]
    tol = (2.0 ** -10 if dtype == torch.float16 else 2.0 ** -7) * bound.abs().clamp(min=1.0) + 1e-3
    assert ((est.float().cpu() - bound).abs() <= tol).all()
    logical = orc.stable_topk(est.float().cpu(), budget)              # [hq, budget] logical pages
    table = c.kv_cache.indices_device.cpu().long()
    assert torch.equal(chosen.cpu().long(), table[logical])
    # attention over the tokens of the chosen pages and of the last page
    want = torch.empty((hq, d))
    last = torch.arange((n_pages - 1) * page, n)
    for h in range(hq):
        tok = torch.cat([(logical[h][:, None] * page + torch.arange(page)[None]).flatten(), last])
        kh, vh = k[tok, h // (hq // hkv)].float(), v[tok, h // (hq // hkv)].float()
        p = torch.softmax(kh @ q[0, h].float() / d ** 0.5, 0)
        want[h] = p @ vh
    tol_o = 2e-3 if dtype == torch.float16 else 1e-2
    assert (o[0].float().cpu() - want).abs().max().item() <= tol_o
    c.clean_states()


@pytest.mark.parametrize("head_dim", [64, 128])
@pytest.mark.parametrize("page_size", [1, 3, 7, 16, 32])
def test_page_score_estimator_reference_grid(cuda, head_dim, page_size):
    """The reference's estimator test grid (kernels/src/test/test_max_possible.cu:158-165: ten
    sequence lengths x five page sizes x two head dims, 32 heads, fp16) at the kernel boundary:
    the metadata pool is filled with the brute-force per-page key max / min."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    h, dtype = 32, torch.float16
    for n in (65, 127, 213, 1110, 2000, 4099, 8192, 8222, 12345, 28837):
        g = torch.Generator().manual_seed(n * 31 + page_size)
        k = torch.randn((n, h, head_dim), generator=g).to(dtype)
        q = torch.randn((1, h, head_dim), generator=g).to(dtype)
        n_kv_pages = (n + page_size - 1) // page_size            # one metadata entry per KV page
        n_meta_pages = (n_kv_pages + page_size - 1) // page_size
        pad = n_kv_pages * page_size - n
        kf = k.float()
        mx = torch.cat([kf, torch.full((pad, h, head_dim), -65504.0)]).view(n_kv_pages, page_size, h, head_dim).max(1).values
        mn = torch.cat([kf, torch.full((pad, h, head_dim), 65504.0)]).view(n_kv_pages, page_size, h, head_dim).min(1).values
        table = torch.randperm(n_meta_pages + 2, generator=g)[:n_meta_pages]
        meta = torch.full((n_meta_pages + 2, 2, page_size, h, head_dim), 7.0)
        epad = n_meta_pages * page_size - n_kv_pages
        meta[table, 0] = torch.cat([mx, torch.zeros(epad, h, head_dim)]).view(n_meta_pages, page_size, h, head_dim)
        meta[table, 1] = torch.cat([mn, torch.zeros(epad, h, head_dim)]).view(n_meta_pages, page_size, h, head_dim)
        last_len = (n_kv_pages - 1) % page_size + 1
        n_out = n_kv_pages - 1
        o = torch.full((h, max(n_out, 1)), float("nan"), dtype=dtype, device=cuda)
        _kernels.estimate_attn_score(q.to(cuda), o, meta.to(dtype).to(cuda),
                                     table.to(torch.int32).to(cuda), None, last_len,
                                     int(table[-1]), 0)
        torch.cuda.synchronize()
        if n_out == 0:
            continue
        want = orc.page_score_bound(q[0].float(), kf, page_size)[:, :n_out]
        tol = 2.0 ** -10 * want.abs().clamp(min=1.0) + 1e-3
        assert ((o[:, :n_out].float().cpu() - want).abs() <= tol).all(), (n, page_size, head_dim)

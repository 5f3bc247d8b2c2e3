"""GPU parity of the short-list decode-attention kernel (csrc/sparse_attn.cuh), the launch that
serves TidalDecode's sparse layers: every workgroup shape, both dtypes, list lengths around the
tile edges, the forced last page, several tiles per wave, both merge paths, grouped queries with
per-query-head lists, the HND layout, ragged batches whose lengths live on the device, and the
fused decode step.  Each case is checked against the CPU oracle (max-abs 2e-3 fp16 / 1e-2 bf16)
and against the streaming kernel on the same inputs (the two must agree far inside that bound).
Semantics: kernels/include/decode/decode_attn.cuh:432-658, decode_page.cuh:320-346 of the
reference."""
import numpy as np
import pytest
import torch

from _util import ATOL, PagedCase, randn, rotated, tolerance_report, within_ulps

pytestmark = pytest.mark.gpu

SHAPES = [(8, 8), (4, 8), (4, 16), (8, 16)]


def _wrapper(layout, hq, hkv, d, page, dtype, **knobs):
    from tidaldecode_amd import _kernels

    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(layout)
    for key, val in knobs.items():
        setattr(w, key, val)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    return w


def _uses_short_list_kernel(w, batch, rows, items):
    return w._plan(batch, rows, items).sparse_waves > 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sw,sr", SHAPES)
def test_list_lengths_around_the_tile_edges(cuda, dtype, sw, sr):
    """k = 1 ... a few tiles: one split and many, full and ragged last tiles, lse out."""
    from oracle import tidal_oracle as orc

    h, d, page, n = 8, 128, 16, 5000
    tile = sw * 4 * sr
    case = PagedCase(n, h, d, page, dtype, seed=sw * 100 + sr)
    pool = case.pool.to(cuda)
    q = randn((h, d), 7, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    w = _wrapper(0, h, h, d, page, dtype, sparse_waves=sw, sparse_rows=sr)
    gen = _wrapper(0, h, h, d, page, dtype, sparse_waves=-1)
    g = torch.Generator().manual_seed(1)
    for k in [1, 2, 4 * sr - 1, 4 * sr, 4 * sr + 1, tile - 1, tile, tile + 1, 2 * tile + 3, 1000, 2048,
              4096 + 37]:
        assert _uses_short_list_kernel(w, 1, h, k) and not _uses_short_list_kernel(gen, 1, h, k)
        pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(h)])
        want = orc.sparse_layer_gather(q, case.k, case.v, pos)
        slots = case.slots_of(pos).to(torch.int32).to(cuda)
        od = torch.full_like(qd, float("nan"))
        lse = torch.full((1, h), float("nan"), dtype=torch.float32, device=cuda)
        w.forward(qd, od, pool, slots, None, 0, 0, None, index_kind="slots", lse=lse)
        og = torch.full_like(qd, float("nan"))
        gen.forward(qd, og, pool, slots, None, 0, 0, None, index_kind="slots")
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want) <= ATOL[dtype], (k, sw, sr)
        assert (od.float() - og.float()).abs().max().item() <= ATOL[dtype] / 4, (k, sw, sr)
        logits = orc.attn_logits(q, case.k)
        want_lse = torch.logsumexp(torch.gather(logits, 1, pos), -1)
        assert (lse[0].cpu() - want_lse).abs().max() <= 1e-3, k


@pytest.mark.parametrize("sw,sr", SHAPES)
@pytest.mark.parametrize("knobs", [dict(chunk_tokens=1024), dict(fused_merge=0),
                                   dict(chunk_tokens=2048, fused_merge=0), dict(chunk_tokens=16384)])
def test_several_tiles_per_wave_and_both_merges(cuda, sw, sr, knobs):
    """Chunks of several workgroup tiles (every wave loops) and the second-launch merge; repeated
    calls reuse the ticket counters and the partial buffers."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page, n, k = torch.bfloat16, 16, 128, 16, 9000, 3000
    case = PagedCase(n, h, d, page, dtype, seed=11)
    q = randn((h, d), 12, dtype)
    g = torch.Generator().manual_seed(13)
    pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(h)])
    want = orc.sparse_layer_gather(q, case.k, case.v, pos)
    slots = case.slots_of(pos).to(torch.int32).to(cuda)
    w = _wrapper(0, h, h, d, page, dtype, sparse_waves=sw, sparse_rows=sr, **knobs)
    assert _uses_short_list_kernel(w, 1, h, k)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    pool = case.pool.to(cuda)
    for _ in range(3):
        od = torch.full_like(qd, float("nan"))
        w.forward(qd, od, pool, slots, None, 0, 0, None, index_kind="slots")
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want) <= ATOL[dtype], knobs


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("hq,hkv,rows", [(8, 8, 8), (8, 8, 1), (16, 4, 16), (16, 8, 16), (32, 2, 32)])
def test_forced_last_page_layouts_and_grouped_queries(cuda, dtype, layout, hq, hkv, rows):
    """Slot lists followed by the first last_page_len entries of the newest page (the reference's
    forced last page, decode_page.cuh:326-329), NHD and HND pools, one list per query head under
    grouped queries (the KV head of a list walk is hrow / group) and one shared list."""
    from oracle import tidal_oracle as orc

    d, page, n = 128, 16, 2000 + 5           # 5 tokens in the last page
    case = PagedCase(n, hkv, d, page, dtype, layout=layout, seed=hq + rows + layout)
    q = randn((hq, d), 3, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    pool = case.pool.to(cuda)
    before_last = (case.n_pages - 1) * page
    g = torch.Generator().manual_seed(2)
    w = _wrapper(layout, hq, hkv, d, page, dtype)
    for k in (0, 1, 63, 300):
        pos = torch.stack([torch.randperm(before_last, generator=g)[:k] for _ in range(rows)]) \
            if k else torch.zeros((rows, 0), dtype=torch.long)
        assert _uses_short_list_kernel(w, 1, rows, k + case.last_page_len)
        slots = case.slots_of(pos).to(torch.int32)
        want, _ = orc.paged_selected_attention(q.numpy(), case.pool_np, slots.numpy(),
                                               int(case.page_table[-1]), case.last_page_len,
                                               layout=layout, kind="slots")
        # the same thing said on the contiguous cache: listed tokens + the tokens of the last page
        allpos = torch.cat([pos, torch.arange(before_last, n).repeat(rows, 1)], 1)
        want2 = orc.sparse_layer_gather(q, case.k, case.v, allpos)
        assert (torch.from_numpy(want) - want2).abs().max() < 1e-5
        od = torch.full_like(qd, float("nan"))
        w.forward(qd, od, pool, slots.to(cuda).contiguous(), None, case.last_page_len,
                  int(case.page_table[-1]), None, index_kind="slots")
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want2) <= ATOL[dtype], (k, layout, rows)


@pytest.mark.parametrize("counts_kind", ["indptr", "padded"])
def test_ragged_batch_with_lengths_on_the_device(cuda, counts_kind):
    """Eight sequences in one pool: list segments through indptr (packed) or indptr + counts (padded
    table), last-page fill and id per sequence as device arrays -- the state words the kernel
    fetches through the scalar cache."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page = torch.float16, 8, 128, 16
    g = torch.Generator().manual_seed(0)
    lens = torch.randint(300, 4000, (8,), generator=g).tolist()
    ks = [int(x) for x in torch.randint(0, 700, (8,), generator=g)]
    ks[3] = 0                                      # a sequence with nothing but its last page
    cases = [PagedCase(n, h, d, page, dtype, seed=70 + i, spare=1) for i, n in enumerate(lens)]
    offs = np.cumsum([0] + [c.max_pages for c in cases])
    pool = torch.cat([c.pool for c in cases]).to(cuda)
    q = randn((8, h, d), 9, dtype)
    width = max(ks) + 3
    rows, wants = [], []
    for i, c in enumerate(cases):
        before_last = (c.n_pages - 1) * page
        pos = torch.stack([torch.randperm(before_last, generator=g)[: ks[i]] for _ in range(h)])
        allpos = torch.cat([pos, torch.arange(before_last, c.n).repeat(h, 1)], 1)
        wants.append(orc.sparse_layer_gather(q[i], c.k, c.v, allpos))
        rows.append((c.slots_of(pos) + int(offs[i]) * page).to(torch.int32))
    if counts_kind == "indptr":
        idx = torch.cat(rows, 1).contiguous()
        indptr = torch.tensor([0] + list(np.cumsum(ks)), dtype=torch.int32, device=cuda)
        counts = None
    else:
        idx = torch.full((h, 8 * width), 2**30, dtype=torch.int32)   # padding would be out of range
        for i, r in enumerate(rows):
            idx[:, i * width: i * width + ks[i]] = r
        indptr = torch.arange(0, 9 * width, width, dtype=torch.int32, device=cuda)
        counts = torch.tensor(ks, dtype=torch.int32, device=cuda)
    ll = torch.tensor([c.last_page_len for c in cases], dtype=torch.int32, device=cuda)
    li = torch.tensor([int(c.page_table[-1]) + int(offs[i]) for i, c in enumerate(cases)],
                      dtype=torch.int32, device=cuda)
    w = _wrapper(0, h, h, d, page, dtype)
    assert _uses_short_list_kernel(w, 8, h, max(ks) + page)
    qd = q.to(dtype).to(cuda)
    od = torch.full_like(qd, float("nan"))
    w.forward(qd, od, pool, idx.to(cuda), indptr, ll, li, None, index_kind="slots", n_list=max(ks),
              counts=counts)
    torch.cuda.synchronize()
    for i in range(8):
        assert tolerance_report(od[i], wants[i]) <= ATOL[dtype], i


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sw,sr", SHAPES)
def test_fused_decode_step(cuda, dtype, sw, sr):
    """RoPE + append inside the launch: the new token's slot sits somewhere in every list (so some
    wave of every head takes it from registers), the cache gets the rotated key exactly once, and
    the output equals the oracle's attention over float64-rotated, storage-rounded q and K as
    well as separate RoPE/append launches followed by the same attention (the two GPU paths share
    every rounding but that of the rotated key).  The last case is the benchmark's head row:
    32 heads x 2048 tokens."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    d, page, n, b = 128, 16, 1500, 2
    theta = 1e4
    for h, k in ((8, 1), (8, 4 * sr + 1), (8, 700), (32, 2048)):
        n = 1500 if k < 1000 else 5000
        cases = [PagedCase(n, h, d, page, dtype, seed=40 + i, spare=0, shuffle=False) for i in range(b)]
        npg = cases[0].n_pages
        pool = torch.cat([c.pool for c in cases]).to(cuda)
        offs = [0, npg]
        q = randn((b, h, d), 1, dtype).to(dtype).to(cuda)
        knew = randn((b, h, d), 2, dtype).to(dtype).to(cuda)
        vnew = randn((b, h, d), 3, dtype).to(dtype).to(cuda)
        positions = torch.tensor([n - 1, 31000], dtype=torch.int32, device=cuda)
        last_len = (n - 1) % page + 1
        last_idx = torch.tensor([offs[i] + npg - 1 for i in range(b)], dtype=torch.int32, device=cuda)
        dst = (last_idx * page + last_len - 1).to(torch.int32)
        g = torch.Generator().manual_seed(5 + k)
        lists, wants, k_rot = [], [], []
        q_cpu, knew_cpu, vnew_cpu = q.float().cpu(), knew.float().cpu(), vnew.float().cpu()
        for i in range(b):
            pos = torch.stack([torch.randperm(n - 1, generator=g)[: k - 1] for _ in range(h)])
            pos = torch.cat([pos, torch.full((h, 1), n - 1)], 1)[:, torch.randperm(k, generator=g)]
            lists.append(pos + offs[i] * page)
            p_i = [int(positions[i])]
            kk, vv = cases[i].k.clone(), cases[i].v.clone()
            kk[n - 1] = rotated(knew_cpu[i:i + 1], p_i, dtype, theta)[0]
            vv[n - 1] = vnew_cpu[i]
            k_rot.append(kk[n - 1])
            wants.append(orc.sparse_layer_gather(rotated(q_cpu[i:i + 1], p_i, dtype, theta)[0], kk, vv, pos))
        idx = torch.cat(lists, 1).to(torch.int32).to(cuda).contiguous()
        indptr = torch.tensor([0, k, 2 * k], dtype=torch.int32, device=cuda)
        zeros = torch.zeros(b, dtype=torch.int32, device=cuda)
        w = _wrapper(0, h, h, d, page, dtype, sparse_waves=sw, sparse_rows=sr)
        assert _uses_short_list_kernel(w, b, h, k)

        def run(fused):
            pl, qq, o = pool.clone(), q.clone(), torch.full_like(q, float("nan"))
            if fused:
                cos, sin = _kernels.rope_table(positions, d, 1.0, theta)
                w.forward(qq, o, pl, idx, indptr, zeros, zeros, None, index_kind="slots", n_list=k,
                          fresh=(knew, vnew, cos, sin, dst))
                assert torch.equal(qq, q)
            else:
                _kernels.rope_append_decode(qq, knew, vnew, pl, positions, dst, 0, 1.0, theta)
                w.forward(qq, o, pl, idx, indptr, zeros, zeros, None, index_kind="slots", n_list=k)
            torch.cuda.synchronize()
            return o, pl

        o1, p1 = run(False)
        o2, p2 = run(True)
        for i in range(b):
            assert tolerance_report(o2[i], wants[i]) <= ATOL[dtype], (h, k, i)
            assert tolerance_report(o1[i], wants[i]) <= ATOL[dtype], (h, k, i)
            page_i, entry_i = int(dst[i]) // page, int(dst[i]) % page
            assert within_ulps(p2[page_i, 0, entry_i], k_rot[i], dtype), (h, k, i)
            assert torch.equal(p2[page_i, 1, entry_i], vnew[i]), (h, k, i)
        assert (o1.float() - o2.float()).abs().max().item() <= ATOL[dtype] / 4, (h, k)
        ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
        assert ((p2.float() - p1.float()).abs() <= ulp * p1.float().abs() + 1e-6).all()
        changed = (p1 != pool).any(dim=(1, 2, 3, 4)).nonzero().flatten().tolist()
        assert changed == sorted(set(last_idx.tolist()))


def test_unlisted_entries_and_bad_slots_never_reach_the_output(cuda):
    """Entries past the list length hold out-of-range garbage, listed entries outside the pool are
    clamped: no fault, a finite result, and the same result as without the garbage."""
    dtype, h, d, page, n, k = torch.float16, 8, 128, 16, 700, 77
    case = PagedCase(n, h, d, page, dtype, seed=31)
    w = _wrapper(0, h, h, d, page, dtype)
    qd = randn((1, h, d), 1, dtype).to(dtype).to(cuda)
    pool = case.pool.to(cuda)
    g = torch.Generator().manual_seed(4)
    pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(h)])
    clean = case.slots_of(pos).to(torch.int32)
    wide = torch.full((h, 300), 2**30, dtype=torch.int32)
    wide[:, :k] = clean
    o1, o2 = torch.empty_like(qd), torch.empty_like(qd)
    w.forward(qd, o1, pool, clean.to(cuda), None, 0, 0, None, index_kind="slots")
    w.forward(qd, o2, pool, wide.to(cuda), None, 0, 0, None, index_kind="slots", n_list=k)
    bad = torch.full((h, 8), 2**30, dtype=torch.int32, device=cuda)
    bad[:, 1] = -5
    o3 = torch.empty_like(qd)
    w.forward(qd, o3, pool, bad, None, 0, 0, None, index_kind="slots")
    torch.cuda.synchronize()
    assert torch.equal(o1, o2)
    assert torch.isfinite(o3.float()).all()


def test_plans_of_both_kernels_share_one_workspace(cuda):
    """A handle alternates between the streaming kernel (page lists with logits) and the short-list
    kernel on shapes that lay their partials out differently: the ticket counters must come back
    to zero after every call, whichever kernel took them."""
    from oracle import tidal_oracle as orc

    dtype, h, d, page, n = torch.bfloat16, 8, 128, 16, 6000
    case = PagedCase(n, h, d, page, dtype, seed=8)
    q = randn((h, d), 9, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    pool = case.pool.to(cuda)
    w = _wrapper(0, h, h, d, page, dtype)
    logits = orc.attn_logits(q, case.k)
    want_full = orc.softmax_pv(logits, case.v)
    table = case.page_table[:-1].to(torch.int32).unsqueeze(0).to(cuda)
    g = torch.Generator().manual_seed(3)
    for k in (2048, 300, 1111, 5000):
        scores = torch.empty((h, case.n_pages * page), dtype=torch.float32, device=cuda)
        od = torch.empty_like(qd)
        w.forward(qd, od, pool, table, None, case.last_page_len, int(case.page_table[-1]), scores)
        pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(h)])
        want = orc.sparse_layer_gather(q, case.k, case.v, pos)
        os_ = torch.empty_like(qd)
        w.forward(qd, os_, pool, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
                  index_kind="slots")
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want_full) <= ATOL[dtype], k
        assert tolerance_report(os_[0], want) <= ATOL[dtype], k
        assert int(w._workspace[: 1 << 20].view(torch.int32).abs().sum()) == 0


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,rows", [(8, 4, 4), (16, 4, 4), (32, 4, 4), (16, 4, 1), (32, 8, 8), (64, 8, 8)])
@pytest.mark.parametrize("sw", [4, 8])
def test_shared_kv_rows(cuda, dtype, hq, hkv, rows, sw):
    """Grouped queries whose 2, 4 or 8 query heads share the list of their KV head (or one list for
    all): one walk of the list per KV head, the group's heads scored against every loaded row,
    p.V on the matrix cores.  Lengths around the tile edges, forced last page, both merges, several
    tiles per wave; oracle and streaming kernel as above."""
    from oracle import tidal_oracle as orc

    d, page, n = 128, 16, 3000 + 7
    case = PagedCase(n, hkv, d, page, dtype, seed=hq + hkv + rows)
    pool = case.pool.to(cuda)
    q = randn((hq, d), 3, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    before_last = (case.n_pages - 1) * page
    g = torch.Generator().manual_seed(2)
    gen = _wrapper(0, hq, hkv, d, page, dtype, sparse_waves=-1)
    tile = sw * 32
    for k, knobs in [(1, {}), (31, {}), (tile, {}), (tile + 1, {}), (700, {}), (700, dict(fused_merge=0)),
                     (2500, dict(chunk_tokens=1024)), (2048, {})]:
        w = _wrapper(0, hq, hkv, d, page, dtype, sparse_waves=sw, sparse_rows=8, **knobs)
        pos = torch.stack([torch.randperm(before_last, generator=g)[:k] for _ in range(rows)])
        assert _uses_short_list_kernel(w, 1, rows, k + case.last_page_len)
        slots = case.slots_of(pos).to(torch.int32).to(cuda).contiguous()
        allpos = torch.cat([pos, torch.arange(before_last, n).repeat(rows, 1)], 1)
        want = orc.sparse_layer_gather(q, case.k, case.v, allpos)
        od = torch.full_like(qd, float("nan"))
        lse = torch.full((1, hq), float("nan"), dtype=torch.float32, device=cuda)
        og = torch.full_like(qd, float("nan"))
        for _ in range(2):   # twice: the tickets and partial buffers are reused
            w.forward(qd, od, pool, slots, None, case.last_page_len, int(case.page_table[-1]), None,
                      index_kind="slots", lse=lse)
        gen.forward(qd, og, pool, slots, None, case.last_page_len, int(case.page_table[-1]), None,
                    index_kind="slots")
        torch.cuda.synchronize()
        assert tolerance_report(od[0], want) <= ATOL[dtype], (k, knobs)
        assert (od.float() - og.float()).abs().max().item() <= ATOL[dtype] / 2, (k, knobs)
        logits = orc.attn_logits(q, case.k)
        rows_of_heads = torch.arange(hq) * rows // hq
        want_lse = torch.logsumexp(torch.gather(logits, 1, allpos[rows_of_heads]), -1)
        assert (lse[0].cpu() - want_lse).abs().max() <= 1e-3, (k, knobs)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv", [(8, 4), (16, 4), (32, 4)])
def test_fused_decode_step_with_shared_kv_rows(cuda, dtype, hq, hkv):
    """The fused decode step on the shared-row kernels, against the oracle on float64-rotated,
    storage-rounded q and K and against the separate launches."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    d, page, n, b = 128, 16, 1500, 2
    for k in (1, 40, 700):
        cases = [PagedCase(n, hkv, d, page, dtype, seed=40 + i, spare=0, shuffle=False) for i in range(b)]
        npg = cases[0].n_pages
        pool = torch.cat([c.pool for c in cases]).to(cuda)
        offs = [0, npg]
        q = randn((b, hq, d), 1, dtype).to(dtype).to(cuda)
        knew = randn((b, hkv, d), 2, dtype).to(dtype).to(cuda)
        vnew = randn((b, hkv, d), 3, dtype).to(dtype).to(cuda)
        positions = torch.tensor([n - 1, 31000], dtype=torch.int32, device=cuda)
        last_len = (n - 1) % page + 1
        last_idx = torch.tensor([offs[i] + npg - 1 for i in range(b)], dtype=torch.int32, device=cuda)
        dst = (last_idx * page + last_len - 1).to(torch.int32)
        g = torch.Generator().manual_seed(5 + k)
        lists, wants, k_rot = [], [], []
        q_cpu, knew_cpu, vnew_cpu = q.float().cpu(), knew.float().cpu(), vnew.float().cpu()
        for i in range(b):
            pos = torch.stack([torch.randperm(n - 1, generator=g)[: k - 1] for _ in range(hkv)])
            pos = torch.cat([pos, torch.full((hkv, 1), n - 1)], 1)[:, torch.randperm(k, generator=g)]
            lists.append(pos + offs[i] * page)
            p_i = [int(positions[i])]
            kk, vv = cases[i].k.clone(), cases[i].v.clone()
            kk[n - 1] = rotated(knew_cpu[i:i + 1], p_i, dtype, 5e5)[0]
            vv[n - 1] = vnew_cpu[i]
            k_rot.append(kk[n - 1])
            wants.append(orc.sparse_layer_gather(rotated(q_cpu[i:i + 1], p_i, dtype, 5e5)[0], kk, vv, pos))
        idx = torch.cat(lists, 1).to(torch.int32).to(cuda).contiguous()
        indptr = torch.tensor([0, k, 2 * k], dtype=torch.int32, device=cuda)
        zeros = torch.zeros(b, dtype=torch.int32, device=cuda)
        w = _wrapper(0, hq, hkv, d, page, dtype)
        assert _uses_short_list_kernel(w, b, hkv, k)

        def run(fused):
            pl, qq, o = pool.clone(), q.clone(), torch.full_like(q, float("nan"))
            if fused:
                cos, sin = _kernels.rope_table(positions, d, 1.0, 5e5)
                w.forward(qq, o, pl, idx, indptr, zeros, zeros, None, index_kind="slots", n_list=k,
                          fresh=(knew, vnew, cos, sin, dst))
                assert torch.equal(qq, q)
            else:
                _kernels.rope_append_decode(qq, knew, vnew, pl, positions, dst, 0, 1.0, 5e5)
                w.forward(qq, o, pl, idx, indptr, zeros, zeros, None, index_kind="slots", n_list=k)
            torch.cuda.synchronize()
            return o, pl

        o1, p1 = run(False)
        o2, p2 = run(True)
        for i in range(b):
            assert tolerance_report(o2[i], wants[i]) <= ATOL[dtype], (k, i)
            page_i, entry_i = int(dst[i]) // page, int(dst[i]) % page
            assert within_ulps(p2[page_i, 0, entry_i], k_rot[i], dtype), (k, i)
            assert torch.equal(p2[page_i, 1, entry_i], vnew[i]), (k, i)
        assert (o1.float() - o2.float()).abs().max().item() <= ATOL[dtype] / 4, k
        ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
        assert ((p2.float() - p1.float()).abs() <= ulp * p1.float().abs() + 1e-6).all()
        changed = (p1 != pool).any(dim=(1, 2, 3, 4)).nonzero().flatten().tolist()
        assert changed == sorted(set(last_idx.tolist()))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("page", [1, 3, 7, 12, 31])
@pytest.mark.parametrize("hq,hkv,rows", [(8, 8, 8), (16, 4, 4), (8, 2, 8)])
def test_pages_of_any_size(cuda, dtype, page, hq, hkv, rows):
    """Page sizes that are not a power of two (the reference tests 3, 7 and 31,
    kernels/src/test/test_batch_decode.cu:215-267): the short-list kernel divides the slot by the
    page size once per lane and forms 64-bit row offsets.  Slot lists with the forced last page,
    then the fused decode step, both against the oracle."""
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    d, n = 128, 1000 + page // 2
    case = PagedCase(n, hkv, d, page, dtype, seed=page + hq)
    pool = case.pool.to(cuda)
    q = randn((hq, d), 5, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    before_last = (case.n_pages - 1) * page
    g = torch.Generator().manual_seed(page)
    w = _wrapper(0, hq, hkv, d, page, dtype)
    kernel = "short-list" if page == 1 else "short-list, 64-bit offsets"
    for k in (1, 33, 600):
        pos = torch.stack([torch.randperm(before_last, generator=g)[:k] for _ in range(rows)])
        allpos = torch.cat([pos, torch.arange(before_last, n).repeat(rows, 1)], 1)
        want = orc.sparse_layer_gather(q, case.k, case.v, allpos)
        od = torch.full_like(qd, float("nan"))
        w.forward(qd, od, pool, case.slots_of(pos).to(torch.int32).to(cuda).contiguous(), None,
                  case.last_page_len, int(case.page_table[-1]), None, index_kind="slots")
        torch.cuda.synchronize()
        assert _kernels.last_decode_kernel() == kernel
        assert tolerance_report(od[0], want) <= ATOL[dtype], (k, page)
    # fused step: the newest token is the one being decoded and sits in every list
    theta, new_pos = 1e4, n - 1
    pos = torch.stack([torch.randperm(n - 1, generator=g)[:199] for _ in range(rows)])
    pos = torch.cat([pos, torch.full((rows, 1), n - 1)], 1)
    k_new, v_new = randn((1, hkv, d), 41, dtype), randn((1, hkv, d), 42, dtype)
    k_f, v_f = case.k.clone(), case.v.clone()
    k_f[n - 1] = rotated(k_new, [new_pos], dtype, theta)[0]
    v_f[n - 1] = v_new[0]
    want = orc.sparse_layer_gather(rotated(q[None], [new_pos], dtype, theta)[0], k_f, v_f, pos)
    dst = case.slots_of(torch.tensor([n - 1])).to(torch.int32).to(cuda)
    cos, sin = _kernels.rope_table(torch.tensor([new_pos], dtype=torch.int32, device=cuda), d, 1.0, theta)
    pool_f = pool.clone()
    od = torch.full_like(qd, float("nan"))
    w.forward(qd, od, pool_f, case.slots_of(pos).to(torch.int32).to(cuda).contiguous(), None, 0, 0, None,
              index_kind="slots", fresh=(k_new.to(dtype).to(cuda), v_new.to(dtype).to(cuda), cos, sin, dst))
    torch.cuda.synchronize()
    assert _kernels.last_decode_kernel() == kernel
    assert tolerance_report(od[0], want) <= ATOL[dtype], page
    page_f, entry_f = int(dst[0]) // page, int(dst[0]) % page
    assert within_ulps(pool_f[page_f, 0, entry_f], k_f[n - 1], dtype)
    assert torch.equal(pool_f[page_f, 1, entry_f].cpu(), v_new[0].to(dtype))
    pool_f[page_f, :, entry_f] = pool[page_f, :, entry_f]
    assert torch.equal(pool_f, pool)

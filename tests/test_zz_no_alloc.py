"""GPU: td_decode_attn_noalloc (scratch inside the library image) against td_decode_attn (caller's
workspace) through the C ABI: bit-identical outputs on two calls in a row, the second one with a
smaller input, for the short-list kernel, the streaming kernel with logits, and the fused step;
plans beyond the built-in scratch are refused."""
import pytest
import torch

from _util import ATOL, PagedCase, randn, tolerance_report

pytestmark = pytest.mark.gpu


def _pair(layout, hq, hkv, d, page, dtype):
    from tidaldecode_amd import _kernels

    ws, st = (_kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(layout) for _ in range(2))
    st.static_scratch = True
    for w in (ws, st):
        w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    return ws, st


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_same_bits_as_the_workspace_entry_point(cuda, dtype):
    from oracle import tidal_oracle as orc

    h, d, page, n = 32, 128, 16, 9000
    case = PagedCase(n, h, d, page, dtype, seed=3)
    pool = case.pool.to(cuda)
    q = randn((h, d), 4, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    ws, st = _pair(0, h, h, d, page, dtype)
    g = torch.Generator().manual_seed(5)
    for k in (2048, 300):                      # two calls in a row, the second one smaller
        pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(h)])
        slots = case.slots_of(pos).to(torch.int32).to(cuda)
        o1, o2 = torch.full_like(qd, float("nan")), torch.full_like(qd, float("nan"))
        ws.forward(qd, o1, pool, slots, None, 0, 0, None, index_kind="slots")
        st.forward(qd, o2, pool, slots, None, 0, 0, None, index_kind="slots")
        torch.cuda.synchronize()
        assert st._workspace is None            # nothing was allocated for it
        assert torch.equal(o1, o2), k
        assert tolerance_report(o2[0], orc.sparse_layer_gather(q, case.k, case.v, pos)) <= ATOL[dtype]
    # the streaming kernel with logits (selection layer), then a shorter sequence
    for n2 in (n, 1000):
        c2 = case if n2 == n else PagedCase(n2, h, d, page, dtype, seed=6)
        p2 = pool if n2 == n else c2.pool.to(cuda)
        table = c2.page_table[:-1].to(torch.int32).unsqueeze(0).to(cuda)
        outs = []
        for w in (ws, st):
            o = torch.full_like(qd, float("nan"))
            scores = torch.full((h, c2.n_pages * page), float("nan"), dtype=torch.float32, device=cuda)
            lse = torch.empty((1, h), dtype=torch.float32, device=cuda)
            w.forward(qd, o, p2, table, None, c2.last_page_len, int(c2.page_table[-1]), scores, lse=lse)
            outs.append((o, scores[:, :n2].clone(), lse))
        torch.cuda.synchronize()
        for a, b in zip(*outs):
            assert torch.equal(a, b), n2
        logits = orc.attn_logits(q, c2.k)
        assert tolerance_report(outs[1][0][0], orc.softmax_pv(logits, c2.v)) <= ATOL[dtype]


def test_fused_step_and_graph_replay(cuda):
    """The entry point inside a captured graph (its reason to exist): replayed three times with
    eager work in between, every replay equal to the workspace entry point's eager result."""
    from tidaldecode_amd import _kernels

    dtype, h, d, page, n, k = torch.bfloat16, 32, 128, 16, 4000, 1024
    case = PagedCase(n, h, d, page, dtype, seed=9, spare=0, shuffle=False)
    pool = case.pool.to(cuda)
    q = randn((1, h, d), 1, dtype).to(dtype).to(cuda)
    knew = randn((1, h, d), 2, dtype).to(dtype).to(cuda)
    vnew = randn((1, h, d), 3, dtype).to(dtype).to(cuda)
    positions = torch.tensor([n - 1], dtype=torch.int32, device=cuda)
    dst = torch.tensor([(case.n_pages - 1) * page + (n - 1) % page], dtype=torch.int32, device=cuda)
    g = torch.Generator().manual_seed(2)
    pos = torch.stack([torch.randperm(n - 1, generator=g)[: k - 1] for _ in range(h)])
    pos = torch.cat([pos, torch.full((h, 1), n - 1)], 1)
    slots = pos.to(torch.int32).to(cuda)        # pages are not shuffled: slot == position
    cos, sin = _kernels.rope_table(positions, d)
    ws, st = _pair(0, h, h, d, page, dtype)
    want = torch.empty_like(q)
    ws.forward(q, want, pool.clone(), slots, None, 0, 0, None, index_kind="slots",
               fresh=(knew, vnew, cos, sin, dst))
    pl, got = pool.clone(), torch.empty_like(q)
    st.forward(q, got, pl, slots, None, 0, 0, None, index_kind="slots", fresh=(knew, vnew, cos, sin, dst))
    torch.cuda.synchronize()                    # first call outside the capture (address lookup)
    assert torch.equal(got, want)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(s):
        with torch.cuda.graph(graph, stream=s):
            st.forward(q, got, pl, slots, None, 0, 0, None, index_kind="slots",
                       fresh=(knew, vnew, cos, sin, dst))
    torch.cuda.current_stream().wait_stream(s)
    for _ in range(3):
        got.fill_(float("nan"))
        other = torch.empty_like(q)             # eager work between the replays
        ws.forward(q, other, pool.clone(), slots[:, :100].contiguous(), None, 0, 0, None, index_kind="slots")
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(got, want)


def test_plans_beyond_the_scratch_are_refused(cuda):
    from tidaldecode_amd import _lib

    dtype, h, d, page = torch.float16, 32, 128, 16
    b, k = 64, 2048                             # 64 x 32 head rows x 5 splits of 520 bytes > 4 MiB of partials
    pool = torch.zeros((8, 2, page, h, d), dtype=dtype, device=cuda)
    q = torch.zeros((b, h, d), dtype=dtype, device=cuda)
    idx = torch.zeros((h, b * k), dtype=torch.int32, device=cuda)
    indptr = torch.arange(0, (b + 1) * k, k, dtype=torch.int32, device=cuda)
    zeros = torch.zeros(b, dtype=torch.int32, device=cuda)
    _, st = _pair(0, h, h, d, page, dtype)
    st.chunk_tokens = 512                       # (the default plan of this shape is one split per head)
    assert st._plan(b, h, k + page).workspace_bytes > _lib.TD_STATIC_SCRATCH_BYTES
    with pytest.raises(RuntimeError, match="built-in scratch"):
        st.forward(q, q.clone(), pool, idx, indptr, zeros, zeros, None, index_kind="slots", n_list=k)

"""GPU: the fused decode step (fresh=...) against the CPU oracle on float64-rotated,
storage-rounded q and K, and against the three separate calls it replaces (RoPE in place, append,
attention): same attention output far inside the attention tolerance (the two GPU paths share
every rounding but the rotated key's), same cache contents up to one rounding of the rotated key,
logits of the new token included."""
import pytest
import torch

from _util import ATOL, PagedCase, randn, rotated, tolerance_report, within_ulps

pytestmark = pytest.mark.gpu


def _ulp_close(a, b, dtype):
    ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    return ((a.float() - b.float()).abs() <= ulp * b.float().abs() + 1e-6).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("hq,hkv,rows,mode", [(32, 32, 32, "slots"), (32, 32, 1, "pages"),
                                              (32, 8, 8, "slots"), (32, 8, 32, "slots"),
                                              (32, 8, 1, "pages"), (8, 8, 8, "slots"),
                                              # groups of 3 and 7 run padded on the 4- and 8-head kernels
                                              (24, 8, 8, "slots"), (28, 4, 1, "pages"),
                                              (28, 4, 4, "slots"),
                                              # 12 heads per KV head: two head rows (8 + 4) per KV head
                                              (24, 2, 2, "slots"), (24, 2, 1, "pages")])
def test_fused_equals_separate(cuda, dtype, hq, hkv, rows, mode):
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    d, page, n, k, b = 128, 16, 1000, 96, 2   # n counts the new token
    theta = 5e5
    cases = [PagedCase(n, hkv, d, page, dtype, seed=40 + i, spare=0, shuffle=False) for i in range(b)]
    # two sequences in one pool: pages of sequence 1 follow those of sequence 0
    npg = cases[0].n_pages
    pool = torch.cat([c.pool for c in cases]).to(cuda)
    offs = [0, npg]
    q = randn((b, hq, d), 1, dtype).to(dtype).to(cuda)
    knew = randn((b, hkv, d), 2, dtype).to(dtype).to(cuda)
    vnew = randn((b, hkv, d), 3, dtype).to(dtype).to(cuda)
    positions = torch.tensor([n - 1, 70000], dtype=torch.int32, device=cuda)
    last_len = (n - 1) % page + 1
    last_idx = torch.tensor([offs[i] + npg - 1 for i in range(b)], dtype=torch.int32, device=cuda)
    dst = (last_idx * page + last_len - 1).to(torch.int32)
    g = torch.Generator().manual_seed(5)
    attended = []         # per sequence: the positions each list row attends to
    if mode == "pages":   # selection layer: every page in order + last page
        idx = torch.cat([torch.arange(npg - 1) + offs[i] for i in range(b)]).to(torch.int32)[None]
        indptr = torch.tensor([0, npg - 1, 2 * (npg - 1)], dtype=torch.int32, device=cuda)
        ll = torch.full((b,), last_len, dtype=torch.int32, device=cuda)
        li = last_idx
        n_list = npg - 1
        attended = [torch.arange(n)[None] for _ in range(b)]
    else:                 # sparse layer: k slots per row, the new token's slot among them
        lists = []
        for i in range(b):
            pos = torch.stack([torch.randperm(n - 1, generator=g)[: k - 1] for _ in range(rows)])
            pos = torch.cat([pos, torch.full((rows, 1), n - 1)], 1)[:, torch.randperm(k, generator=g)]
            lists.append(pos + offs[i] * page)
            attended.append(pos)
        idx = torch.cat(lists, 1).to(torch.int32)
        indptr = torch.tensor([0, k, 2 * k], dtype=torch.int32, device=cuda)
        ll = torch.zeros(b, dtype=torch.int32, device=cuda)
        li = torch.zeros(b, dtype=torch.int32, device=cuda)
        n_list = k
    idx = idx.to(cuda).contiguous()
    kind = "pages" if mode == "pages" else "slots"
    stride = npg * page
    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))

    def run(fused):
        pl = pool.clone()
        qq = q.clone()
        o = torch.empty_like(q)
        scores = torch.zeros((b * hq, stride), dtype=torch.float32, device=cuda) if mode == "pages" else None
        if fused:
            cos, sin = _kernels.rope_table(positions, d, 1.0, theta)
            w.forward(qq, o, pl, idx, indptr, ll, li, scores, index_kind=kind, n_list=n_list,
                      fresh=(knew, vnew, cos, sin, dst))
            assert torch.equal(qq, q)  # q in memory is left as it was
        else:
            _kernels.rope_append_decode(qq, knew, vnew, pl, positions, dst, 0, 1.0, theta)
            w.forward(qq, o, pl, idx, indptr, ll, li, scores, index_kind=kind, n_list=n_list)
        torch.cuda.synchronize()
        return o, pl, scores

    o1, p1, s1 = run(False)
    o2, p2, s2 = run(True)
    q_cpu, knew_cpu, vnew_cpu = q.float().cpu(), knew.float().cpu(), vnew.float().cpu()
    for i in range(b):
        p_i = [int(positions[i])]
        kk, vv = cases[i].k.clone(), cases[i].v.clone()
        kk[n - 1] = rotated(knew_cpu[i:i + 1], p_i, dtype, theta)[0]
        vv[n - 1] = vnew_cpu[i]
        q_rot = rotated(q_cpu[i:i + 1], p_i, dtype, theta)[0]
        want = orc.sparse_layer_gather(q_rot, kk, vv, attended[i])
        assert tolerance_report(o2[i], want) <= ATOL[dtype], i
        page_i, entry_i = int(dst[i]) // page, int(dst[i]) % page
        assert within_ulps(p2[page_i, 0, entry_i], kk[n - 1], dtype), i
        assert torch.equal(p2[page_i, 1, entry_i], vnew[i]), i
        if s2 is not None:
            logits = orc.attn_logits(q_rot, kk)
            # a rotated q element that lands on the other side of a rounding boundary than the
            # float64 rotation moves a head's logits by up to one storage ulp of q times |k| / sqrt(d)
            ulp = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
            bound = 2e-4 * max(1.0, logits.abs().max().item()) + 0.5 * ulp
            assert (s2[i * hq:(i + 1) * hq, :n].cpu() - logits).abs().max() <= bound, i
    assert (o1.float() - o2.float()).abs().max().item() <= ATOL[dtype] / 4
    assert _ulp_close(p2, p1, dtype)                         # the cache got the new token
    changed = (p1 != pool).any(dim=(1, 2, 3, 4)).nonzero().flatten().tolist()
    assert changed == sorted(set(last_idx.tolist()))         # ... and nothing else
    if s1 is not None:
        assert (s1[:, :n] - s2[:, :n]).abs().max().item() <= 2e-2
        assert s2[:, n - 1].abs().max() > 0                  # the new token's logit is there


def test_fused_needs_lean_pool(cuda):
    from tidaldecode_amd import _kernels

    dtype, h, d, page = torch.float16, 8, 64, 3   # page size 3: no fused kernel
    pool = torch.zeros((10, 2, page, h, d), dtype=dtype, device=cuda)
    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, h, h, d, page, torch.empty(0, dtype=dtype))
    q = torch.zeros((1, h, d), dtype=dtype, device=cuda)
    pos = torch.zeros(1, dtype=torch.int32, device=cuda)
    cos, sin = _kernels.rope_table(pos, d)
    assert torch.equal(cos.cpu(), torch.ones(1, d // 2)) and torch.equal(sin.cpu(), torch.zeros(1, d // 2))
    idx = torch.zeros((h, 4), dtype=torch.int32, device=cuda)
    with pytest.raises(RuntimeError, match="power-of-two"):
        w.forward(q, q.clone(), pool, idx, None, 0, 0, None, index_kind="slots",
                  fresh=(q.clone(), q.clone(), cos, sin, pos))

"""GPU parity on pools larger than 4 GiB: byte offsets no longer fit 32 bits, so every kernel that
addresses the pool (decode attention with slot and page lists, the selection mode with logits,
append, RoPE + append, prefill, the page estimator's metadata aside) must form 64-bit addresses.
The sequence's pages are placed at both ends of the pool, the very last page included; the pool is
built on the device and only the sequence's own K/V (a few MB) exists on the host for the oracle.
Tolerances as in the other attention tests: max-abs 2e-3 (fp16) / 1e-2 (bf16).
"""
import numpy as np
import pytest
import torch

from _util import ATOL, randn, rotated, tolerance_report, within_ulps

pytestmark = pytest.mark.gpu


class BigPool:
    """n tokens of seeded K/V in a device pool of `pool_pages` pages (NHD), garbage elsewhere;
    every second logical page sits in the last pages of the pool."""

    def __init__(self, cuda, n, hkv, d, page, dtype, pool_pages, seed):
        self.n, self.hkv, self.d, self.page, self.dtype = n, hkv, d, page, dtype
        self.k, self.v = randn((n, hkv, d), seed, dtype), randn((n, hkv, d), seed + 1, dtype)
        self.n_pages = (n + page - 1) // page
        assert pool_pages * 2 * page * hkv * d * 2 > (1 << 32) + (1 << 28)
        g = torch.Generator().manual_seed(seed)
        hi = pool_pages - 1 - torch.randperm(self.n_pages, generator=g)[: (self.n_pages + 1) // 2]
        lo = torch.randperm(self.n_pages, generator=g)[: self.n_pages // 2]
        table = torch.empty(self.n_pages, dtype=torch.int64)
        table[0::2], table[1::2] = hi, lo
        table[-1] = pool_pages - 1 if (pool_pages - 1) not in table[:-1].tolist() else table[-1]
        self.page_table = table
        assert len(set(table.tolist())) == self.n_pages
        self.last_page_len = (n - 1) % page + 1
        pad = self.n_pages * page - n
        self.pool = torch.full((pool_pages, 2, page, hkv, d), 77.0, dtype=dtype, device=cuda)
        kp = torch.cat([self.k, torch.full((pad, hkv, d), 77.0)]).view(self.n_pages, page, hkv, d)
        vp = torch.cat([self.v, torch.full((pad, hkv, d), 77.0)]).view(self.n_pages, page, hkv, d)
        t = table.to(cuda)
        self.pool[t, 0] = kp.to(dtype).to(cuda)
        self.pool[t, 1] = vp.to(dtype).to(cuda)

    def slots_of(self, pos):
        pos = pos.long()
        return self.page_table[pos // self.page] * self.page + pos % self.page


def _wrapper(hq, hkv, d, page, dtype):
    from tidaldecode_amd import _kernels

    w = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(0)
    w.begin_forward(None, hq, hkv, d, page, torch.empty(0, dtype=dtype))
    return w


@pytest.mark.parametrize("dtype,hq,hkv,pool_pages", [(torch.float16, 32, 32, 18000),
                                                     (torch.bfloat16, 32, 8, 72000)])
def test_decode_attention_beyond_4gib(cuda, dtype, hq, hkv, pool_pages):
    from oracle import tidal_oracle as orc

    d, page, n, k = 128, 16, 3001, 257
    case = BigPool(cuda, n, hkv, d, page, dtype, pool_pages, seed=5)
    q = randn((hq, d), 17, dtype)
    qd = q.to(dtype).to(cuda).unsqueeze(0)
    w = _wrapper(hq, hkv, d, page, dtype)
    g = torch.Generator().manual_seed(3)

    # token-slot lists: one per query head, and one per KV head -- the short-list kernel with 64-bit
    # row offsets; then the same call as a fused decode step (the newest token is the one being
    # decoded: RoPE of q and its key, the cache write at the far end of the pool, attention)
    from tidaldecode_amd import _kernels

    for rows in (hq, hkv):
        pos = torch.stack([torch.randperm(n, generator=g)[:k] for _ in range(rows)])
        want = orc.sparse_layer_gather(q, case.k, case.v, pos)
        od = torch.empty_like(qd)
        w.forward(qd, od, case.pool, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
                  index_kind="slots")
        torch.cuda.synchronize()
        assert _kernels.last_decode_kernel().startswith("short-list, 64-bit offsets")
        assert tolerance_report(od[0], want) <= ATOL[dtype], rows

        pos[::2, 0] = n - 1                                   # every second list names the new token
        for r in range(1, rows, 2):
            pos[r][pos[r] == n - 1] = int((set(range(n - 1)) - set(pos[r].tolist())).pop())
        for r in range(0, rows, 2):                           # ... once
            dup = (pos[r, 1:] == n - 1).nonzero().flatten()
            if dup.numel():
                pos[r, 1 + int(dup[0])] = int((set(range(n - 1)) - set(pos[r].tolist())).pop())
        theta, new_pos = 5e5, 70001
        k_new, v_new = randn((1, hkv, d), 31, dtype), randn((1, hkv, d), 32, dtype)
        k_f, v_f = case.k.clone(), case.v.clone()
        k_f[n - 1] = rotated(k_new, [new_pos], dtype, theta)[0]
        v_f[n - 1] = v_new[0]
        want = orc.sparse_layer_gather(rotated(q[None], [new_pos], dtype, theta)[0], k_f, v_f, pos)
        dst = case.slots_of(torch.tensor([n - 1])).to(torch.int32).to(cuda)
        cos, sin = _kernels.rope_table(torch.tensor([new_pos], dtype=torch.int32, device=cuda), d, 1.0, theta)
        page_f, entry_f = int(dst[0]) // page, int(dst[0]) % page
        before = case.pool[page_f].clone()
        w.forward(qd, od, case.pool, case.slots_of(pos).to(torch.int32).to(cuda), None, 0, 0, None,
                  index_kind="slots", fresh=(k_new.to(dtype).to(cuda), v_new.to(dtype).to(cuda), cos, sin, dst))
        torch.cuda.synchronize()
        assert _kernels.last_decode_kernel().startswith("short-list, 64-bit offsets")
        assert tolerance_report(od[0], want) <= ATOL[dtype], rows
        assert within_ulps(case.pool[page_f, 0, entry_f], k_f[n - 1], dtype)
        assert torch.equal(case.pool[page_f, 1, entry_f].cpu(), v_new[0].to(dtype))
        case.pool[page_f] = before                            # the later checks use the original token

    # the whole page table in order, logits and log-sum-exp out (selection layer)
    logits = orc.attn_logits(q, case.k)
    want = orc.softmax_pv(logits, case.v)
    od = torch.empty_like(qd)
    scores = torch.full((hq, case.n_pages * page), float("nan"), dtype=torch.float32, device=cuda)
    lse = torch.empty((1, hq), dtype=torch.float32, device=cuda)
    table = case.page_table[:-1].to(torch.int32).unsqueeze(0).to(cuda)
    w.forward(qd, od, case.pool, table, None, case.last_page_len, int(case.page_table[-1]), scores,
              lse=lse)
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype]
    assert (scores[:, :n].cpu() - logits).abs().max() <= 2e-4 * max(1.0, logits.abs().max().item())
    assert torch.isnan(scores[:, n:]).all()
    assert (lse[0].cpu() - torch.logsumexp(logits, -1)).abs().max() <= 1e-3

    # per-head page lists with the forced last page (the reference's sparse call)
    budget = 40
    lists = torch.stack([case.page_table[torch.randperm(case.n_pages - 1, generator=g)[: budget - 1]]
                         for _ in range(hq)])
    pos = []
    for h in range(hq):
        logical = [int((case.page_table == p).nonzero()[0]) for p in lists[h]]
        toks = torch.cat([torch.arange(p * page, (p + 1) * page) for p in logical] +
                         [torch.arange((case.n_pages - 1) * page, n)])
        pos.append(toks)
    assert len({len(p) for p in pos}) == 1
    want = orc.sparse_layer_gather(q, case.k, case.v, torch.stack(pos))
    od = torch.empty_like(qd)
    w.forward(qd, od, case.pool, lists.to(torch.int32).to(cuda), None, case.last_page_len,
              int(case.page_table[-1]), None)
    torch.cuda.synchronize()
    assert tolerance_report(od[0], want) <= ATOL[dtype]


def test_append_rope_and_prefill_beyond_4gib(cuda):
    from oracle import tidal_oracle as orc
    from tidaldecode_amd import _kernels

    dtype, hq, hkv, d, page, n, pool_pages = torch.float16, 32, 32, 128, 16, 700, 18000
    case = BigPool(cuda, n, hkv, d, page, dtype, pool_pages, seed=9)

    # prefill attention of the newest 300 tokens over pages at both ends of the pool
    n_q = 300
    q = randn((n_q, hq, d), 23, dtype)
    got = _kernels.prefill_with_paged_kv_cache(q.to(dtype).to(cuda), case.pool,
                                               case.page_table.to(torch.int32).to(cuda),
                                               case.last_page_len, True, 0, False, 1.0, 1e4)
    torch.cuda.synchronize()
    for row in (0, 150, n_q - 1):
        upto = n - n_q + row + 1
        want = orc.softmax_pv(orc.attn_logits(q[row], case.k[:upto]), case.v[:upto])
        assert ((got[row].float().cpu() - want).abs() <= ATOL[dtype] * want.abs().clamp(min=1.0)).all()

    # RoPE + append of one token into the pool's very last slot, then the plain append beside it
    last_slot = pool_pages * page - 1
    qn, kn, vn = (randn(s_, 31 + i, dtype) for i, s_ in enumerate(((1, hq, d), (1, hkv, d), (1, hkv, d))))
    position = 4321
    qd, kd, vd = (t.to(dtype).to(cuda) for t in (qn, kn, vn))
    _kernels.rope_append_decode(qd, kd, vd, case.pool,
                                torch.tensor([position], dtype=torch.int32, device=cuda),
                                torch.tensor([last_slot], dtype=torch.int32, device=cuda), 0, 1.0, 1e4)
    torch.cuda.synchronize()
    want_k = torch.from_numpy(orc.rope_closed_form(kn.numpy(), np.array([position])))[0]
    want_q = torch.from_numpy(orc.rope_closed_form(qn.numpy(), np.array([position])))[0]
    got_k = case.pool[pool_pages - 1, 0, page - 1].double().cpu()
    assert ((got_k - want_k).abs() <= 2e-3 * want_k.abs().clamp(min=1.0)).all()
    assert torch.equal(case.pool[pool_pages - 1, 1, page - 1].cpu(), vd[0].cpu())
    assert ((qd[0].double().cpu() - want_q).abs() <= 2e-3 * want_q.abs().clamp(min=1.0)).all()

    # append_kv_cache_decode: the new token is the last entry of the sequence's last page
    table = torch.tensor([pool_pages - 2], dtype=torch.int32, device=cuda)
    indptr = torch.tensor([0, 1], dtype=torch.int32, device=cuda)
    k2, v2 = (randn((1, hkv, d), 41 + i, dtype).to(dtype).to(cuda) for i in range(2))
    before = case.pool[pool_pages - 2].clone()
    _kernels.append_kv_cache_decode(k2, v2, case.pool, table, indptr, 7, int(table[0]),
                                    torch.empty(0, device=cuda), table, indptr, 1, int(table[0]), 0)
    torch.cuda.synchronize()
    after = case.pool[pool_pages - 2]
    assert torch.equal(after[0, 6], k2[0]) and torch.equal(after[1, 6], v2[0])
    before[0, 6], before[1, 6] = k2[0], v2[0]
    assert torch.equal(after, before)   # nothing else on the page changed

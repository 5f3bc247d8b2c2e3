"""CPU: pin the oracle (oracle/tidal_oracle.py, oracle/cpu_reference.c) before anything trusts it.

The reference holds no golden vectors for this path (its tests draw from std::random_device), so
every oracle function is pinned against something independent of its own formula: a library
routine (torch SDPA, torch.topk, transformers' rotary embedding), a pure-Python brute force on tiny
inputs, a second independent implementation (numpy/torch vs. C), or a closed-form special case.
"""
import math

import numpy as np
import pytest
import torch

from oracle import cref
from oracle import tidal_oracle as orc


def _qkv(hq, hkv, n, d, seed):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn((hq, d), generator=g), torch.randn((n, hkv, d), generator=g),
            torch.randn((n, hkv, d), generator=g))


# ---------------------------------------------------------------------------------------------
# dense attention
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("hq,hkv,n,d", [(4, 4, 37, 16), (8, 2, 129, 64), (32, 8, 500, 128)])
def test_full_attention_equals_sdpa(hq, hkv, n, d):
    q, k, v = _qkv(hq, hkv, n, d, 1)
    kk = orc.repeat_kv(k, hq // hkv).permute(1, 0, 2)[None]
    vv = orc.repeat_kv(v, hq // hkv).permute(1, 0, 2)[None]
    want = torch.nn.functional.scaled_dot_product_attention(q[None, :, None, :], kk, vv)[0, :, 0]
    assert (orc.full_attention(q, k, v) - want).abs().max() < 1e-5


def test_full_attention_brute_force():
    """pure-Python loops on a tiny case; also pins the GQA head mapping h -> h // group"""
    hq, hkv, n, d = 4, 2, 5, 3
    q, k, v = _qkv(hq, hkv, n, d, 2)
    got = orc.full_attention(q, k, v)
    for h in range(hq):
        kvh = h // (hq // hkv)
        s = [sum(float(q[h, f]) * float(k[i, kvh, f]) for f in range(d)) / math.sqrt(d)
             for i in range(n)]
        mx = max(s)
        e = [math.exp(x - mx) for x in s]
        z = sum(e)
        for f in range(d):
            want = sum(e[i] / z * float(v[i, kvh, f]) for i in range(n))
            assert abs(float(got[h, f]) - want) < 1e-5


@pytest.mark.parametrize("layout", [0, 1])
def test_c_single_mha_equals_torch(layout):
    q, k, v = _qkv(8, 4, 77, 32, 3)
    kc, vc = k.numpy(), v.numpy()
    if layout == 1:
        kc, vc = kc.transpose(1, 0, 2).copy(), vc.transpose(1, 0, 2).copy()
    got = cref.single_mha(q.numpy(), kc, vc, layout)
    assert np.abs(got - orc.full_attention(q, k, v).numpy()).max() < 1e-5


# ---------------------------------------------------------------------------------------------
# top-k
# ---------------------------------------------------------------------------------------------
def test_stable_topk_equals_torch_topk_as_sets():
    g = torch.Generator().manual_seed(4)
    s = torch.randn((16, 3000), generator=g)
    for k in (1, 7, 256, 2999, 3000):
        want = torch.topk(s, k, dim=-1).indices.sort(-1).values
        assert torch.equal(orc.stable_topk(s, k), want)
        assert np.array_equal(cref.stable_topk(s.numpy(), k), want.numpy().astype(np.int32))


def test_stable_topk_tie_rule_brute_force():
    """ties at the threshold go to the lower index: brute force by Python's stable sort"""
    g = torch.Generator().manual_seed(5)
    s = torch.randint(0, 4, (6, 50), generator=g).float()
    for k in (1, 5, 20, 49):
        for r in range(6):
            row = s[r].tolist()
            order = sorted(range(50), key=lambda i: (-row[i], i))[:k]
            assert orc.stable_topk(s[r:r + 1], k)[0].tolist() == sorted(order)
            assert cref.stable_topk(s[r:r + 1].numpy(), k)[0].tolist() == sorted(order)


def test_stable_topk_closed_forms():
    g = torch.Generator().manual_seed(6)
    s = torch.randn((5, 100), generator=g)
    assert torch.equal(orc.stable_topk(s, 1)[:, 0], s.argmax(-1))
    assert torch.equal(orc.stable_topk(s, 100), torch.arange(100).repeat(5, 1))
    assert torch.equal(orc.stable_topk(s, 1000), torch.arange(100).repeat(5, 1))  # k clamps to N
    # NaN orders above everything, as torch.topk does
    s[0, 17] = float("nan")
    assert 17 in orc.stable_topk(s, 1)[0].tolist()
    assert 17 in cref.stable_topk(s.numpy(), 1)[0].tolist()


def test_head_sum_scores_closed_form():
    g = torch.Generator().manual_seed(7)
    logits = torch.randn((8, 33), generator=g) * 4
    got = orc.head_sum_scores(logits, 1)
    want = torch.zeros(33, dtype=torch.float64)
    for h in range(8):
        e = torch.exp(logits[h].double() - logits[h].double().max())
        want += e / e.sum()
    assert (got[0].double() - want).abs().max() < 1e-6
    assert abs(float(got.sum()) - 8.0) < 1e-5
    grp = orc.head_sum_scores(logits, 2)
    assert (grp.sum(0) - got[0]).abs().max() < 1e-6  # groups partition the heads
    # per-head selection: top-k of logits == top-k of softmax (monotone)
    assert torch.equal(orc.stable_topk(logits, 5), orc.stable_topk(torch.softmax(logits, -1), 5))


# ---------------------------------------------------------------------------------------------
# selection / sparse layers
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("mode,rows", [("per_head", 8), ("group_sum", 2), ("head_sum", 1)])
def test_select_and_sparse_layer_properties(mode, rows):
    hq, hkv, n, d, k = 8, 2, 300, 32, 40
    q, kk, vv = _qkv(hq, hkv, n, d, 8)
    o, idx, logits = orc.select_layer(q, kk, vv, k, mode)
    assert idx.shape == (rows, k)
    assert (o - orc.full_attention(q, kk, vv)).abs().max() < 1e-6  # selection layer attends to all
    mask = orc.mask_from_indices(idx, hq, n)
    assert mask.shape == (hq, n) and (mask.sum(-1) == k).all()
    # the reference's definition (masked_fill) == attention over the gathered rows
    q2, k2, v2 = _qkv(hq, hkv, n, d, 9)
    a = orc.sparse_layer(q2, k2, v2, mask)
    b = orc.sparse_layer_gather(q2, k2, v2, idx)
    assert (a - b).abs().max() < 1e-5
    # permutation of the list leaves the result unchanged
    perm = torch.randperm(k, generator=torch.Generator().manual_seed(1))
    assert (orc.sparse_layer_gather(q2, k2, v2, idx[:, perm]) - b).abs().max() < 1e-5
    # k = N is full attention, k = 1 returns the value row
    everything = torch.arange(n).repeat(rows, 1)
    assert (orc.sparse_layer_gather(q2, k2, v2, everything)
            - orc.full_attention(q2, k2, v2)).abs().max() < 1e-5
    one = idx[:, :1]
    got = orc.sparse_layer_gather(q2, k2, v2, one)
    for h in range(hq):
        assert torch.equal(got[h], v2[one[h * rows // hq, 0], h // (hq // hkv)])


def test_budget_clamps_to_sequence_length():
    q, k, v = _qkv(4, 4, 10, 8, 10)
    _, idx, _ = orc.select_layer(q, k, v, 256)
    assert idx.shape == (4, 10)  # token_budget = min(N, top_k)


def test_schedule_and_index_persistence():
    """full below sparse_layer_start, selection at start and correction layer, sparse elsewhere;
    lists persist until the next selection layer; a sparse layer without a list is an error."""
    sch = orc.TidalSchedule(8, sparse_layer_start=2, correction_layer=5)
    assert [sch.kind(i) for i in range(8)] == ["full", "full", "select", "sparse", "sparse",
                                               "select", "sparse", "sparse"]
    g = torch.Generator().manual_seed(11)
    qs = [torch.randn((4, 16), generator=g) for _ in range(8)]
    ks = [torch.randn((50, 4, 16), generator=g) for _ in range(8)]
    vs = [torch.randn((50, 4, 16), generator=g) for _ in range(8)]
    outs, used = orc.decode_step_layers(qs, ks, vs, sch, 7)
    assert used[0] is None and used[1] is None
    assert used[3] is used[2] and used[4] is used[2] and used[6] is used[5] and used[5] is not used[2]
    assert (outs[3] - orc.sparse_layer_gather(qs[3], ks[3], vs[3], used[2])).abs().max() < 1e-5
    bad = orc.TidalSchedule(3, sparse_layer_start=0, correction_layer=9)
    bad.kind = lambda layer: "sparse"
    with pytest.raises(ValueError):
        orc.decode_step_layers(qs[:3], ks[:3], vs[:3], bad, 7)
    # benchmark configuration: selection at layers 0 and 2
    b = orc.TidalSchedule(4, sparse_layer_start=0, correction_layer=2)
    assert [b.kind(i) for i in range(4)] == ["select", "sparse", "select", "sparse"]


# ---------------------------------------------------------------------------------------------
# RoPE
# ---------------------------------------------------------------------------------------------
def test_rope_hf_equals_transformers():
    """oracle's fp32 pipeline == the installed transformers' LlamaRotaryEmbedding + apply_rotary_pos_emb"""
    tf = pytest.importorskip("transformers")
    from transformers.models.llama.modeling_llama import LlamaRotaryEmbedding, apply_rotary_pos_emb

    cfg = tf.LlamaConfig(hidden_size=8 * 64, num_attention_heads=8, num_key_value_heads=8,
                         max_position_embeddings=4096, rope_theta=10000.0)
    rot = LlamaRotaryEmbedding(cfg)
    g = torch.Generator().manual_seed(12)
    x = torch.randn((5, 8, 64), generator=g)  # [N, H, D]
    pos = torch.tensor([0, 1, 17, 1000, 4095])
    cos, sin = rot(x, pos[None])
    want, _ = apply_rotary_pos_emb(x.transpose(0, 1)[None], x.transpose(0, 1)[None], cos, sin)
    got = orc.rope_hf(x, pos, 10000.0)
    assert (got - want[0].transpose(0, 1)).abs().max() < 1e-5


def test_rope_closed_form_invariants():
    g = np.random.default_rng(13)
    x = g.standard_normal((3, 2, 64))
    y = g.standard_normal((3, 2, 64))
    assert np.array_equal(orc.rope_closed_form(x, np.zeros(3)), x)  # position 0: identity
    r = orc.rope_closed_form(x, np.array([5, 1000, 99999]))
    pair = lambda a: a[..., :32] ** 2 + a[..., 32:] ** 2
    assert np.abs(pair(r) - pair(x)).max() < 1e-9  # rotation preserves each pair's norm
    # <R_m q, R_n k> depends only on m - n
    d1 = (orc.rope_closed_form(x, np.full(3, 50)) * orc.rope_closed_form(y, np.full(3, 20))).sum(-1)
    d2 = (orc.rope_closed_form(x, np.full(3, 90030)) * orc.rope_closed_form(y, np.full(3, 90000))).sum(-1)
    assert np.abs(d1 - d2).max() < 1e-7
    # scale divides the position
    assert np.abs(orc.rope_closed_form(x, np.full(3, 40), scale=4.0)
                  - orc.rope_closed_form(x, np.full(3, 10))).max() < 1e-12


def test_rope_reference_formulas_within_their_own_error():
    """Both fp32 formulas of the reference (model: inv_freq * pos; kernel checker: (pos/scale) /
    theta^e) stay within position * 2^-22 (+1e-5) of the float64 closed form, and agree with it
    tightly at small positions.  This bounds what 'matching the reference' can mean for RoPE."""
    g = torch.Generator().manual_seed(14)
    x = torch.randn((1, 4, 128), generator=g)
    for pos, theta in ((3, 1e4), (4095, 1e4), (32768, 1e4), (102399, 5e5)):
        exact = orc.rope_closed_form(x.numpy(), np.array([pos]), theta)
        hf = orc.rope_hf(x, torch.tensor([pos]), theta).double().numpy()
        cr = np.stack([cref.apply_llama_rope(x[0, h].numpy(), pos, 1.0, theta) for h in range(4)])[None]
        bound = (pos * 2.0 ** -22 + 1e-5) * float(x.abs().max()) * 2
        assert np.abs(hf - exact).max() <= bound
        assert np.abs(cr - exact).max() <= bound
    small = orc.rope_closed_form(x.numpy(), np.array([3]), 1e4)
    assert np.abs(orc.rope_hf(x, torch.tensor([3]), 1e4).numpy() - small).max() < 1e-5


# ---------------------------------------------------------------------------------------------
# paged addressing
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("layout", [0, 1])
def test_offsets_match_array_indexing(layout):
    """the offset formulas are the row-major strides of the documented pool shape, and the C
    restatement agrees"""
    pages, p, h, d = 5, 3, 4, 8
    shape = orc.pool_shape(pages, p, h, d, layout)
    flat = np.arange(np.prod(shape)).reshape(shape)
    for page, head, entry, feat in ((0, 0, 0, 0), (4, 3, 2, 7), (2, 1, 1, 5)):
        kk = flat[page, 0, head, entry, feat] if layout == 1 else flat[page, 0, entry, head, feat]
        vv = flat[page, 1, head, entry, feat] if layout == 1 else flat[page, 1, entry, head, feat]
        assert orc.k_elem_offset(page, head, entry, feat, h, p, d, layout) == kk
        assert orc.v_elem_offset(page, head, entry, feat, h, p, d, layout) == vv
        assert cref.lib.ref_k_elem_offset(page, head, entry, feat, h, p, d, layout) == kk
        assert cref.lib.ref_v_elem_offset(page, head, entry, feat, h, p, d, layout) == vv


@pytest.mark.parametrize("layout", [0, 1])
@pytest.mark.parametrize("page_size", [1, 3, 7, 16])
def test_append_then_gather_round_trip(layout, page_size):
    """append through a shuffled page table (numpy oracle and C restatement), then reading the
    pages in table order returns the contiguous K, V; untouched entries keep their fill"""
    g = np.random.default_rng(page_size)
    n, h, d = 53, 3, 8
    k = g.standard_normal((n, h, d)).astype(np.float32)
    v = g.standard_normal((n, h, d)).astype(np.float32)
    n_pages = (n + page_size - 1) // page_size
    table = g.permutation(n_pages + 4)[:n_pages]
    shape = orc.pool_shape(n_pages + 4, page_size, h, d, layout)
    a = np.full(shape, -7.0, dtype=np.float32)
    b = np.full(shape, -7.0, dtype=np.float32)
    # two appends: 20 tokens, then the rest
    orc.paged_append(a, table.tolist(), 20, k[:20], v[:20], layout)
    orc.paged_append(a, table.tolist(), n, k[20:], v[20:], layout)
    cref.append_paged_kv_cache(b, table, 20, k[:20], v[:20], layout)
    cref.append_paged_kv_cache(b, table, n, k[20:], v[20:], layout)
    assert np.array_equal(a, b)
    pages = a[table]
    if layout == 1:
        pages = pages.transpose(0, 1, 3, 2, 4)
    assert np.array_equal(pages[:, 0].reshape(-1, h, d)[:n], k)
    assert np.array_equal(pages[:, 1].reshape(-1, h, d)[:n], v)
    assert (pages[:, 0].reshape(-1, h, d)[n:] == -7.0).all()
    unused = np.setdiff1d(np.arange(n_pages + 4), table)
    assert (a[unused] == -7.0).all()


@pytest.mark.parametrize("layout", [0, 1])
def test_paged_selected_attention_equals_dense_on_the_same_tokens(layout):
    """numpy paged oracle == torch gather oracle == C restatement of selected_single_mha"""
    g = torch.Generator().manual_seed(15)
    n, h, d, p, budget = 203, 4, 16, 7, 6
    k = torch.randn((n, h, d), generator=g)
    v = torch.randn((n, h, d), generator=g)
    q = torch.randn((h, d), generator=g)
    n_pages = (n + p - 1) // p
    last_len = (n - 1) % p + 1
    table = torch.randperm(n_pages + 2, generator=g)[:n_pages]
    pool = np.full(orc.pool_shape(n_pages + 2, p, h, d, layout), 9.0, dtype=np.float32)
    orc.paged_append(pool, table.tolist(), n, k.numpy(), v.numpy(), layout)
    logical = torch.stack([torch.randperm(n_pages - 1, generator=g)[: budget - 1] for _ in range(h)])
    got, _ = orc.paged_selected_attention(q.numpy(), pool, table[logical].numpy(), int(table[-1]),
                                          last_len, layout, "pages")
    # the same tokens, gathered from the contiguous tensors
    pos = torch.cat([(logical[:, :, None] * p + torch.arange(p)).reshape(h, -1),
                     ((n_pages - 1) * p + torch.arange(last_len)).repeat(h, 1)], dim=1)
    want = orc.sparse_layer_gather(q, k, v, pos)
    assert np.abs(got - want.numpy()).max() < 1e-5
    sel = torch.cat([logical, torch.full((h, 1), n_pages - 1)], 1)
    kc, vc = k.numpy(), v.numpy()
    if layout == 1:
        kc, vc = kc.transpose(1, 0, 2).copy(), vc.transpose(1, 0, 2).copy()
    c = cref.selected_single_mha(q.numpy(), kc, vc, sel.numpy(), last_len, p, layout)
    assert np.abs(c - want.numpy()).max() < 1e-5
    # token-slot lists without a forced last page
    slots = table[pos // p] * p + pos % p
    got2, _ = orc.paged_selected_attention(q.numpy(), pool, slots.numpy(), 0, 0, layout, "slots")
    assert np.abs(got2 - want.numpy()).max() < 1e-5


def test_page_score_bound_properties():
    """The page estimator is an upper bound of every q.k inside the page, is tight for one-token
    pages, and equals the closed form q.(max+min)/2 + |q|.(max-min)/2."""
    g = torch.Generator().manual_seed(4)
    q = torch.randn((8, 32), generator=g)
    k = torch.randn((100, 4, 32), generator=g)
    for page in (1, 3, 16, 100):
        b = orc.page_score_bound(q, k, page)
        raw = orc.attn_logits(q, k) * math.sqrt(32)          # unscaled q.k, [8, 100]
        n_pages = (100 + page - 1) // page
        assert b.shape == (8, n_pages)
        for pg in range(n_pages):
            inside = raw[:, pg * page: (pg + 1) * page]
            assert (b[:, pg] >= inside.max(-1).values - 1e-4).all()
            if page == 1:
                assert (b[:, pg] - inside[:, 0]).abs().max() < 1e-4
            rows = k[pg * page: (pg + 1) * page]
            mx = rows.max(0).values.repeat_interleave(2, 0)
            mn = rows.min(0).values.repeat_interleave(2, 0)
            closed = (q * (mx + mn) / 2).sum(-1) + (q.abs() * (mx - mn) / 2).sum(-1)
            assert (b[:, pg] - closed).abs().max() < 1e-4

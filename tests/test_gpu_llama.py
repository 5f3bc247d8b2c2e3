"""GPU: the decoder harness (tidaldecode_amd/llama.py) against a plain fp32 torch restatement of the
same Llama forward pass with the same weights.

With top_k >= context every sparse layer attends to every token, so the TidalDecode model must
reproduce dense attention (the reference's k = N special case); tolerance is that of bf16 GEMMs
against fp32 (relative 3e-2 of the logit scale).  With a small budget the persisted lists must be
the ones the last selection layer wrote, and the logits must equal a dense-mask evaluation
(src/tidal_build/modify_llama.py:121-133) that uses those lists.
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu


def _small(**kw):
    from tidaldecode_amd.llama import TidalLlamaConfig

    base = dict(num_layers=5, hidden_size=256, num_heads=4, num_kv_heads=2, head_dim=64,
                intermediate_size=512, vocab_size=1000, rope_theta=1e4, top_k=4096,
                sparse_layer_start=1, correction_layer=3)
    base.update(kw)
    return TidalLlamaConfig(**base)


def _rope(x, pos, theta):
    d = x.shape[-1]
    inv = 1.0 / (theta ** (torch.arange(0, d, 2, device=x.device, dtype=torch.float64) / d))
    ang = pos.double()[:, None] * inv[None]
    cos, sin = torch.cat([ang.cos(), ang.cos()], -1)[:, None], torch.cat([ang.sin(), ang.sin()], -1)[:, None]
    x = x.double()
    rot = torch.cat([-x[..., d // 2:], x[..., : d // 2]], -1)
    return (x * cos + rot * sin).float()


def _reference_logits(model, ids, masks=None):
    """fp32 forward of the whole sequence; returns logits of the last position and per-layer
    (q_last, k, v).  masks: optional {layer: [H, N] 0/1} applied to the last position's attention."""
    c = model.config
    f = lambda t: t.float()
    n = ids.numel()
    pos = torch.arange(n, device=ids.device)
    x = f(model.embed)[ids]
    rms = lambda t, w: t * torch.rsqrt(t.pow(2).mean(-1, keepdim=True) + c.rms_norm_eps) * f(w)
    for idx, layer in enumerate(model.layers):
        h = rms(x, layer["ln1"])
        qkv = h @ f(layer["wqkv"]).t()
        qe, ke = c.num_heads * c.head_dim, (c.num_heads + c.num_kv_heads) * c.head_dim
        q = _rope(qkv[:, :qe].reshape(n, c.num_heads, c.head_dim), pos, c.rope_theta)
        k = _rope(qkv[:, qe:ke].reshape(n, c.num_kv_heads, c.head_dim), pos, c.rope_theta)
        v = qkv[:, ke:].reshape(n, c.num_kv_heads, c.head_dim)
        g = c.num_heads // c.num_kv_heads
        kk, vv = k.repeat_interleave(g, 1), v.repeat_interleave(g, 1)
        logit = torch.einsum("qhd,khd->hqk", q, kk) / math.sqrt(c.head_dim)
        causal = torch.ones(n, n, device=ids.device).tril().bool()
        logit = logit.masked_fill(~causal, float("-inf"))
        if masks is not None and idx in masks:
            logit[:, -1] = logit[:, -1].masked_fill(masks[idx] == 0, torch.finfo(torch.float32).min)
        o = torch.einsum("hqk,khd->qhd", logit.softmax(-1), vv).reshape(n, -1)
        x = x + o @ f(layer["wo"]).t()
        h2 = rms(x, layer["ln2"])
        gu = h2 @ f(layer["w_gate_up"]).t()
        x = x + (torch.nn.functional.silu(gu[:, : c.intermediate_size]) * gu[:, c.intermediate_size:]) @ f(layer["w_down"]).t()
    return (rms(x[-1:], model.norm) @ f(model.lm_head).t())[0]


def _close(got, want, rel=3e-2):
    scale = want.abs().max().item()
    return (got.float() - want).abs().max().item() <= rel * scale


@pytest.mark.parametrize("use_gemv", [True, False])
@pytest.mark.parametrize("select_mode", ["per_head", "head_sum"])
def test_budget_covering_the_context_equals_dense_attention(cuda, select_mode, use_gemv):
    """use_gemv: the fused matrix-vector launches of the library; otherwise torch GEMMs"""
    from tidaldecode_amd.llama import TidalLlama

    torch.manual_seed(0)
    model = TidalLlama(_small(select_mode=select_mode), cuda, seed=1, init_std=0.05)
    model.use_gemv = use_gemv
    model.tidal_init(page_size=16, max_seq_len=256, page_order_seed=3)
    ids = torch.randint(0, 1000, (70,), device=cuda)
    logits = model.prefill(ids)
    assert _close(logits, _reference_logits(model, ids))
    seq = ids
    for _ in range(5):  # greedy steps, each compared with a fresh dense forward
        tok = logits.argmax().view(1)
        seq = torch.cat([seq, tok])
        logits = model.decode_step(tok)
        assert _close(logits, _reference_logits(model, seq))
    assert model.iController.kv_cache.seqlen == 75
    assert len(model.iController.decode_latency) == 5 and len(model.iController.prefill_latency) == 1
    model.tidal_clear()
    assert model.iController.kv_cache.seqlen == 0


@pytest.mark.parametrize("head_dim,page", [(64, 16), (128, 8)])
def test_quest_style_decoder_with_every_page_in_budget_equals_dense_attention(cuda, head_dim, page):
    """attn_type "quest" (the comparison bar of the reference's end-to-end figure): with a page
    budget that covers the cache, the chosen pages plus the page being filled are every token, so
    the decoder must reproduce dense attention; with a small budget it still runs and differs."""
    from tidaldecode_amd.llama import TidalLlama

    torch.manual_seed(0)
    cfg = _small(head_dim=head_dim, hidden_size=4 * head_dim)
    cfg.attn_type = "quest"
    model = TidalLlama(cfg, cuda, seed=4, init_std=0.05)
    model.tidal_init(page_size=page, max_seq_len=256, page_order_seed=2, with_metadata=True)
    ids = torch.randint(0, 1000, (70,), device=cuda)
    logits = model.prefill(ids)
    assert _close(logits, _reference_logits(model, ids))
    seq = ids
    for _ in range(4):
        tok = logits.argmax().view(1)
        seq = torch.cat([seq, tok])
        logits = model.decode_step(tok)
        assert _close(logits, _reference_logits(model, seq))
    model.iController.set_token_budget(2 * page)      # two pages + the one being filled
    tok = logits.argmax().view(1)
    few = model.decode_step(tok)
    assert torch.isfinite(few).all() and not _close(few, _reference_logits(model, torch.cat([seq, tok])), rel=1e-3)
    model.tidal_clear()


def test_sparse_layers_use_the_persisted_lists(cuda):
    """small budget: logits equal a dense evaluation masked with the lists the selection layers
    wrote (layers 2 and 4 reuse the lists of layers 1 and 3)"""
    from tidaldecode_amd.llama import TidalLlama
    from tidaldecode_amd import utils as ops

    cfg = _small(top_k=12)
    model = TidalLlama(cfg, cuda, seed=2, init_std=0.05)
    model.tidal_init(page_size=4, max_seq_len=128, page_order_seed=1)
    ids = torch.randint(0, 1000, (60,), device=cuda)
    logits = model.prefill(ids)
    tok = logits.argmax().view(1)
    seq = torch.cat([ids, tok])
    # record the list after every selection layer
    lists, orig = {}, ops.decode_topk

    def spy(ctrl):
        orig(ctrl)
        lists[len(lists)] = ctrl.topk_dindices_buffer.clone()

    import tidaldecode_amd.llama as mod
    mod.tidal_utils.decode_topk = spy
    try:
        got = model.decode_step(tok)
    finally:
        mod.tidal_utils.decode_topk = orig
    assert len(lists) == 2 and lists[0].shape == (4, 12)
    ctrl = model.iController
    table = ctrl.kv_cache.indices_device.long()
    inv = torch.full((int(table.max()) + 1,), -1, device=cuda)
    inv[table] = torch.arange(table.numel(), device=cuda)

    def mask_of(slots):
        pos = inv[slots.long() // 4] * 4 + slots.long() % 4
        assert (pos >= 0).all() and (pos < 61).all()
        return torch.zeros(4, 61, device=cuda).scatter_(1, pos, 1.0)

    masks = {2: mask_of(lists[0]), 4: mask_of(lists[1])}
    assert (masks[2].sum(1) == 12).all()
    assert _close(got, _reference_logits(model, seq, masks))
    # and the result is not what dense attention gives
    assert not _close(got, _reference_logits(model, seq), rel=1e-3)


def test_layer_schedule_and_full_mode(cuda):
    from tidaldecode_amd.llama import TidalLlama, TidalLlamaConfig

    c = TidalLlamaConfig(num_layers=6, sparse_layer_start=0, correction_layer=2)
    assert [c.layer_kind(i) for i in range(6)] == ["select", "sparse", "select", "sparse", "sparse", "sparse"]
    c = TidalLlamaConfig(num_layers=4, sparse_layer_start=2, correction_layer=13)
    assert [c.layer_kind(i) for i in range(4)] == ["full", "full", "select", "sparse"]
    cfg = _small(top_k=8, attn_type="full")
    assert all(cfg.layer_kind(i) == "full" for i in range(5))
    model = TidalLlama(cfg, cuda, seed=3, init_std=0.05)
    model.tidal_init(page_size=16, max_seq_len=128)
    ids = torch.randint(0, 1000, (40,), device=cuda)
    logits = model.prefill(ids)
    tok = logits.argmax().view(1)
    assert _close(model.decode_step(tok), _reference_logits(model, torch.cat([ids, tok])))
    dt, how = model.timed_decode(steps=3, warmup=1)
    assert dt > 0 and how in ("hipGraph", "eager")


@pytest.mark.parametrize("select_mode,top_k", [("per_head", 4096), ("head_sum", 4096), ("per_head", 12),
                                               ("group_sum", 24)])
def test_generation_by_replaying_one_captured_step(cuda, select_mode, top_k):
    """generate_graph: the step state lives on the device and one captured step is replayed per
    token.  Every replay must give what the same step gives when launched eagerly (bit for bit:
    same kernels, same plans), and the logits must be those of the host-driven decode_step fed
    with the same tokens (another split plan: bf16 tolerance; with a small budget a near-tie in
    the selection may pick another token, so that comparison is looser)."""
    from tidaldecode_amd import _lib
    from tidaldecode_amd.llama import TidalLlama

    n_prompt, n_new = 70, 40   # crosses two page boundaries
    model = TidalLlama(_small(select_mode=select_mode, top_k=top_k), cuda, seed=4, init_std=0.05)
    model.tidal_init(page_size=16, max_seq_len=256, page_order_seed=5)
    ids = torch.randint(0, 1000, (n_prompt,), device=cuda, generator=torch.Generator(device=cuda).manual_seed(9))
    tokens, kept = model.generate_graph(ids, n_new, keep_logits=True)
    assert model.iController.kv_cache.seqlen == n_prompt + n_new
    model.tidal_clear()
    tokens_e, kept_e = model.generate_graph(ids, n_new, keep_logits=True, use_graph=False)
    assert torch.equal(tokens, tokens_e) and torch.equal(kept, kept_e)
    assert torch.equal(tokens[1:], kept[:-1].argmax(-1))       # greedy: each row chose the next token
    model.tidal_clear()
    # host-driven steps with the same tokens
    logits = model.prefill(ids)
    assert int(logits.argmax()) == int(tokens[0])
    rel = 2e-2 if top_k >= 4096 else 1e-1
    for i in range(n_new):
        logits = model.decode_step(tokens[i: i + 1])
        assert _close(kept[i], logits.float(), rel=rel), i
    model.tidal_clear()
    assert model._dev is None


@pytest.mark.parametrize("heads,kv,hd,page,mode,gemv", [(8, 2, 128, 5, "group_sum", True),    # un-fused step
                                                         (6, 2, 128, 16, "head_sum", False),  # padded group
                                                         (2, 1, 256, 1, "per_head", True),
                                                         (8, 2, 64, 16, "group_sum", True),   # shared rows, head_dim 64
                                                         (6, 2, 256, 16, "head_sum", True)])  # padded group, head_dim 256
def test_replayed_generation_on_other_shapes(cuda, heads, kv, hd, page, mode, gemv):
    """Page sizes without a fused step (RoPE + append as their own launch, positions and slots
    read from the device state), shared-row and padded query groups, head_dim 256."""
    from tidaldecode_amd.llama import TidalLlama

    cfg = _small(num_heads=heads, num_kv_heads=kv, head_dim=hd, select_mode=mode, top_k=10)
    model = TidalLlama(cfg, cuda, seed=4, init_std=0.05)
    model.use_gemv = gemv
    model.tidal_init(page_size=page, max_seq_len=160, page_order_seed=5)
    ids = torch.randint(0, 1000, (50,), device=cuda, generator=torch.Generator(device=cuda).manual_seed(9))
    tokens, kept = model.generate_graph(ids, 30, keep_logits=True)
    model.tidal_clear()
    tokens_e, kept_e = model.generate_graph(ids, 30, keep_logits=True, use_graph=False)
    assert torch.equal(tokens, tokens_e) and torch.equal(kept, kept_e)
    model.tidal_clear()
    logits = model.prefill(ids)
    assert int(logits.argmax()) == int(tokens[0])
    for i in range(30):
        logits = model.decode_step(tokens[i: i + 1])
        assert _close(kept[i], logits.float(), rel=1.5e-1), i


def test_replays_with_eager_work_in_between_and_a_large_vocabulary(cuda):
    """A 32000-entry vocabulary (the size the token choice runs at in the benchmark) and, between
    the replays, synchronisations and eager launches of the program's own: every replay must
    still give what the eagerly launched step gives."""
    from tidaldecode_amd.llama import TidalLlama

    model = TidalLlama(_small(vocab_size=32000, top_k=16, num_layers=3, correction_layer=2), cuda,
                       seed=6, init_std=0.05)
    model.tidal_init(page_size=16, max_seq_len=128, page_order_seed=2)
    ids = torch.randint(0, 32000, (50,), device=cuda, generator=torch.Generator(device=cuda).manual_seed(3))
    junk = torch.randn(1 << 16, device=cuda)

    def between():
        torch.cuda.synchronize()
        junk.mul_(1.0001).sum().item()      # eager work, a multi-block reduction and a host sync

    tokens, kept = model.generate_graph(ids, 24, keep_logits=True, between_steps=between)
    model.tidal_clear()
    tokens_e, kept_e = model.generate_graph(ids, 24, keep_logits=True, use_graph=False)
    assert torch.equal(tokens, tokens_e) and torch.equal(kept, kept_e)
    assert torch.equal(tokens[1:], kept[:-1].argmax(-1))


def test_argmax_kernel(cuda):
    from tidaldecode_amd import _kernels

    g = torch.Generator().manual_seed(1)
    out = torch.zeros(1, dtype=torch.int64, device=cuda)
    for dtype in (torch.float32, torch.float16, torch.bfloat16):
        for n in (1, 63, 1000, 32000, 128256):
            x = torch.randn(n, generator=g).to(dtype)
            _kernels.argmax(x.to(cuda), out)
            assert int(out) == int(x.float().argmax()), (dtype, n)   # CPU argmax: first maximum
        x = torch.zeros(5000, dtype=dtype)
        x[[77, 4000, 1234]] = 3.0                                     # ties: the lowest index
        _kernels.argmax(x.to(cuda), out)
        assert int(out) == 77
        x[2222] = float("nan")                                        # NaN ranks highest
        _kernels.argmax(x.to(cuda), out)
        assert int(out) == 2222
        x[10] = float("inf")                                          # ... on a par with +inf
        _kernels.argmax(x.to(cuda), out)
        assert int(out) == 10
    with pytest.raises(RuntimeError):
        _kernels.argmax(torch.zeros(4, device=cuda), torch.zeros(1, dtype=torch.int32, device=cuda))


def test_step_state_words(cuda):
    from tidaldecode_amd import _kernels, _lib

    table = torch.tensor([7, 3, 9, 1], dtype=torch.int32, device=cuda)
    state = torch.zeros(_lib.TD_STEP_WORDS, dtype=torch.int32, device=cuda)
    state[_lib.TD_STEP_SEQ_LEN] = 6
    token = torch.tensor([41], dtype=torch.int64, device=cuda)
    out = torch.full((5,), -1, dtype=torch.int64, device=cuda)
    want = []
    for step in range(7):   # lengths 7 .. 13 with pages of 4
        token.fill_(100 + step)
        _kernels.step_advance(state, table, 4, 10, token, out)
        n = 7 + step
        pos = n - 1
        page = [7, 3, 9, 1][pos // 4]
        want = [n, pos // 4, pos % 4 + 1, page, page * 4 + pos % 4, pos, min(10, n), step + 1]
        assert state.tolist() == want, step
    assert out.tolist() == [100, 101, 102, 103, 104]          # recording stops at the capacity
    with pytest.raises(RuntimeError):
        _kernels.step_advance(state, table, 4, 10, token, None)

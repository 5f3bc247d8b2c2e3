"""GPU: enable_tidal() on a Hugging Face LlamaForCausalLM with random weights (the installed
transformers; the reference pins 4.45 whose attention classes no longer exist)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _tiny(cuda, dtype=torch.bfloat16):
    tf = pytest.importorskip("transformers")
    cfg = tf.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=5,
                         num_attention_heads=4, num_key_value_heads=2, head_dim=64, vocab_size=1000,
                         max_position_embeddings=512, rope_theta=10000.0)
    torch.manual_seed(0)
    model = tf.LlamaForCausalLM(cfg).to(dtype).to(cuda).eval()
    return model


def _close(a, b, rel=4e-2):
    return (a.float() - b.float()).abs().max().item() <= rel * b.float().abs().max().item()


@torch.no_grad()
def test_same_signature_and_patching(cuda):
    import inspect

    from tidaldecode_amd.enable_tidal import enable_tidal

    sig = inspect.signature(enable_tidal)
    assert list(sig.parameters)[:5] == ["model", "attn_type", "top_k", "sparse_layer_start",
                                        "correction_layer"]
    assert (sig.parameters["top_k"].default, sig.parameters["sparse_layer_start"].default,
            sig.parameters["correction_layer"].default) == (256, 2, 13)
    model = _tiny(cuda)
    state = enable_tidal(model, top_k=64, sparse_layer_start=1, correction_layer=3, page_size=16)
    attn = model.model.layers[0].self_attn
    assert hasattr(attn, "flash_forward") and attn._tidal_state is state
    assert [state.layer_kind(i) for i in range(5)] == ["full", "select", "sparse", "select", "sparse"]


@torch.no_grad()
def test_incremental_decode_matches_the_unpatched_model(cuda):
    """budget >= context: prefill + cached decode through the paged kernels must reproduce the
    stock model's logits on the full sequence"""
    from tidaldecode_amd.enable_tidal import enable_tidal

    ref = _tiny(cuda)
    model = _tiny(cuda)
    model.load_state_dict(ref.state_dict())
    enable_tidal(model, top_k=4096, sparse_layer_start=1, correction_layer=3, page_size=16,
                 max_seq_len=256)
    ids = torch.randint(0, 1000, (1, 50), device=cuda)
    out = model(ids, use_cache=True)
    assert _close(out.logits[0, -1], ref(ids).logits[0, -1])
    past, seq = out.past_key_values, ids
    for _ in range(4):
        tok = out.logits[0, -1].argmax().view(1, 1)
        seq = torch.cat([seq, tok], dim=1)
        out = model(tok, past_key_values=past, use_cache=True)
        past = out.past_key_values
        assert past.get_seq_length() == seq.shape[1]
        assert _close(out.logits[0, -1], ref(seq).logits[0, -1])
    assert model._tidal_state.controller.kv_cache.seqlen == 54


@torch.no_grad()
def test_other_attention_types_leave_forward_alone(cuda):
    """modify_llama.py:365-367: forward is replaced only for attn_type == "tidal"; any other value
    only stores the original under flash_forward.  enable_llama_tidal_attention's own default
    for the re-selection layer is 9 (modify_llama.py:331-333), enable_tidal's is 13."""
    import inspect

    from tidaldecode_amd.enable_tidal import enable_llama_tidal_attention, enable_tidal

    assert inspect.signature(enable_llama_tidal_attention).parameters["correction_layer"].default == 9
    ref, model = _tiny(cuda), _tiny(cuda)
    model.load_state_dict(ref.state_dict())
    before = [layer.self_attn.forward.__func__ for layer in model.model.layers]
    enable_tidal(model, attn_type="quest", top_k=8, sparse_layer_start=1, correction_layer=3)
    for layer, fn in zip(model.model.layers, before):
        assert layer.self_attn.forward.__func__ is fn
        assert layer.self_attn.flash_forward.__func__ is fn
    ids = torch.randint(0, 1000, (1, 30), device=cuda)
    assert torch.equal(model(ids).logits, ref(ids).logits)


def _dense_reference_logits(model, seq, masks):
    """fp32 evaluation of the Hugging Face model on the whole sequence, token by token causal; in
    the layers named by `masks` the LAST token attends only where masks[layer][head, pos] == 1
    (masked_fill before the softmax, modify_llama.py:125-128).  Returns the last token's logits."""
    import copy

    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb, repeat_kv

    ref = copy.deepcopy(model).float()
    t = seq.numel()
    h = ref.model.embed_tokens(seq[None])
    pos = torch.arange(t, device=seq.device)[None]
    cos, sin = ref.model.rotary_emb(h, pos)
    causal = torch.full((t, t), float("-inf"), device=seq.device).triu(1)
    cfg = ref.config
    hq, hkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim
    for i, layer in enumerate(ref.model.layers):
        x = layer.input_layernorm(h)
        att = layer.self_attn
        q = att.q_proj.forward(x).view(1, t, hq, d).transpose(1, 2)
        k = att.k_proj.forward(x).view(1, t, hkv, d).transpose(1, 2)
        v = att.v_proj.forward(x).view(1, t, hkv, d).transpose(1, 2)
        q, k = apply_rotary_pos_emb(q, k, cos, sin)
        k, v = repeat_kv(k, hq // hkv), repeat_kv(v, hq // hkv)
        logits = q @ k.transpose(-1, -2) / d ** 0.5 + causal
        if i in masks:
            logits[0, :, -1, :] = logits[0, :, -1, :].masked_fill(masks[i] == 0, float("-inf"))
        o = torch.softmax(logits, -1) @ v
        h = h + att.o_proj.forward(o.transpose(1, 2).reshape(1, t, hq * d))
        h = h + layer.mlp(layer.post_attention_layernorm(h))
    return ref.lm_head(ref.model.norm(h))[0, -1]


@torch.no_grad()
@pytest.mark.parametrize("page_size", [4, 16])
def test_small_budget_decode_matches_a_dense_forward_masked_by_the_recorded_lists(cuda, page_size):
    """budget 8 of 41..44 tokens: every decode step's logits must equal a dense fp32 forward whose
    sparse layers (2 and 4) see only the tokens that the selection layers (1 and 3) of the same
    step wrote into the controller -- the hand-off of llama_tidaldecoding.py:983-985,1019 -- and
    must differ from the unmasked dense forward."""
    import tidaldecode_amd.enable_tidal as mod
    from tidaldecode_amd.enable_tidal import enable_tidal

    model = _tiny(cuda)
    state = enable_tidal(model, top_k=8, sparse_layer_start=1, correction_layer=3,
                         page_size=page_size, max_seq_len=256)
    plain = _tiny(cuda)
    plain.load_state_dict(model.state_dict())
    ids = torch.randint(0, 1000, (1, 40), device=cuda)
    out = model(ids, use_cache=True)
    past, seq = out.past_key_values, ids[0]
    orig, differs = mod.tidal_utils.decode_topk, 0
    for step in range(4):
        tok = out.logits[0, -1].argmax().view(1, 1)
        seq = torch.cat([seq, tok[0]])
        lists = []

        def spy(ctrl):
            orig(ctrl)
            lists.append(ctrl.topk_dindices_buffer.clone())

        mod.tidal_utils.decode_topk = spy
        try:
            out = model(tok, past_key_values=past, use_cache=True)
        finally:
            mod.tidal_utils.decode_topk = orig
        past = out.past_key_values
        ctrl = state.controller
        t = seq.numel()
        assert len(lists) == 2 and lists[0].shape == (4, 8) and ctrl.kv_cache.seqlen == t
        table = ctrl.kv_cache.indices_device.long()
        inv = torch.full((int(table.max()) + 1,), -1, device=cuda)
        inv[table] = torch.arange(table.numel(), device=cuda)

        def mask_of(slots):
            pos = inv[slots.long() // page_size] * page_size + slots.long() % page_size
            assert (pos >= 0).all() and (pos < t).all()
            m = torch.zeros(4, t, device=cuda).scatter_(1, pos, 1.0)
            assert (m.sum(1) == 8).all()          # eight distinct tokens per head
            return m

        want = _dense_reference_logits(plain, seq, {2: mask_of(lists[0]), 4: mask_of(lists[1])})
        assert _close(out.logits[0, -1], want), step
        differs += not _close(out.logits[0, -1], _dense_reference_logits(plain, seq, {}), rel=1e-3)
    assert differs == 4


@torch.no_grad()
def test_generate_runs_with_a_small_budget(cuda):
    from tidaldecode_amd.enable_tidal import enable_tidal

    model = _tiny(cuda)
    state = enable_tidal(model, top_k=8, sparse_layer_start=1, correction_layer=3, page_size=4,
                         max_seq_len=256)
    ids = torch.randint(0, 1000, (1, 40), device=cuda)
    out = model.generate(ids, max_new_tokens=6, do_sample=False)
    assert out.shape == (1, 46)
    assert state.controller.num_selected == 8
    # a second, independent prompt restarts the paged cache
    out2 = model.generate(ids[:, :20], max_new_tokens=3, do_sample=False)
    assert out2.shape == (1, 23) and state.controller.kv_cache.seqlen == 22

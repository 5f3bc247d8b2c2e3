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

"""``enable_tidal(model, ...)``: switch a Hugging Face Llama model to TidalDecode attention
(counterpart of src/enable_tidal.py:1-12 and enable_llama_tidal_attention,
src/tidal_build/modify_llama.py:331-392 of the reference; same keyword arguments and defaults).

The reference replaces ``forward`` of every attention module by a closure that carries
``(top_k, sparse_layer_start, correction_layer)`` and keeps the original as ``flash_forward``
(modify_llama.py:336-369); the mask chosen by a selection layer travels from layer to layer as
``pos_dict`` (src/models/llama_tidaldecoding.py:983-985,1019).  Here the closure drives the
library's kernels over a paged KV cache that is shared by all layers through one state object
on the model, and the persisted selection is the token list inside that state:

    prefill (q_len > 1)            K/V appended to the paged cache, causal attention kernel over it
    decode, layer < sparse_layer_start                 full attention kernel
    decode, layer == sparse_layer_start / correction   full attention + logits -> top-k
    decode, other layers                               sparse attention over the persisted list

Rotary embedding uses the cos/sin the model computes, so every RoPE variant of the model works;
in decode steps they go, with the un-rotated q and k, into the fused launch (RoPE + cache append +
attention in one kernel) wherever the cache geometry allows it.  Batch size 1 and no padding, as
the reference's kernel path (tidal/ops/csrc/approx_attn.cu:33,78): ``attention_mask`` is not
consulted, the attention is causal over everything cached.  As in the reference
(modify_llama.py:365-367) ``forward`` is replaced only for ``attn_type == "tidal"``; any other value
just leaves the original under ``flash_forward``.
"""
import types
from typing import Optional

import torch

from . import utils as tidal_utils
from .utils import InferenceController


class TidalState:
    """Per-model state: controller + paged cache, created at the first forward."""

    def __init__(self, top_k, sparse_layer_start, correction_layer, page_size, max_seq_len,
                 select_mode):
        self.top_k = top_k
        self.sparse_layer_start = sparse_layer_start
        self.correction_layer = correction_layer
        self.page_size = page_size
        self.max_seq_len = max_seq_len
        self.select_mode = select_mode
        self.controller: Optional[InferenceController] = None
        self.first_layer = None
        self.last_layer = None
        self.step_len = 0
        self.dst_slot = None   # device int32 [1]: slot of the token being decoded (fused step)

    def layer_kind(self, layer_idx: int) -> str:
        if layer_idx < self.sparse_layer_start:
            return "full"
        if layer_idx in (self.sparse_layer_start, self.correction_layer):
            return "select"
        return "sparse"

    def ensure(self, config, dtype, device):
        if self.controller is None:
            head_dim = getattr(config, "head_dim", None) or config.hidden_size // config.num_attention_heads
            max_len = self.max_seq_len or config.max_position_embeddings
            self.controller = InferenceController(
                config.num_hidden_layers, config.num_attention_heads, head_dim, self.page_size,
                self.top_k, max_len, dtype, device, num_kv_heads=config.num_key_value_heads,
                select_mode=self.select_mode, select_scope="all")
        return self.controller

    def reset(self):
        """Forget the cached sequence (call between independent generations)."""
        if self.controller is not None:
            self.controller.clean_states()


def _rotate_half(x):
    d = x.shape[-1] // 2
    return torch.cat((-x[..., d:], x[..., :d]), dim=-1)


def _tidal_attention_forward(self, hidden_states, position_embeddings=None, attention_mask=None,
                             past_key_values=None, **kwargs):
    state: TidalState = self._tidal_state
    bsz, q_len, _ = hidden_states.shape
    if bsz != 1:
        raise NotImplementedError("TidalDecode attention supports batch size 1")
    cfg = self.config
    ctrl = state.ensure(cfg, hidden_states.dtype, hidden_states.device)
    hq, hkv, d = cfg.num_attention_heads, cfg.num_key_value_heads, self.head_dim

    q = self.q_proj(hidden_states).view(q_len, hq, d)
    k = self.k_proj(hidden_states).view(q_len, hkv, d)
    v = self.v_proj(hidden_states).view(q_len, hkv, d).contiguous()
    cos, sin = position_embeddings  # [1, q_len, D]

    if self.layer_idx == state.first_layer:
        # a model forward starts; whenever the framework's cache is empty (or absent) it is a new
        # sequence and the paged cache starts over, whatever the length of the input
        if past_key_values is None or past_key_values.get_seq_length(self.layer_idx) == 0:
            state.reset()
        ctrl.prepare_metadata(q_len)
        ctrl.begin_forward(q_len)
        state.step_len = q_len
        if q_len == 1 and ctrl.fused_step_ok:
            pos = ctrl.kv_cache.seqlen - 1
            slot = ctrl.kv_cache.indicies[pos // ctrl.page_size] * ctrl.page_size + pos % ctrl.page_size
            state.dst_slot = torch.tensor([slot], dtype=torch.int32, device=hidden_states.device)
    fused = q_len == 1 and ctrl.fused_step_ok
    if fused:
        # the launch rotates q and k itself, with the model's own cos/sin (first half of the
        # duplicated table), and writes k, v into the cache
        half = d // 2
        fresh = (k.contiguous(), v, cos[0, :, :half].float().contiguous(),
                 sin[0, :, :half].float().contiguous(), state.dst_slot)
        k_cache = k
        q = q.contiguous()
    else:
        fresh = None
        cos, sin = cos[0].unsqueeze(1), sin[0].unsqueeze(1)
        q = (q * cos + _rotate_half(q) * sin).contiguous()
        k = (k * cos + _rotate_half(k) * sin).contiguous()
        k_cache = k
    if past_key_values is not None:
        # keep the framework's cache length in step (generation code derives positions from it);
        # one element per row is enough for that, the real K/V live in the paged cache
        past_key_values.update(k_cache.transpose(0, 1)[None, :, :, :1],
                               v.transpose(0, 1)[None, :, :, :1], self.layer_idx)

    if not fused:
        tidal_utils.append_kv(k, v, ctrl, self.layer_idx)
    if q_len > 1:
        o = tidal_utils.prefill_forward(q, ctrl, self.layer_idx)
    else:
        kind = state.layer_kind(self.layer_idx)
        if kind == "sparse":
            o = tidal_utils.decode_sparse_attn(q, ctrl, self.layer_idx, ctrl.topk_dindices_buffer,
                                               False, fresh=fresh)
        else:
            o = tidal_utils.decode_sparse_attn(q, ctrl, self.layer_idx,
                                               ctrl.kv_indices_without_last, kind == "select",
                                               fresh=fresh)
            if kind == "select":
                tidal_utils.decode_topk(ctrl)
    if self.layer_idx == state.last_layer:
        ctrl.end_forward()
    out = self.o_proj(o.reshape(1, q_len, hq * d))
    return out, None


def enable_llama_tidal_attention(model, top_k, attn_type="tidal", sparse_layer_start=2,
                                 correction_layer=9, *, page_size=16, max_seq_len=None,
                                 select_mode="per_head"):
    """Arguments and defaults of the reference's function of this name (modify_llama.py:331-333:
    ``correction_layer=9`` here, 13 in ``enable_tidal``)."""
    state = TidalState(top_k, sparse_layer_start, correction_layer, page_size, max_seq_len,
                       select_mode)
    layers = []
    for module in model.modules():
        if type(module).__name__ == "LlamaAttention" and hasattr(module, "layer_idx"):
            layers.append(module)
    if not layers:
        raise ValueError("no LlamaAttention modules found")
    state.first_layer = min(m.layer_idx for m in layers)
    state.last_layer = max(m.layer_idx for m in layers)
    for module in layers:
        module._tidal_state = state
        module.flash_forward = module.forward  # the reference keeps the original under this name
        if attn_type == "tidal":                # modify_llama.py:365-367
            module.forward = types.MethodType(_tidal_attention_forward, module)
    model._tidal_state = state
    return state


def enable_tidal(model, attn_type="tidal", top_k=256, sparse_layer_start=2, correction_layer=13,
                 **extensions):
    """Same signature as the reference's ``enable_tidal``.  Keyword-only extensions:
    ``page_size`` (16), ``max_seq_len`` (model's max_position_embeddings), ``select_mode``
    ("per_head")."""
    model_type = model.config.model_type
    print(f"token budget: {top_k}")
    print(f"sparse layer starts from: Layer {sparse_layer_start}")
    print(f"reselection layer: {correction_layer}")
    if "llama" in model_type:
        return enable_llama_tidal_attention(model, top_k, attn_type, sparse_layer_start,
                                            correction_layer, **extensions)
    return None

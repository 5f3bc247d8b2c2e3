"""Llama-style decoder whose attention runs through the TidalDecode operator surface
(counterpart of the decode driver in the reference: tidal/models/llama.py:498-578 for the layer
loop and budget handling, tidal/models/{Full,Search,Sparse}Attention.py:131-190 for the three
attention flavours, scripts/bench_textgen.py:41-101 for the latency harness).

Only what the decode-attention path needs is here: random-initialised weights of a given
shape (there is no checkpoint loading), torch GEMMs and norms around the library's kernels, and
the layer schedule of the PyTorch path of the reference (src/tidal_build/modify_llama.py:84,116):

    layer <  sparse_layer_start                      full attention
    layer == sparse_layer_start or correction_layer  full attention + token selection
    otherwise                                         sparse attention over the persisted tokens
"""
import time
from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _kernels, _lib
from . import utils as tidal_utils
from .utils import InferenceController


@dataclass
class TidalLlamaConfig:
    num_layers: int = 32
    hidden_size: int = 4096
    num_heads: int = 32
    num_kv_heads: int = 32
    head_dim: int = 128
    intermediate_size: int = 11008
    vocab_size: int = 32000
    rope_theta: float = 1e4
    rope_scale: float = 1.0
    rms_norm_eps: float = 1e-5
    # TidalDecode
    top_k: int = 256
    sparse_layer_start: int = 2
    correction_layer: int = 13
    select_mode: str = "per_head"
    # "tidal", "full" (every layer attends to the whole cache) or "quest" (the comparison bar of the
    # reference's latency figures: full attention in layers 0 and 1, then per layer a page-score
    # estimate, the best pages and attention over those pages plus the one being filled)
    attn_type: str = "tidal"
    dtype: torch.dtype = torch.bfloat16

    @staticmethod
    def llama2_7b(**kw):
        return TidalLlamaConfig(32, 4096, 32, 32, 128, 11008, 32000, 1e4, **kw)

    @staticmethod
    def llama3_8b(**kw):
        return TidalLlamaConfig(32, 4096, 32, 8, 128, 14336, 128256, 5e5, **kw)

    @staticmethod
    def cfg4(**kw):
        """The deep decoder of the latency sweep: 64 layers, hidden 5120, 40 heads (MHA), MLP width
        of the 13B Llama."""
        return TidalLlamaConfig(64, 5120, 40, 40, 128, 13824, 32000, 1e4, **kw)

    def layer_kind(self, layer: int) -> str:
        if self.attn_type == "quest":
            return "full" if layer < 2 else "quest"
        if self.attn_type == "full" or layer < self.sparse_layer_start:
            return "full"
        if layer in (self.sparse_layer_start, self.correction_layer):
            return "select"
        return "sparse"


class TidalLlama:
    """Decoder with random weights.  ``tidal_init`` allocates the paged cache and controller,
    ``prefill`` / ``synthetic_prefill`` fills it, ``decode_step`` produces next-token logits."""

    def __init__(self, config: TidalLlamaConfig, device, seed: int = 0, init_std: float = 0.02):
        self.config = c = config
        self.device = torch.device(device)
        g = torch.Generator(device=self.device).manual_seed(seed)

        def w(*shape):
            return (torch.randn(shape, generator=g, device=self.device) * init_std).to(c.dtype)

        qkv_out = (c.num_heads + 2 * c.num_kv_heads) * c.head_dim
        self.embed = w(c.vocab_size, c.hidden_size)
        self.layers = []
        for _ in range(c.num_layers):
            self.layers.append(dict(
                ln1=torch.ones(c.hidden_size, dtype=c.dtype, device=self.device),
                wqkv=w(qkv_out, c.hidden_size),
                wo=w(c.hidden_size, c.num_heads * c.head_dim),
                ln2=torch.ones(c.hidden_size, dtype=c.dtype, device=self.device),
                w_gate_up=w(2 * c.intermediate_size, c.hidden_size),
                w_down=w(c.hidden_size, c.intermediate_size),
            ))
        self.norm = torch.ones(c.hidden_size, dtype=c.dtype, device=self.device)
        self.lm_head = w(c.vocab_size, c.hidden_size)
        self.iController: Optional[InferenceController] = None
        self._positions = torch.zeros(1, dtype=torch.int32, device=self.device)
        self._dst_slot = torch.zeros(1, dtype=torch.int32, device=self.device)
        self._cos = torch.zeros((1, c.head_dim // 2), dtype=torch.float32, device=self.device)
        self._sin = torch.zeros((1, c.head_dim // 2), dtype=torch.float32, device=self.device)
        self.fuse_decode_step = True  # RoPE + append inside the attention launch when possible
        # batch-1 decode: one launch per projection with the norm / gate / residual folded in
        # (False: torch GEMMs and separate element-wise kernels, as the reference's driver)
        self.use_gemv = True
        # set by generate_graph: the sequence's step state lives on the device and every launch of
        # a decode step reads it there, so one captured step serves every token
        self._dev = None
        self._quest = None  # per-step state of the Quest-style steps (begin_decode_step)

    # ----- cache lifecycle (tidal/models/llama.py:616-656) -----------------------------------
    def tidal_init(self, page_size: int, max_seq_len: int, token_budget: Optional[int] = None,
                   page_order_seed=None, with_metadata: bool = False):
        """``with_metadata``: also keep the per-page key max / min pool that the Quest-style steps
        (``attn_type = "quest"``) estimate page scores from."""
        c = self.config
        self.iController = InferenceController(
            c.num_layers, c.num_heads, c.head_dim, page_size,
            c.top_k if token_budget is None else token_budget, max_seq_len, c.dtype, self.device,
            num_kv_heads=c.num_kv_heads, select_mode=c.select_mode, select_scope="all",
            page_order_seed=page_order_seed, with_metadata=with_metadata)

    def tidal_clear(self):
        self.iController.clean_states()

    # ----- pieces -------------------------------------------------------------------------------
    def _rms(self, x, weight):
        return tidal_utils.rms_norm_forward(x, weight, self.config.rms_norm_eps)

    def _mlp(self, layer, x):
        c = self.config
        gu = x @ layer["w_gate_up"].t()
        gate, up = gu[..., : c.intermediate_size], gu[..., c.intermediate_size:]
        return (torch.nn.functional.silu(gate) * up) @ layer["w_down"].t()

    def _qkv(self, layer, h):
        c = self.config
        qkv = h @ layer["wqkv"].t()
        n = qkv.shape[0]
        q_end = c.num_heads * c.head_dim
        k_end = q_end + c.num_kv_heads * c.head_dim
        q = qkv[:, :q_end].reshape(n, c.num_heads, c.head_dim).contiguous()
        k = qkv[:, q_end:k_end].reshape(n, c.num_kv_heads, c.head_dim).contiguous()
        v = qkv[:, k_end:].reshape(n, c.num_kv_heads, c.head_dim).contiguous()
        return q, k, v

    # ----- prefill ----------------------------------------------------------------------------
    @torch.no_grad()
    def prefill(self, input_ids: torch.Tensor) -> torch.Tensor:
        """Run the prompt [N] through all layers (full causal attention), fill the cache, return
        the logits of the last position."""
        c, ctrl = self.config, self.iController
        n = input_ids.numel()
        past = ctrl.kv_cache.seqlen
        t0 = time.perf_counter()
        ctrl.prepare_metadata(n)
        ctrl.begin_forward(n)
        x = self.embed[input_ids.to(self.device)]
        for idx, layer in enumerate(self.layers):
            h = self._rms(x, layer["ln1"])
            q, k, v = self._qkv(layer, h)
            tidal_utils.apply_rope_in_place(q, k, past, c.rope_scale, c.rope_theta)
            tidal_utils.append_kv(k, v, ctrl, idx)
            o = tidal_utils.prefill_forward(q, ctrl, idx)
            x = x + o.reshape(n, -1) @ layer["wo"].t()
            x = x + self._mlp(layer, self._rms(x, layer["ln2"]))
        ctrl.end_forward()
        logits = self._rms(x[-1:], self.norm) @ self.lm_head.t()
        torch.cuda.synchronize()
        ctrl.prefill_latency.append(time.perf_counter() - t0)
        return logits[0]

    @torch.no_grad()
    def synthetic_prefill(self, n: int):
        """Latency-only stand-in for a prompt of n tokens: the cache is filled with N(0,1) data
        (what the reference's harness gets from random input embeddings)."""
        ctrl = self.iController
        ctrl.kv_cache.pool.buf.normal_()
        if ctrl.metadata_cache is not None:
            ctrl.metadata_cache.pool.buf.normal_()
        ctrl.prepare_metadata(n)

    # ----- decode -----------------------------------------------------------------------------
    @torch.no_grad()
    def begin_decode_step(self):
        """Host bookkeeping of one decode step: reserve the slot of the new token and publish its
        position / physical slot to the device."""
        ctrl = self.iController
        ctrl.prepare_metadata(1)
        ctrl.begin_forward(1)
        pos = ctrl.kv_cache.seqlen - 1
        page = ctrl.kv_cache.indicies[pos // ctrl.page_size]
        self._positions.fill_(pos)
        self._dst_slot.fill_(page * ctrl.page_size + pos % ctrl.page_size)
        _kernels.rope_table(self._positions, self.config.head_dim, self.config.rope_scale,
                            self.config.rope_theta, self._cos, self._sin)
        self._quest = None
        if self.config.attn_type == "quest":
            if ctrl.metadata_cache is None:
                raise RuntimeError('attn_type "quest" needs tidal_init(..., with_metadata=True)')
            n_pages = len(ctrl.kv_cache.indicies)
            budget = max(1, min(int(ctrl._token_budget) // ctrl.page_size, n_pages - 1))
            self._quest = dict(
                pos=pos, budget=budget,
                page_ids=ctrl.kv_indices_without_last.expand(self.config.num_heads, -1).contiguous(),
                chosen=torch.zeros((self.config.num_heads, budget), dtype=torch.int32, device=self.device))

    def _attention_quest(self, idx, q, k, v):
        """One layer of a Quest-style step built from the library's pieces: RoPE and append as
        launches of their own (the append also updates the page's key bounds), then in layers 0 and 1
        full attention, later an upper bound of the logits per page (decode_estimate), the best
        pages (top-k over the bounds) and attention over those pages plus the page being filled.
        Query heads of a group choose their own pages (one list per query head)."""
        c, ctrl, qs = self.config, self.iController, self._quest
        tidal_utils.apply_rope_in_place(q, k, qs["pos"], c.rope_scale, c.rope_theta)
        tidal_utils.append_kv(k, v, ctrl, idx)
        kv = ctrl.kv_cache.buf_layer(idx)
        o = torch.empty_like(q)
        if idx < 2:
            ctrl._decode_handler.forward(q, o, kv, ctrl.kv_indices_without_last, None,
                                         ctrl.kv_cache.last_page_len, ctrl.kv_last_page_idx, None)
            return o
        est = tidal_utils.decode_estimate(q, ctrl, idx)
        _kernels.topk_filtering(est, qs["page_ids"], None, qs["chosen"], ctrl.topk_buf, qs["budget"])
        ctrl._decode_handler.forward(q, o, kv, qs["chosen"], None, ctrl.kv_cache.last_page_len,
                                     ctrl.kv_last_page_idx, None, index_kind="pages")
        return o

    def _attention_dev(self, idx, q, k, v):
        """_attention with every per-step quantity (list lengths, last page, slot and position of
        the new token) read from the device-resident step state instead of host integers."""
        c, ctrl, dev = self.config, self.iController, self._dev
        st = dev["state"]

        def word(i):
            return st[i: i + 1]

        fresh = None
        if self.fuse_decode_step and ctrl.fused_step_ok:
            fresh = (k, v, self._cos, self._sin, word(_lib.TD_STEP_DST_SLOT))
        else:
            _kernels.rope_append_decode(q, k, v, ctrl.kv_cache.buf_layer(idx),
                                        word(_lib.TD_STEP_POSITION), word(_lib.TD_STEP_DST_SLOT),
                                        ctrl.layout, c.rope_scale, c.rope_theta)
        kind = c.layer_kind(idx)
        o = torch.empty_like(q)
        buf = ctrl.kv_cache.buf_layer(idx)
        if kind == "sparse":
            ctrl._decode_handler.forward(q, o, buf, dev["lists"], dev["list_indptr"], 0, 0, None,
                                         index_kind="slots", n_list=dev["k"],
                                         counts=word(_lib.TD_STEP_N_SELECTED), fresh=fresh)
            return o
        select = kind == "select"
        ctrl._decode_handler.forward(q, o, buf, dev["table"].unsqueeze(0), dev["table_indptr"],
                                     word(_lib.TD_STEP_LAST_PAGE_LEN),
                                     word(_lib.TD_STEP_LAST_PAGE_IDX),
                                     ctrl.qk_product if select else None,
                                     lse=ctrl.lse if select else None,
                                     n_list=dev["table"].numel() - 1,
                                     counts=word(_lib.TD_STEP_PAGES_BEFORE_LAST), fresh=fresh)
        if select:
            scores, bound, n = ctrl.qk_product, ctrl.lse.view(-1), dev["final_len"]
            if ctrl.select_mode != "per_head":   # columns past the current length are never ranked
                _kernels.score_reduce(ctrl.qk_product, ctrl.lse.view(-1), ctrl.num_kv_heads, n,
                                      ctrl.select_mode, out=ctrl.score_sum)
                scores, bound = ctrl.score_sum, ctrl.score_bound
            _kernels.topk_filtering(scores[:, :n], None, None, dev["lists"], ctrl.topk_buf,
                                    dev["k"], page_table=dev["table"], page_size=ctrl.page_size,
                                    lengths=word(_lib.TD_STEP_SEQ_LEN), upper_bound=bound)
        return o

    def _attention(self, idx, q, k, v):
        """attention of one decode step for layer idx; q [1, H, D], k/v [1, H_kv, D] un-rotated"""
        if self._dev is not None:
            return self._attention_dev(idx, q, k, v)
        if self.config.attn_type == "quest":
            return self._attention_quest(idx, q, k, v)
        c, ctrl = self.config, self.iController
        fresh = None
        if self.fuse_decode_step and ctrl.fused_step_ok:
            fresh = (k, v, self._cos, self._sin, self._dst_slot)
        else:
            tidal_utils.rope_append_kv(q, k, v, ctrl, idx, self._positions, self._dst_slot,
                                       c.rope_scale, c.rope_theta)
        kind = c.layer_kind(idx)
        if kind == "sparse":
            return tidal_utils.decode_sparse_attn(q, ctrl, idx, ctrl.topk_dindices_buffer, False,
                                                  fresh=fresh)
        o = tidal_utils.decode_sparse_attn(q, ctrl, idx, ctrl.kv_indices_without_last,
                                           kind == "select", fresh=fresh)
        if kind == "select":
            tidal_utils.decode_topk(ctrl)
        return o

    @torch.no_grad()
    def decode_layers(self, x: torch.Tensor) -> torch.Tensor:
        """The layer loop of one decode step on hidden state x [1, hidden]; device work only (safe
        to capture in a hipGraph once begin_decode_step has run)."""
        c = self.config
        if self.use_gemv:
            eps = c.rms_norm_eps
            q_end = c.num_heads * c.head_dim
            k_end = q_end + c.num_kv_heads * c.head_dim
            h = x.reshape(-1).clone()  # residual stream, updated in place by the projections
            for idx, layer in enumerate(self.layers):
                qkv = _kernels.gemv(layer["wqkv"], h, norm_weight=layer["ln1"], eps=eps)
                q = qkv[:q_end].view(1, c.num_heads, c.head_dim)
                k = qkv[q_end:k_end].view(1, c.num_kv_heads, c.head_dim)
                v = qkv[k_end:].view(1, c.num_kv_heads, c.head_dim)
                o = self._attention(idx, q, k, v)
                _kernels.gemv(layer["wo"], o.view(-1), residual=h, out=h)
                act = _kernels.gemv(layer["w_gate_up"], h, norm_weight=layer["ln2"], eps=eps,
                                    pair_gated=True)
                _kernels.gemv(layer["w_down"], act, residual=h, out=h)
            return _kernels.gemv(self.lm_head, h, norm_weight=self.norm, eps=eps).view(1, -1)
        for idx, layer in enumerate(self.layers):
            hn = self._rms(x, layer["ln1"])
            q, k, v = self._qkv(layer, hn)
            o = self._attention(idx, q, k, v)
            x = x + o.reshape(1, -1) @ layer["wo"].t()
            x = x + self._mlp(layer, self._rms(x, layer["ln2"]))
        return self._rms(x, self.norm) @ self.lm_head.t()

    @torch.no_grad()
    def decode_step(self, token: torch.Tensor) -> torch.Tensor:
        """One eager decode step for token id(s) [1]; returns logits [vocab]."""
        ctrl = self.iController
        t0 = time.perf_counter()
        self.begin_decode_step()
        logits = self.decode_layers(self.embed[token.to(self.device).view(1)])
        ctrl.end_forward()
        torch.cuda.synchronize()
        ctrl.decode_latency.append(time.perf_counter() - t0)
        return logits[0]

    @torch.no_grad()
    def generate(self, input_ids: torch.Tensor, max_new_tokens: int) -> torch.Tensor:
        """Greedy decoding (prefill + max_new_tokens steps)."""
        logits = self.prefill(input_ids)
        out = []
        for _ in range(max_new_tokens):
            tok = logits.argmax().view(1)
            out.append(tok)
            logits = self.decode_step(tok)
        return torch.cat(out)

    @torch.no_grad()
    def generate_graph(self, input_ids: torch.Tensor, max_new_tokens: int,
                       keep_logits: bool = False, use_graph: bool = True, between_steps=None):
        """Greedy decoding in which ONE captured decode step is replayed for every token: the
        sequence's step state (length, last page, slot and position of the new token, list
        length) lives on the device and is advanced by a one-thread launch inside the step, the
        next token id never leaves the device, and pages for all tokens to come are reserved up
        front.  No host work, copy or synchronisation between tokens.  Returns the token ids
        (and, with ``keep_logits``, the logits that chose them: row i chose token i + 1).
        ``between_steps`` (a callable, for tests) runs on the host after every step."""
        c = self.config
        logits = self.prefill(input_ids)
        ctrl = self.iController
        prompt_len = ctrl.kv_cache.seqlen
        ctrl.prepare_metadata(max_new_tokens)   # pages for every token to come
        ctrl.begin_forward(1)
        final_len = ctrl.kv_cache.seqlen
        table = ctrl.kv_cache.indices_device      # covers all of them already
        k = min(int(ctrl._token_budget), final_len, ctrl.topk_dindices_buffer_full.size(1))
        i32 = dict(dtype=torch.int32, device=self.device)
        state = torch.zeros(_lib.TD_STEP_WORDS, **i32)
        state[_lib.TD_STEP_SEQ_LEN] = prompt_len
        self._dev = dict(state=state, table=table, final_len=final_len, k=k,
                         lists=ctrl.topk_dindices_buffer_full[:, :k],
                         list_indptr=torch.tensor([0, k], **i32),
                         table_indptr=torch.tensor([0, table.numel()], **i32))
        token = logits.argmax().view(1)
        tokens = torch.zeros(max_new_tokens, dtype=torch.int64, device=self.device)
        kept = torch.zeros((max_new_tokens, c.vocab_size), dtype=torch.float32,
                           device=self.device) if keep_logits else None

        def step():
            _kernels.step_advance(state, table, ctrl.page_size, k, token, tokens)
            _kernels.rope_table(state[_lib.TD_STEP_POSITION: _lib.TD_STEP_POSITION + 1], c.head_dim,
                                c.rope_scale, c.rope_theta, self._cos, self._sin)
            out = self.decode_layers(self.embed.index_select(0, token)).view(-1)
            if kept is not None:
                row = (state[_lib.TD_STEP_COUNT: _lib.TD_STEP_COUNT + 1] - 1).long()
                kept.index_copy_(0, row, out.float().view(1, -1))
            _kernels.argmax(out, token)

        try:
            run = step
            if use_graph:
                # warm-up on a side stream (plans, scratch), then undo its one step on the device
                s = torch.cuda.Stream()
                s.wait_stream(torch.cuda.current_stream())
                saved = (state.clone(), token.clone())
                with torch.cuda.stream(s):
                    step()
                torch.cuda.current_stream().wait_stream(s)
                torch.cuda.synchronize()
                state.copy_(saved[0])
                token.copy_(saved[1])
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    step()
                run = g.replay
            t0 = time.perf_counter()
            for _ in range(max_new_tokens):
                run()
                if between_steps is not None:
                    between_steps()
            torch.cuda.synchronize()
            ctrl.decode_latency.append((time.perf_counter() - t0) / max(1, max_new_tokens))
        finally:
            self._dev = None
            ctrl.end_forward()
        return (tokens, kept) if keep_logits else tokens

    @torch.no_grad()
    def timed_decode(self, steps: int, warmup: int = 3, use_graph: bool = True) -> Tuple[float, str]:
        """Steady-state latency of a decode step at the current context length: the step that
        appends token number seqlen is captured once (hipGraph) and replayed; returns
        (seconds per step, "hipGraph" | "eager")."""
        ctrl = self.iController
        self.begin_decode_step()
        x = self.embed[:1].clone()
        run, how = (lambda: self.decode_layers(x)), "eager"
        if use_graph:
            try:
                s = torch.cuda.Stream()
                s.wait_stream(torch.cuda.current_stream())
                with torch.cuda.stream(s):
                    self.decode_layers(x)
                torch.cuda.current_stream().wait_stream(s)
                torch.cuda.synchronize()
                g = torch.cuda.CUDAGraph()
                with torch.cuda.graph(g):
                    self.decode_layers(x)
                run, how = g.replay, "hipGraph"
            except Exception as e:  # pragma: no cover - runtime dependent
                print(f"[tidal] graph capture failed ({e}); timing eager launches")
                torch.cuda.synchronize()
        for _ in range(warmup):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            run()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / steps
        ctrl.end_forward()
        ctrl.decode_latency.append(dt)
        return dt, how

"""Operator surface of the decode path (counterpart of tidal/utils/__init__.py:26-287).

The seven functions keep the reference's names and arguments.  ``decode_sparse_attn`` serves both
uses the reference makes of it: with ``iController.kv_indices_without_last`` it is the full
attention of a Full / Search layer (optionally writing logits for the selection that follows),
with ``iController.topk_dindices_buffer`` it is the sparse attention over the persisted tokens.
"""
from typing import Optional

import torch

from .. import _kernels
from .batch_controller import BatchInferenceController
from .controller import InferenceController
from .paged import BatchDecodeWithPagedKVCacheWrapper, KvCache, KvPool, TensorLayout

__all__ = [
    "TensorLayout",
    "KvCache",
    "KvPool",
    "InferenceController",
    "BatchInferenceController",
    "BatchDecodeWithPagedKVCacheWrapper",
    "append_kv",
    "prefill_forward",
    "decode_estimate",
    "decode_topk",
    "decode_sparse_attn",
    "rms_norm_forward",
    "apply_rope_in_place",
    "rope_append_kv",
]


def apply_rope_in_place(q: torch.Tensor, k: torch.Tensor, past_kv_len: int,
                        rope_scale: Optional[float] = None, rope_theta: Optional[float] = None):
    """Rotate q ``[N, H, D]`` and k ``[N, H_kv, D]`` in place; token i is at ``past_kv_len + i``."""
    if rope_scale is None:
        rope_scale = 1.0
    if rope_theta is None:
        rope_theta = 1e4
    _kernels.apply_rope_in_place(q, k, past_kv_len, rope_scale, rope_theta)


def rms_norm_forward(input: torch.Tensor, weight: torch.Tensor, epsilon: float) -> torch.Tensor:
    o = torch.empty_like(input)
    _kernels.rms_norm_forward(input, weight, o, epsilon)
    return o


def _meta_args(iController: InferenceController, layer_idx: int):
    if iController.metadata_cache is None:
        return (None, None, None, 0, 0)
    return (iController.metadata_cache.buf_layer(layer_idx), iController.metadata_indices,
            iController.metadata_indptr_for_append, iController.metadata_cache.last_page_len,
            iController.metadata_last_page_idx)


def append_kv(k: torch.Tensor, v: torch.Tensor, iController: InferenceController, layer_idx: int):
    """Append the new k/v ``[N, H_kv, D]`` to the paged cache of a layer (prefill for N > 1,
    decode for N == 1)."""
    fn = _kernels.append_kv_cache_prefill if k.size(0) > 1 else _kernels.append_kv_cache_decode
    fn(k, v, iController.kv_cache.buf_layer(layer_idx), iController.kv_indices_with_last,
       iController.kv_indptr_for_append, iController.kv_cache.last_page_len,
       iController.kv_last_page_idx, *_meta_args(iController, layer_idx), iController.layout)


def rope_append_kv(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                   iController: InferenceController, layer_idx: int, positions: torch.Tensor,
                   dst_slot: torch.Tensor, rope_scale: Optional[float] = None,
                   rope_theta: Optional[float] = None):
    """Decode-step fusion of ``apply_rope_in_place`` and ``append_kv`` (one launch)."""
    _kernels.rope_append_decode(q, k, v, iController.kv_cache.buf_layer(layer_idx), positions,
                                dst_slot, iController.layout,
                                1.0 if rope_scale is None else rope_scale,
                                1e4 if rope_theta is None else rope_theta)


def prefill_forward(q: torch.Tensor, iController: InferenceController, layer_idx: int,
                    rope_scale: Optional[float] = None, rope_theta: Optional[float] = None
                    ) -> torch.Tensor:
    """Causal attention of the new tokens over the cache (K/V already appended)."""
    return _kernels.prefill_with_paged_kv_cache(
        q, iController.kv_cache.buf_layer(layer_idx), iController.kv_indices_with_last,
        iController.kv_cache.last_page_len, True, iController.layout, False,
        1.0 if rope_scale is None else rope_scale, 1e4 if rope_theta is None else rope_theta)


def decode_estimate(q: torch.Tensor, iController: InferenceController, layer_idx: int
                    ) -> torch.Tensor:
    """Page-score estimator of the reference's ancestor (tidal/utils/__init__.py:176-214): upper
    bound of the logits per KV page from the page metadata, ``[H, pages - 1]`` (the page being
    filled is left out).  Needs a controller built ``with_metadata=True``; TidalDecode's own
    layers never call it."""
    c = iController
    if c.metadata_cache is None:
        raise RuntimeError("decode_estimate needs InferenceController(..., with_metadata=True)")
    o = torch.empty((q.size(1), c.metadata_cache.seqlen - 1), dtype=q.dtype, device=q.device)
    _kernels.estimate_attn_score(q, o, c.metadata_cache.buf_layer(layer_idx), c.metadata_indices,
                                 c.metadata_indptr_for_append, c.metadata_cache.last_page_len,
                                 c.metadata_last_page_idx, c.layout)
    return o


def decode_topk(iController: InferenceController):
    """Select the token budget from the logits the last selection layer wrote into
    ``iController.qk_product``; result: physical token slots in
    ``iController.topk_dindices_buffer`` (one row per query head, per KV head, or shared)."""
    c = iController
    k, n = c.num_selected, c.num_candidates
    if k == 0:
        return
    # no logit exceeds its head's log-sum-exp, no summed probability the head count
    scores, bound = c.qk_product, c.lse.view(-1)
    if c.select_mode != "per_head":
        _kernels.score_reduce(c.qk_product, c.lse.view(-1), c.num_kv_heads, n, c.select_mode,
                              out=c.score_sum)
        scores, bound = c.score_sum, c.score_bound
    _kernels.topk_filtering(scores[:, :n], None, None, c.topk_dindices_buffer, c.topk_buf, k,
                            page_table=c.kv_indices_with_last, page_size=c.page_size,
                            upper_bound=bound)


def decode_sparse_attn(q: torch.Tensor, iController: InferenceController, layer_idx: int,
                       topk_indices: torch.Tensor, output_qk_product: bool,
                       rope_scale: Optional[float] = None, rope_theta: Optional[float] = None,
                       fresh=None) -> torch.Tensor:
    """Attention of the new token ``q [1, H, D]`` over the listed part of the cache.

    ``topk_indices is iController.kv_indices_without_last``: every page in order plus the last
    page, i.e. full attention; with ``output_qk_product`` the logits (and log-sum-exp) are kept
    for ``decode_topk``.  Otherwise ``topk_indices`` holds token slots chosen by ``decode_topk``.

    ``fresh=(k, v, cos, sin, dst_slot)`` (extension) folds ``apply_rope_in_place`` and
    ``append_kv`` of the new token into this launch: q and k are then un-rotated.
    """
    c = iController
    o = torch.empty_like(q)
    full = topk_indices is c.kv_indices_without_last
    if full:
        c._decode_handler.forward(q, o, c.kv_cache.buf_layer(layer_idx), topk_indices, None,
                                  c.kv_cache.last_page_len, c.kv_last_page_idx,
                                  c.qk_product if output_qk_product else None, rope_scale,
                                  rope_theta, lse=c.lse if output_qk_product else None,
                                  fresh=fresh)
    else:
        forced = c.select_scope == "exclude_last_page"
        c._decode_handler.forward(q, o, c.kv_cache.buf_layer(layer_idx), topk_indices, None,
                                  c.kv_cache.last_page_len if forced else 0,
                                  c.kv_last_page_idx if forced else 0,
                                  c.qk_product if output_qk_product else None, rope_scale,
                                  rope_theta, index_kind="slots",
                                  lse=c.lse if output_qk_product else None, fresh=fresh)
    return o

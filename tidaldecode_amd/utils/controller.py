"""Host-side bookkeeping of one sequence during inference (counterpart of
tidal/utils/controller.py:8-193 of the reference).

Same attribute and method names as the reference so that model code written against it keeps
working; what differs is what the reference gets wrong or does slowly:

* index tensors live on the device and grow in place; nothing is rebuilt or re-uploaded per
  decode step (the reference re-creates ``[H, n_pages]`` tensors every step, controller.py:120-137);
* score / top-k buffers are allocated once, not in every ``begin_forward`` (controller.py:149-168),
  so the indices a selection layer wrote survive the budget switch that follows it;
* any ``page_size`` (the reference asserts 1, controller.py:20) with token-granular selection;
* grouped-query attention (``num_kv_heads``), bf16, and three selection modes:
  ``per_head`` (one list per query head: the reference's behaviour), ``group_sum`` (one list per
  KV head from summed softmax probabilities) and ``head_sum`` (one shared list);
* ``select_scope="all"`` selects among every cached token including the newest one
  (src/tidal_build/modify_llama.py:112-120); ``"exclude_last_page"`` reproduces the kernel
  path of the reference, which always attends to the newest page and selects among the rest
  (kernels/include/decode/decode_page.cuh:326-329).
"""
from typing import Optional

import torch

from .paged import BatchDecodeWithPagedKVCacheWrapper, KvCache, TensorLayout

_SELECT_MODES = ("per_head", "group_sum", "head_sum")
_SELECT_SCOPES = ("all", "exclude_last_page")


def _logits_dtype(logits_dtype, kv_dtype, select_mode):
    """The type of the logits buffer that a selection layer fills: float32 (default), or the KV
    dtype, which is what the reference allocates (tidal/utils/controller.py:149-151: the logits
    are then rounded to 16 bits before the top-k sees them).  The summed selection modes read
    float32 logits only."""
    if logits_dtype is None:
        return torch.float32
    if logits_dtype not in (torch.float32, kv_dtype):
        raise ValueError(f"logits_dtype must be torch.float32 or the KV dtype {kv_dtype}, not {logits_dtype}")
    if logits_dtype != torch.float32 and select_mode != "per_head":
        raise ValueError(f"select_mode {select_mode} sums probabilities from float32 logits")
    return logits_dtype


class InferenceController:
    def __init__(self, num_layers, num_heads, head_dim, page_size, token_budget, max_seq_len,
                 dtype, device, *, num_kv_heads: Optional[int] = None,
                 select_mode: str = "per_head", select_scope: str = "all",
                 kv_layout: str = "NHD", with_metadata: bool = False, page_order_seed=None,
                 logits_dtype: Optional[torch.dtype] = None):
        if select_mode not in _SELECT_MODES:
            raise KeyError(f"Invalid select_mode {select_mode}")
        logits_dtype = _logits_dtype(logits_dtype, dtype, select_mode)
        if select_scope not in _SELECT_SCOPES:
            raise KeyError(f"Invalid select_scope {select_scope}")
        num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        if num_heads % num_kv_heads != 0:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        self.layout = TensorLayout.parse(kv_layout)
        self.kv_cache = KvCache(num_layers=num_layers, num_heads=num_kv_heads, head_dim=head_dim,
                                max_seq_len=max_seq_len, page_size=page_size, dtype=dtype,
                                device=device, layout=self.layout,
                                page_order_seed=page_order_seed)
        max_kv_pages_num = (max_seq_len + page_size - 1) // page_size
        # per-page key max/min pool of the reference's page estimator; unused by TidalDecode
        self.metadata_cache = None
        if with_metadata:
            self.metadata_cache = KvCache(num_layers=num_layers, num_heads=num_kv_heads,
                                          head_dim=head_dim, max_seq_len=max_kv_pages_num,
                                          page_size=page_size, dtype=dtype, device=device,
                                          layout=self.layout)
        self.device = device
        self.dtype = dtype
        self.num_heads = num_heads
        self.num_kv_heads = num_kv_heads
        self.head_dim = head_dim
        self.page_size = page_size
        self.max_seq_len = max_seq_len
        self.select_mode = select_mode
        self.select_scope = select_scope

        self._token_budget = token_budget
        self._decode_handler = BatchDecodeWithPagedKVCacheWrapper(kv_layout=kv_layout)

        self.kv_indices_with_last = None
        self.kv_indices_with_last_decode = None
        self.kv_indices_without_last = None
        self.metadata_indices = None
        self.kv_last_page_idx = None
        self.metadata_last_page_idx = None
        self.kv_indptr_for_append = None
        self.metadata_indptr_for_append = None
        self.kv_indptr_for_approx_decode = None
        self.inference_token_budget = None

        # selection state, allocated once
        self.index_rows = {"per_head": num_heads, "group_sum": num_kv_heads, "head_sum": 1}[select_mode]
        score_cols = max_kv_pages_num * page_size
        self.qk_product = torch.zeros((num_heads, score_cols), dtype=logits_dtype, device=device)
        self.lse = torch.zeros((1, num_heads), dtype=torch.float32, device=device)
        self.score_sum = None
        if select_mode != "per_head":
            self.score_sum = torch.zeros((self.index_rows, score_cols), dtype=torch.float32,
                                         device=device)
            # a probability is at most 1: the head count bounds every summed score
            self.score_bound = torch.full((self.index_rows,), num_heads // self.index_rows + 1.0,
                                          dtype=torch.float32, device=device)
        self._index_capacity = min(int(token_budget), score_cols)
        self.topk_dindices_buffer_full = torch.zeros((self.index_rows, self._index_capacity),
                                                     dtype=torch.int32, device=device)
        self.topk_dindices_buffer = self.topk_dindices_buffer_full
        self.topk_dout_buffer = None  # selected values are not needed downstream
        # scratch of the top-k kernels (the reference's RAFT buffer): zeroed once, kept zeroed
        from .. import _kernels
        self.topk_buf = torch.zeros(_kernels.topk_workspace_bytes(self.index_rows),
                                    dtype=torch.uint8, device=device) \
            if torch.device(device).type == "cuda" else None
        self.num_candidates = 0
        self.num_selected = 0
        self._indptr2 = torch.zeros(2, dtype=torch.int32, device=device)
        self._meta_indptr2 = torch.zeros(2, dtype=torch.int32, device=device)

        self.prefill_latency = []
        self.decode_latency = []
        # the fused decode step (RoPE + append inside the attention launch) exists for
        # power-of-two pages and per-layer pools below 4 GiB
        layer_bytes = self.kv_cache.pool.buf[0].numel() * self.kv_cache.pool.buf.element_size()
        self.fused_step_ok = (page_size & (page_size - 1)) == 0 and layer_bytes < (1 << 32)

    # Used for controlling the number of pages (the reference skips its first layers with it)
    def set_token_budget(self, token_budget: int):
        self._token_budget = token_budget

    # Called once per forward: reserve room for the new tokens
    def prepare_metadata(self, seq_len: int):
        appended_new_pages = self.kv_cache.append_seq(seq_len)
        if self.metadata_cache is not None:
            self.metadata_cache.append_seq(appended_new_pages)

    # Called once per forward (and again after a budget switch, as the reference's model loop does)
    def begin_forward(self, seq_len: int, updateTensor: bool = True):
        cache = self.kv_cache
        n_pages = len(cache.indicies)
        if updateTensor:
            self._indptr2[1] = n_pages
            self.kv_indptr_for_append = self._indptr2
            self.kv_last_page_idx = cache.indicies[-1]
            self.kv_indices_with_last = cache.indices_device
            if self.metadata_cache is not None:
                self._meta_indptr2[1] = len(self.metadata_cache.indicies)
                self.metadata_indptr_for_append = self._meta_indptr2
                self.metadata_last_page_idx = self.metadata_cache.indicies[-1]
                self.metadata_indices = self.metadata_cache.indices_device
        if seq_len > 1:
            return
        # decode
        if updateTensor:
            # one shared row; every head walks the same page list
            self.kv_indices_with_last_decode = cache.indices_device.unsqueeze(0)
            self.kv_indices_without_last = cache.indices_device[: n_pages - 1].unsqueeze(0)
        if self.select_scope == "all":
            self.num_candidates = cache.seqlen
            self.num_selected = min(int(self._token_budget), self.num_candidates,
                                    self._index_capacity)
        else:
            self.num_candidates = (n_pages - 1) * self.page_size
            want = min(int(self._token_budget), cache.seqlen) - cache.last_page_len
            self.num_selected = max(0, min(want, self.num_candidates, self._index_capacity))
        self.inference_token_budget = self.num_selected
        self.topk_dindices_buffer = self.topk_dindices_buffer_full[:, : self.num_selected]
        self._decode_handler.begin_forward(None, self.num_heads, self.num_kv_heads, self.head_dim,
                                           self.page_size, self.dtype)

    def end_forward(self):
        self._decode_handler.end_forward()

    def need_estimate(self) -> bool:
        if self.inference_token_budget is None:
            return False
        return self.kv_cache.seqlen > self.inference_token_budget

    def clean_states(self):
        self.kv_cache.release()
        if self.metadata_cache is not None:
            self.metadata_cache.release()

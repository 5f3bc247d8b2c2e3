"""Bookkeeping of several sequences that decode in lock step over one shared page pool.

The reference's controller serves one sequence (tidal/utils/controller.py:8-193, its kv cache
asserts a single page table, tidal/utils/kv_cache.py:70-137); its kernels already take a batch
(``indptr``, kernels/include/decode/decode_attn.cuh:432-470).  This class is the batched
counterpart of ``InferenceController`` for that kernel surface:

* one pool per layer shared by all sequences, one fixed-width page-table segment per sequence in a
  device tensor ``[max_batch, pages_per_seq]`` that grows in place;
* the per-sequence metadata of a decode step (pages before the last one, fill of the last page,
  its id, the slot and the position of the new token, the number of selected tokens, the length) is one
  ``[8, max_batch]`` int32 device tensor (the words of ``td_step_advance``), refreshed by a single
  small copy per step (``begin_step``) or, with pages reserved ahead (``reserve_ahead``), advanced
  on the device by a one-launch ``begin_step_on_device`` — never the page tables themselves;
* selection state for the whole batch: logits ``[B * H_q, max tokens]`` (``-inf`` where a sequence
  has no token, so that one top-k call serves ragged lengths), the log-sum-exp per head and the
  persisted token lists ``[rows, B * budget]`` with one fixed-width segment per sequence.

Every attention call is ONE launch for the whole batch.  After ``reserve_ahead`` every host-side
argument of a step's calls is an upper bound that holds for the reserved tokens and everything
else is read on the device, so ``begin_step_on_device`` + the attention calls can be captured in a
graph and replayed per token.  Token lists are valid for the decode step they were selected in.
"""
from typing import List, Optional, Sequence

import torch

from .. import _kernels, _lib
from .controller import _logits_dtype
from .paged import BatchDecodeWithPagedKVCacheWrapper, KvPool, TensorLayout

_SELECT_MODES = ("per_head", "group_sum", "head_sum")
# rows of the per-step metadata tensor: the words of the device-resident step state
_SEQ_LEN, _PAGES_BEFORE_LAST, _LAST_LEN = (_lib.TD_STEP_SEQ_LEN, _lib.TD_STEP_PAGES_BEFORE_LAST,
                                           _lib.TD_STEP_LAST_PAGE_LEN)
_LAST_IDX, _DST_SLOT, _POSITION = (_lib.TD_STEP_LAST_PAGE_IDX, _lib.TD_STEP_DST_SLOT,
                                   _lib.TD_STEP_POSITION)
_SELECTED, _STEPS, _META_ROWS = _lib.TD_STEP_N_SELECTED, _lib.TD_STEP_COUNT, _lib.TD_STEP_WORDS


class BatchInferenceController:
    def __init__(self, num_layers: int, num_heads: int, head_dim: int, page_size: int,
                 token_budget: int, max_seq_len: int, max_batch: int, dtype, device, *,
                 num_kv_heads: Optional[int] = None, select_mode: str = "per_head",
                 kv_layout: str = "NHD", page_order_seed=None,
                 logits_dtype: Optional[torch.dtype] = None):
        if select_mode not in _SELECT_MODES:
            raise KeyError(f"Invalid select_mode {select_mode}")
        num_kv_heads = num_heads if num_kv_heads is None else num_kv_heads
        if num_heads % num_kv_heads != 0:
            raise ValueError("num_heads must be a multiple of num_kv_heads")
        if max_batch < 1 or max_seq_len < 1:
            raise ValueError("max_batch and max_seq_len must be positive")
        self.layout = TensorLayout.parse(kv_layout)
        self.device, self.dtype = device, dtype
        self.num_heads, self.num_kv_heads, self.head_dim = num_heads, num_kv_heads, head_dim
        self.page_size, self.max_seq_len, self.max_batch = page_size, max_seq_len, max_batch
        self.select_mode = select_mode
        self.pages_per_seq = -(-max_seq_len // page_size)
        self.pool = KvPool(num_layers, num_kv_heads, head_dim, max_batch * self.pages_per_seq,
                           page_size, dtype, device, self.layout, page_order_seed)

        i32 = dict(dtype=torch.int32, device=device)
        self.page_table = torch.zeros((max_batch, self.pages_per_seq), **i32)
        self._pages: List[List[int]] = []
        self.seq_lens: List[int] = []
        self._cap: List[int] = []   # tokens each sequence has pages for (>= its length)
        self._meta = torch.zeros((_META_ROWS, max_batch), **i32)
        # staging for the per-step copy: a small ring of pinned rows, so that the copy is
        # asynchronous and a buffer is only rewritten after its copy has completed
        self._on_gpu = torch.device(device).type == "cuda"
        self._stage = [torch.zeros((_META_ROWS, max_batch), dtype=torch.int32, pin_memory=self._on_gpu)
                       for _ in range(4)]
        self._stage_done = [None] * len(self._stage)
        self._stage_next = 0
        self._steps = 0
        self._table_starts = torch.arange(max_batch + 1, **i32) * self.pages_per_seq

        self.score_cols = self.pages_per_seq * page_size
        self.budget = min(int(token_budget), self.score_cols)
        self.index_rows = {"per_head": num_heads, "group_sum": num_kv_heads, "head_sum": 1}[select_mode]
        # float32, or the KV dtype as in the reference (see controller._logits_dtype)
        self.qk_product = torch.full((max_batch * num_heads, self.score_cols), float("-inf"),
                                     dtype=_logits_dtype(logits_dtype, dtype, select_mode),
                                     device=device)
        self.lse = torch.zeros((max_batch, num_heads), dtype=torch.float32, device=device)
        self.score_sum = None
        if select_mode != "per_head":
            self.score_sum = torch.zeros((max_batch * self.index_rows, self.score_cols),
                                         dtype=torch.float32, device=device)
            # a probability is at most 1: the head count bounds every summed score
            self.score_bound = torch.full((max_batch * self.index_rows,),
                                          num_heads // self.index_rows + 1.0,
                                          dtype=torch.float32, device=device)
        # lists: row r of sequence b lives in columns [b * budget, b * budget + selected[b])
        self.topk_dindices_buffer = torch.zeros((self.index_rows, max_batch * self.budget), **i32)
        self._slots = torch.zeros((max_batch * self.index_rows, self.budget), **i32)
        self._list_starts = torch.arange(max_batch + 1, **i32) * self.budget
        self.topk_buf = torch.zeros(_kernels.topk_workspace_bytes(max_batch * self.index_rows),
                                    dtype=torch.uint8, device=device)
        self._handle = BatchDecodeWithPagedKVCacheWrapper(kv_layout=kv_layout)
        self._handle.begin_forward(None, num_heads, num_kv_heads, head_dim, page_size, dtype)
        layer_bytes = self.pool.buf[0].numel() * self.pool.buf.element_size()
        self.fused_step_ok = (page_size & (page_size - 1)) == 0 and layer_bytes < (1 << 32)

    # ---- sequences ----------------------------------------------------------------------------
    @property
    def batch(self) -> int:
        return len(self.seq_lens)

    def buf_layer(self, layer_idx: int) -> torch.Tensor:
        return self.pool.buf[layer_idx % self.pool.num_layers]

    def _ensure_pages(self, b: int, total: int) -> None:
        """pages for `total` tokens of sequence b"""
        if total > self.max_seq_len:
            raise RuntimeError(f"sequence {b} would hold {total} tokens, max_seq_len is {self.max_seq_len}")
        have = len(self._pages[b])
        grow = -(-total // self.page_size) - have
        if grow > 0:
            fresh = self.pool.take(grow)
            self.page_table[b, have: have + grow] = torch.tensor(fresh, dtype=torch.int32)
            self._pages[b] += fresh
        self._cap[b] = max(self._cap[b], total)

    def _reserve(self, b: int, n_tokens: int) -> None:
        self._ensure_pages(b, self.seq_lens[b] + n_tokens)
        self.seq_lens[b] += n_tokens

    def reserve_ahead(self, n_tokens: int) -> None:
        """Pages for the next ``n_tokens`` decode steps of every sequence, so that those steps
        need nothing from the host (``begin_step_on_device``)."""
        over = [b for b, n in enumerate(self.seq_lens) if n + int(n_tokens) > self.max_seq_len]
        if over:
            raise RuntimeError(f"sequences {over} would exceed max_seq_len = {self.max_seq_len}")
        for b in range(self.batch):
            self._ensure_pages(b, self.seq_lens[b] + int(n_tokens))

    def add_sequences(self, lengths: Sequence[int]) -> None:
        """Open one sequence per entry with room for that many prompt tokens."""
        if self.batch + len(lengths) > self.max_batch:
            raise RuntimeError(f"{self.batch + len(lengths)} sequences, max_batch is {self.max_batch}")
        if any(n < 1 for n in lengths):
            raise ValueError("a sequence starts with at least one token")
        opened = self.batch
        try:
            for n in lengths:
                self._pages.append([])
                self.seq_lens.append(0)
                self._cap.append(0)
                self._reserve(self.batch - 1, int(n))
        except Exception:
            for pages in self._pages[opened:]:   # leave the controller as it was
                self.pool.give_back(pages)
            del self._pages[opened:], self.seq_lens[opened:], self._cap[opened:]
            raise
        self._refresh()

    def release_sequences(self, which: Sequence[int]) -> dict:
        """Close the listed sequences between two decode steps and return their pages; the others
        go on decoding.  The batch stays dense: the last sequences move into the freed places (their
        page-table rows, persisted lists and host mirrors move with them), every other sequence
        keeps its index.  Returns ``{old index: new index}`` of the sequences that moved.  New
        sequences can join at any step boundary with ``add_sequences`` + ``append_prompt``; they
        get their token lists in the first selection layer of their first step.  A captured step
        has the batch size baked into its launches: capture it again after the batch changed."""
        which = sorted(set(int(b) for b in which))
        if any(b < 0 or b >= self.batch for b in which):
            raise IndexError(f"no such sequence among {self.batch}: {which}")
        moved = {}
        H, rows, k = self.num_heads, self.index_rows, self.budget
        lists = self.topk_dindices_buffer.view(rows, self.max_batch, k)
        for b in reversed(which):
            last = self.batch - 1
            self.pool.give_back(self._pages[b])
            if b != last:
                self.page_table[b].copy_(self.page_table[last])
                lists[:, b].copy_(lists[:, last])
                self._pages[b], self.seq_lens[b], self._cap[b] = (self._pages[last], self.seq_lens[last],
                                                                  self._cap[last])
                origin = next((o for o, n in moved.items() if n == last), last)
                moved.pop(origin, None)
                moved[origin] = b
            # logits of a closed place are stale: nothing of them may be ranked for its next owner
            self.qk_product[b * H: (b + 1) * H].fill_(float("-inf"))
            self.qk_product[last * H: (last + 1) * H].fill_(float("-inf"))
            self._pages.pop(), self.seq_lens.pop(), self._cap.pop()
        if self.batch:
            self._refresh()
        return moved

    def release(self) -> None:
        """Close every sequence and return its pages."""
        for pages in self._pages:
            self.pool.give_back(pages)
        self._pages, self.seq_lens, self._cap = [], [], []
        self.qk_product.fill_(float("-inf"))

    def _refresh(self) -> None:
        """Per-sequence metadata of the current lengths: one host row set, one copy."""
        P = self.page_size
        cols = []
        for b, n in enumerate(self.seq_lens):
            before, entry = divmod(n - 1, P)
            page = self._pages[b][before]   # pages may be reserved beyond the one being filled
            row = [0] * _META_ROWS
            row[_SEQ_LEN], row[_PAGES_BEFORE_LAST], row[_LAST_LEN] = n, before, entry + 1
            row[_LAST_IDX], row[_DST_SLOT], row[_POSITION] = page, page * P + entry, n - 1
            row[_SELECTED], row[_STEPS] = min(self.budget, n), self._steps
            cols.append(tuple(row))
        cols += [(0,) * _META_ROWS] * (self.max_batch - len(cols))
        i = self._stage_next
        self._stage_next = (i + 1) % len(self._stage)
        if self._stage_done[i] is not None:
            self._stage_done[i].synchronize()
        m = self._stage[i]
        m.copy_(torch.tensor(cols, dtype=torch.int32).t())
        self._meta.copy_(m, non_blocking=True)
        if self._on_gpu:
            self._stage_done[i] = torch.cuda.Event()
            self._stage_done[i].record()

    def begin_step(self) -> None:
        """Make room for one new token in every sequence (call once per decode step)."""
        full = [b for b, n in enumerate(self.seq_lens) if n + 1 > self.max_seq_len]
        if full:
            raise RuntimeError(f"sequences {full} already hold max_seq_len = {self.max_seq_len} tokens")
        for b in range(self.batch):
            self._reserve(b, 1)
        self._steps += 1
        self._refresh()

    def advance_on_device(self) -> None:
        """The device half of ``begin_step_on_device``: one launch recomputes every sequence's
        metadata for one more token from the page tables.  This is the call to capture."""
        _kernels.step_advance_batch(self._meta, self.batch, self.page_table, self.page_size,
                                    self.budget)

    def note_step(self) -> None:
        """The host half: the mirrors of the lengths move on by one token (call it before every
        replay of a captured step).  The pages must have been reserved (``reserve_ahead``)."""
        short = [b for b, n in enumerate(self.seq_lens) if n + 1 > self._cap[b]]
        if short:
            raise RuntimeError(f"sequences {short} have no page reserved for another token; call "
                               "reserve_ahead first")
        for b in range(self.batch):
            self.seq_lens[b] += 1
        self._steps += 1

    def begin_step_on_device(self) -> None:
        """``begin_step`` without host data: nothing is copied, one launch advances the metadata."""
        self.note_step()
        self.advance_on_device()

    # views of the step's metadata, all int32 device [B]
    def _row(self, r: int) -> torch.Tensor:
        return self._meta[r, : self.batch]

    @property
    def positions(self) -> torch.Tensor:
        return self._row(_POSITION)

    @property
    def dst_slots(self) -> torch.Tensor:
        return self._row(_DST_SLOT)

    @property
    def selected(self) -> torch.Tensor:
        return self._row(_SELECTED)

    def rope_table(self, rope_scale: float = 1.0, rope_theta: float = 1e4):
        """cos, sin ``[B, D/2]`` of the new tokens' positions (once per step, all layers)."""
        return _kernels.rope_table(self.positions, self.head_dim, rope_scale, rope_theta)

    # ---- cache writes -------------------------------------------------------------------------
    def append_prompt(self, b: int, k: torch.Tensor, v: torch.Tensor, layer_idx: int) -> None:
        """Write the (already rotated) prompt K/V ``[n, H_kv, D]`` of sequence b: its first n tokens."""
        n, P = k.size(0), self.page_size
        n_pages = -(-n // P)
        indptr = torch.tensor([0, n_pages], dtype=torch.int32, device=self.device)
        fn = _kernels.append_kv_cache_prefill if n > 1 else _kernels.append_kv_cache_decode
        fn(k, v, self.buf_layer(layer_idx), self.page_table[b, :n_pages], indptr, (n - 1) % P + 1,
           self._pages[b][n_pages - 1], None, None, None, 0, 0, int(self.layout))

    def rope_append(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, layer_idx: int,
                    rope_scale: float = 1.0, rope_theta: float = 1e4) -> None:
        """Rotate q ``[B, H_q, D]`` in place and store the rotated k and v ``[B, H_kv, D]`` of the
        step's new tokens (the un-fused form of ``fresh=``)."""
        _kernels.rope_append_decode(q, k, v, self.buf_layer(layer_idx), self.positions,
                                    self.dst_slots, int(self.layout), rope_scale, rope_theta)

    # ---- attention ----------------------------------------------------------------------------
    def _fresh(self, fresh):
        if fresh is None:
            return None
        k, v, cos, sin = fresh
        return (k, v, cos, sin, self.dst_slots)

    def attend_full(self, q: torch.Tensor, layer_idx: int, output_qk_product: bool = False,
                    fresh=None) -> torch.Tensor:
        """Attention of every sequence's new token over its whole cache; with
        ``output_qk_product`` the logits and log-sum-exps are kept for ``select``.
        ``fresh=(k, v, cos, sin)`` folds RoPE and the append of the new tokens into the launch."""
        B = self.batch
        o = torch.empty_like(q)
        self._handle.forward(
            q, o, self.buf_layer(layer_idx), self.page_table.view(1, -1),
            self._table_starts[: B + 1], self._row(_LAST_LEN), self._row(_LAST_IDX),
            self.qk_product[: B * self.num_heads] if output_qk_product else None,
            lse=self.lse[:B] if output_qk_product else None,
            n_list=-(-max(self._cap) // self.page_size) - 1, counts=self._row(_PAGES_BEFORE_LAST),
            fresh=self._fresh(fresh))
        return o

    def select(self) -> None:
        """Top-k of the last ``attend_full(..., output_qk_product=True)`` for every sequence:
        physical token slots, sorted by position, in its segment of ``topk_dindices_buffer``."""
        B, P, k = self.batch, self.page_size, self.budget
        n = max(self._cap)   # an upper bound; every sequence's own length is read on the device
        rows = self.index_rows
        scores, bound = self.qk_product[: B * self.num_heads], self.lse[:B].view(-1)
        if self.select_mode != "per_head":
            # the B * H_q logit rows form B * rows groups of consecutive heads: one grouped sum
            _kernels.score_reduce(scores, self.lse[:B].view(-1), B * rows, n, "group_sum",
                                  out=self.score_sum[: B * rows])
            scores, bound = self.score_sum[: B * rows], self.score_bound[: B * rows]
        k_eff = min(k, n)
        # one call: row b * rows + r is row r of sequence b, ranks that sequence's tokens only
        # (its length is read on the device) and goes through that sequence's page table
        out = self._slots[: B * rows, :k_eff]
        _kernels.topk_filtering(scores[:, :n], None, None, out, self.topk_buf, k_eff,
                                page_table=self.page_table[:B], page_size=P,
                                lengths=self._row(_SEQ_LEN), upper_bound=bound)
        self.topk_dindices_buffer.view(rows, self.max_batch, k)[:, :B, :k_eff] = \
            out.view(B, rows, k_eff).permute(1, 0, 2)

    def attend_sparse(self, q: torch.Tensor, layer_idx: int, fresh=None) -> torch.Tensor:
        """Attention over the persisted token lists (``fresh`` as in ``attend_full``)."""
        B = self.batch
        o = torch.empty_like(q)
        self._handle.forward(q, o, self.buf_layer(layer_idx), self.topk_dindices_buffer,
                             self._list_starts[: B + 1], 0, 0, None, index_kind="slots",
                             n_list=min(self.budget, max(self._cap)), counts=self.selected,
                             fresh=self._fresh(fresh))
        return o

"""Paged KV storage of one sequence and the decode handle that runs attention over it.

Three things live here because they share one piece of state, the page table:

* ``TensorLayout``   the two page layouts the kernels take (tidal/utils/utils.py:1-5),
* ``KvPool``/``KvCache``   page allocator and per-sequence page table (the roles of
  tidal/utils/kv_cache.py:8-137),
* ``BatchDecodeWithPagedKVCacheWrapper``   the per-forward-pass decode handle (the role of
  tidal/utils/decode_wrapper.py:13-88).

What differs from the reference's behaviour, on purpose:

* each layer owns its pages (the reference folds four layers onto one buffer,
  kv_cache.py:84,115-117), so a cache written by layer i is never overwritten by layer i+4;
* reserving tokens costs O(new pages): the page count is computed, not discovered token by token
  (kv_cache.py:124-129);
* the page table is mirrored in an int32 device tensor that grows in place, so a decode step
  uploads at most one new entry instead of the whole table;
* grouped-query models size the pool by their KV heads.
"""
import enum
from typing import List, Optional

import torch

from .. import _kernels


class TensorLayout(enum.IntEnum):
    """Order of the (token, head) axes inside a page: NHD = [token, head, dim] (the layout every
    kernel here is tuned for), HND = [head, token, dim]."""

    NHD = 0
    HND = 1

    @classmethod
    def parse(cls, name: str) -> "TensorLayout":
        """'NHD' / 'HND' -> member; anything else is a KeyError with the reference's message
        (decode_wrapper.py:8-10, spelling included, since callers match on it)."""
        try:
            return cls[name]
        except KeyError:
            raise KeyError("Invalide kv_layout {}".format(name)) from None


# the reference keeps this map as a class attribute; an enum cannot hold a dict member
TensorLayout.FORMAT2STR = {int(m): m.name for m in TensorLayout}


def _check_kv_layout(kv_layout: str) -> None:
    TensorLayout.parse(kv_layout)


def _page_shape(layout: int, block_len: int, num_heads: int, head_dim: int):
    inner = (block_len, num_heads, head_dim) if int(layout) == TensorLayout.NHD else \
        (num_heads, block_len, head_dim)
    return (2,) + inner          # K plane, V plane


class KvPool:
    """``capacity`` pages for every layer in one allocation ``[layer, page, 2, ...page...]``, and
    a stack of the page ids nobody holds.

    ``page_order_seed`` shuffles the hand-out order so that tests and benchmarks can run on a
    scattered page table; without it pages come out 0, 1, 2, ...
    """

    def __init__(self, num_layers: int, num_heads: int, head_dim: int, capacity: int,
                 block_len: int, dtype: torch.dtype, device: torch.device,
                 layout: int = TensorLayout.NHD, page_order_seed=None):
        self.layout = layout
        self.block_len = int(block_len)
        self.capacity = int(capacity)
        self.num_layers = int(num_layers)
        self.buf = torch.empty((self.num_layers, self.capacity)
                               + _page_shape(layout, self.block_len, num_heads, head_dim),
                               dtype=dtype, device=device)
        if page_order_seed is None:
            order = range(self.capacity)
        else:
            order = torch.randperm(
                self.capacity, generator=torch.Generator().manual_seed(int(page_order_seed))
            ).tolist()
        self._stack: List[int] = list(order)[::-1]       # next page to hand out is at the end
        self._held = bytearray(self.capacity)            # 1 = handed out

    @property
    def num_free_blocks(self) -> int:
        return len(self._stack)

    def take(self, n: int) -> List[int]:
        """Hand out ``n`` pages at once.  Running dry raises KeyError like the reference's
        ``set.pop()`` does (kv_cache.py:60-62) and hands out nothing."""
        if n > len(self._stack):
            raise KeyError("pop from an empty set")
        pages = [self._stack.pop() for _ in range(n)]
        for p in pages:
            self._held[p] = 1
        return pages

    def give_back(self, pages) -> None:
        for p in pages:
            if not (0 <= p < self.capacity and self._held[p]):
                raise AssertionError("page {} is not held".format(p))
            self._held[p] = 0
            self._stack.append(p)

    # one-page forms under the reference's names (kv_cache.py:60-67)
    def alloc_block(self) -> int:
        return self.take(1)[0]

    def free_block(self, idx: int) -> None:
        self.give_back((idx,))


class KvCache:
    """Page table of one sequence over a pool sized for ``max_seq_len`` tokens.

    ``indicies`` (the reference's spelling) is the host-side table; ``indices_device`` is the
    same table in HBM, which is what the kernels read.
    """

    def __init__(self, num_layers, num_heads, head_dim, max_seq_len: int, page_size,
                 dtype: torch.dtype, device: torch.device, layout: int = TensorLayout.NHD,
                 page_order_seed=None):
        if max_seq_len <= 0:
            raise ValueError("init_len must be non-negative")
        self.pool = KvPool(num_layers, num_heads, head_dim, -(-max_seq_len // page_size),
                           page_size, dtype, device, layout, page_order_seed)
        self.indicies: List[int] = []
        self.seqlen = 0
        self._table_dev = torch.zeros(self.pool.capacity, dtype=torch.int32, device=device)

    @property
    def last_page_len(self) -> int:
        """tokens in the last page, in 1..page_size (page_size, not 0, on an exact fill)"""
        return (self.seqlen - 1) % self.pool.block_len + 1

    @property
    def indices_device(self) -> torch.Tensor:
        """int32 [pages in use], physical page ids in sequence order"""
        return self._table_dev[: len(self.indicies)]

    def buf_layer(self, layer_idx: int) -> torch.Tensor:
        return self.pool.buf[layer_idx % self.pool.num_layers]

    def append_seq(self, seq_len: int) -> int:
        """Make room for ``seq_len`` more tokens; returns how many pages that took."""
        if seq_len <= 0:
            return 0
        have = len(self.indicies)
        grow = max(-(-(self.seqlen + seq_len) // self.pool.block_len) - have, 0)
        if grow:
            fresh = self.pool.take(grow)
            self._table_dev[have: have + grow] = torch.tensor(fresh, dtype=torch.int32)
            self.indicies += fresh
        self.seqlen += seq_len
        return grow

    def release(self) -> None:
        """Forget the sequence and return its pages."""
        self.pool.give_back(self.indicies)
        del self.indicies[:]
        self.seqlen = 0


class BatchDecodeWithPagedKVCacheWrapper:
    """One decode handle for a whole forward pass: ``begin_forward`` fixes the split-K plan and
    the scratch buffer for the pass's shape, every layer's ``forward`` reuses them, and
    ``end_forward`` drops the plan."""

    def __init__(self, kv_layout: str = "NHD"):
        layout = TensorLayout.parse(kv_layout)
        self.kv_layout = kv_layout
        self._wrapper = _kernels.BatchDecodeWithPagedKVCachePyTorchWrapper(layout)

    def begin_forward(self, indptr: Optional[torch.Tensor], num_qo_heads: int, num_kv_heads: int,
                      head_dim: int, page_size: int, data_type):
        # the handle learns the element type from an empty tensor (decode_wrapper.py:40-46)
        self._wrapper.begin_forward(indptr, num_qo_heads, num_kv_heads, head_dim, page_size,
                                    torch.empty(0, dtype=data_type))

    def forward(self, q: torch.Tensor, o: torch.Tensor, paged_kv_data: torch.Tensor,
                paged_kv_indices: torch.Tensor, paged_kv_indptr: Optional[torch.Tensor],
                paged_kv_last_page_len, paged_kv_last_page_idx,
                qk_product: Optional[torch.Tensor] = None, rope_scale: Optional[float] = None,
                rope_theta: Optional[float] = None, **extensions):
        """Arguments as decode_wrapper.py:53-88; ``extensions`` are this library's additions
        (``index_kind``, fused RoPE/append operands, ...) and go to the handle untouched."""
        self._wrapper.forward(q, o, paged_kv_data, paged_kv_indices, paged_kv_indptr,
                              paged_kv_last_page_len, paged_kv_last_page_idx, qk_product,
                              1.0 if rope_scale is None else rope_scale,
                              1e4 if rope_theta is None else rope_theta, **extensions)

    def end_forward(self):
        self._wrapper.end_forward()

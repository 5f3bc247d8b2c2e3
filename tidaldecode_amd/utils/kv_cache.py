"""Paged KV pool and the per-sequence page list (counterpart of tidal/utils/kv_cache.py:8-137).

Differences from the reference: every layer has its own buffer (the reference aliases four
layers onto one, kv_cache.py:84,115-117); ``append_seq`` is O(new pages) instead of a Python
loop over tokens (kv_cache.py:124-129); the page list is mirrored in a device tensor that is
extended in place, so nothing is re-uploaded per decode step; GQA pools hold ``num_kv_heads``.
"""
from typing import List

import torch

from .utils import TensorLayout


class KvPool:
    def __init__(self, num_layers: int, num_heads: int, head_dim: int, capacity: int,
                 block_len: int, dtype: torch.dtype, device: torch.device,
                 layout: int = TensorLayout.NHD, page_order_seed=None):
        self._layout = layout
        if layout == TensorLayout.NHD:
            shape = (num_layers, capacity, 2, block_len, num_heads, head_dim)
        else:
            shape = (num_layers, capacity, 2, num_heads, block_len, head_dim)
        self._buf = torch.empty(shape, dtype=dtype, device=device)
        self._block_len = block_len
        # pop() hands out ascending page ids, or a seeded random order (scattered pages)
        self._free = list(range(capacity - 1, -1, -1))
        if page_order_seed is not None:
            g = torch.Generator().manual_seed(int(page_order_seed))
            self._free = torch.randperm(capacity, generator=g).tolist()
        self._free_set = set(self._free)

    @property
    def layout(self):
        return self._layout

    @property
    def buf(self):
        return self._buf

    @property
    def num_layers(self):
        return self._buf.shape[0]

    @property
    def block_len(self):
        return self._block_len

    @property
    def num_free_blocks(self):
        return len(self._free)

    @property
    def capacity(self):
        return self._buf.shape[1]

    def alloc_block(self) -> int:
        if not self._free:
            raise KeyError("pop from an empty set")  # the reference's set.pop() on exhaustion
        idx = self._free.pop()
        self._free_set.discard(idx)
        return idx

    def free_block(self, idx: int):
        assert 0 <= idx < self.capacity
        assert idx not in self._free_set
        self._free.append(idx)
        self._free_set.add(idx)


class KvCache:
    """Key-value cache of one sequence."""

    def __init__(self, num_layers, num_heads, head_dim, max_seq_len: int, page_size,
                 dtype: torch.dtype, device: torch.device, layout: int = TensorLayout.NHD,
                 page_order_seed=None):
        if max_seq_len <= 0:
            raise ValueError("init_len must be non-negative")
        self._pool = KvPool(num_layers=num_layers, num_heads=num_heads, head_dim=head_dim,
                            capacity=(max_seq_len + page_size - 1) // page_size,
                            block_len=page_size, dtype=dtype, device=device, layout=layout,
                            page_order_seed=page_order_seed)
        self._indicies: List[int] = []
        self._seqlen = 0
        # device mirror of the page list; entries past len(self._indicies) are unused
        self._indices_dev = torch.zeros(self._pool.capacity, dtype=torch.int32, device=device)

    @property
    def pool(self) -> KvPool:
        return self._pool

    @property
    def seqlen(self) -> int:
        return self._seqlen

    @property
    def last_page_len(self) -> int:
        return (self.seqlen - 1) % self._pool.block_len + 1

    @property
    def indicies(self) -> List[int]:
        return self._indicies

    @property
    def indices_device(self) -> torch.Tensor:
        """int32 device tensor [num_pages] of the physical pages, in sequence order"""
        return self._indices_dev[: len(self._indicies)]

    def buf_layer(self, layer_idx: int):
        return self._pool.buf[layer_idx % self._pool.num_layers]

    def append_seq(self, seq_len: int) -> int:
        """Reserve space for tokens and return the number of new pages."""
        if seq_len <= 0:
            return 0
        page = self._pool.block_len
        need = (self._seqlen + seq_len + page - 1) // page - len(self._indicies)
        if need > 0:
            start = len(self._indicies)
            new = [self._pool.alloc_block() for _ in range(need)]
            self._indicies.extend(new)
            self._indices_dev[start: start + need] = torch.tensor(new, dtype=torch.int32)
        self._seqlen += seq_len
        return max(need, 0)

    def release(self):
        """Release all blocks."""
        self._seqlen = 0
        for idx in self._indicies:
            self._pool.free_block(idx)
        self._indicies.clear()

"""Pinned host arena for offloaded requests, carved by a buddy allocator whose
unit is one page of every layer (deserve_worker/kvcache/paged/chunk_pool.py:10-113).
A chunk of level k holds 2**k page-units laid out (L * n, 2, P, Hkv, D), layer
major - the layout KVCacheManager writes."""
from __future__ import annotations

import threading
from dataclasses import dataclass

import torch

from deserve_amd.kvcache._alloc import BuddyIndex
from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty


@dataclass
class ChunkHandle:
    id: int
    level: int
    initial_size: int
    pool: "ChunkPool"

    def free(self) -> None:
        self.pool.free(self.id, self.level)

    def retrieve(self) -> torch.Tensor:
        begin, end = BuddyIndex.span(self.id, self.level)
        return self.pool.chunks[begin * self.pool.num_layers: end * self.pool.num_layers]


class ChunkPool:
    def __init__(self, num_layers: int, height: int, page_size: int, main_device: torch.device,
                 main_dtype: torch.dtype, n_kv_heads: int = 8, head_dim: int = 128):
        self.num_layers, self.height, self.page_size = num_layers, height, page_size
        self.main_device, self.main_dtype = torch.device(main_device), main_dtype
        self.mutex = threading.Lock()
        self.per_token_shape = (2, page_size, n_kv_heads, head_dim)
        self.chunks = pinned_empty(((1 << (height - 1)) * num_layers,) + self.per_token_shape,
                                   main_dtype)
        self._buddy = BuddyIndex(height)

    @property
    def available_ids(self) -> list:
        return self._buddy.levels

    def split(self, begin: int, end: int) -> None:
        """Public as in the reference (chunk_pool.py:51-59); like there, the caller holds
        the mutex or owns the pool."""
        self._buddy.split(begin, end)

    def alloc(self, size: int) -> ChunkHandle:
        with self.mutex:
            cid, level = self._buddy.alloc(size)   # RuntimeError when exhausted
        return ChunkHandle(cid, level, size, self)

    def free(self, id: int, level: int) -> None:
        with self.mutex:
            self._buddy.release(id, level)


class CpuChunkPool(ChunkPool):
    def __init__(self, num_layers: int, height: int, page_size: int, main_dtype: torch.dtype,
                 n_kv_heads: int = 8, head_dim: int = 128):
        super().__init__(num_layers, height, page_size, torch.device("cpu"), main_dtype,
                         n_kv_heads, head_dim)

"""One request's cache: a block-table row over a pool, growing by whole pages
(deserve_worker/kvcache/paged/kvcache.py:12-37)."""
from __future__ import annotations

from typing import Generic, TypeVar

from deserve_amd.kvcache.paged.page_pool import CpuPagePool, GpuPagePool, PagePool
from deserve_amd.kvcache.paged.page_table import PageTableAllocator, PageTableHandle

PoolT = TypeVar("PoolT", bound=PagePool)


class PagedKVCache(Generic[PoolT]):
    def __init__(self, page_table: PageTableHandle, pool: PoolT) -> None:
        self.page_table, self.pool = page_table, pool

    @classmethod
    def empty(cls, allocator: PageTableAllocator, pool: PoolT) -> "PagedKVCache[PoolT]":
        return cls(allocator.alloc(), pool)

    def _grow(self, num_tokens: int):
        """Page ids newly allocated so that num_tokens fit (None if nothing to do)."""
        have = self.page_table.occupied
        if num_tokens <= have * self.pool.page_size:
            return None
        return self.pool.alloc(self.pool.calc_num_pages(num_tokens) - have)

    def extend(self, num_tokens: int) -> bool:
        fresh = self._grow(num_tokens)
        if fresh is not None:
            self.page_table.extend(fresh)
        return True

    def free(self) -> None:
        self.pool.free(self.page_table.retrieve())
        self.page_table.free()


GpuPagedKVCache = PagedKVCache[GpuPagePool]
CpuPagedKVCache = PagedKVCache[CpuPagePool]

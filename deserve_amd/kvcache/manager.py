"""Per-request offload / reload of scattered pages
(deserve_worker/kvcache/manager.py:12-89).

A request's pages are named by its block table and lie anywhere in the pool.
Offload packs them, all layers at once, into the request's pinned chunk in the
layout (L * n, 2, P, Hkv, D) - layer major, then block-table order - and reload
does the reverse into freshly allocated pages.  Both are enqueued on the swap
engine's side streams (gather/scatter kernel + one large copy per staging
chunk) instead of the reference's blocking advanced-index copy; ``synchronize``
blocks the host until they are done, and the compute stream is fenced behind
them so a caller that keeps the reference's call order sees the same results.
"""
from __future__ import annotations

import torch

from deserve_amd.kvcache import _native
from deserve_amd.kvcache.paged.chunk_pool import ChunkHandle, CpuChunkPool
from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.kvcache.paged.page_table import PageTableAllocator
from deserve_amd.kvcache.virtual import VirtualPagedKVCache, VirtualPagePool


class KVCacheManager:
    def __init__(self, virtual_page_pool: VirtualPagePool, cpu_chunk_pool: CpuChunkPool,
                 page_table_allocator: PageTableAllocator, staging_bytes: int = 128 << 20):
        self.virtual_page_pool = virtual_page_pool
        self.cpu_chunk_pool = cpu_chunk_pool
        self.page_table_allocator = page_table_allocator
        # the pool's engine (its two streams also carry the bulk slice swap) unless another
        # staging size is asked for
        shared = getattr(virtual_page_pool, "engine", None)
        self.engine = shared if shared is not None and staging_bytes == shared.staging_bytes \
            else _native.SwapEngine(staging_bytes)

    def copy_gpu_to_cpu(self, paged_kvcache: PagedKVCache[VirtualPagePool],
                        task_id: str) -> ChunkHandle:
        """Only the copy; the caller frees the GPU pages and owns the handle."""
        table = paged_kvcache.page_table
        n = table.occupied
        handle = self.cpu_chunk_pool.alloc(n)
        rows = n * self.cpu_chunk_pool.num_layers
        self.engine.swap_out(handle.retrieve()[:rows], self.virtual_page_pool, table.retrieve())
        # pages may be handed to another request right after this returns
        self.engine.fence()
        return handle

    def copy_cpu_to_gpu(self, chunk_handle: ChunkHandle, task_id: str) -> VirtualPagedKVCache:
        """Only the copy; the caller frees the chunk and owns the new cache."""
        pool = self.virtual_page_pool
        n = chunk_handle.initial_size
        ids = pool.alloc(n)
        if ids is None:
            raise RuntimeError("Failed to allocate page tables")
        table = self.page_table_allocator.alloc()
        table.extend(ids)
        rows = n * self.cpu_chunk_pool.num_layers
        self.engine.swap_in(pool, chunk_handle.retrieve()[:rows], ids)
        self.engine.fence()   # attention on the current stream must see the pages
        isswap = torch.zeros((self.page_table_allocator.max_context_len,), dtype=torch.bool)
        isswap[:n] = ids >= pool.num_pages_main
        return VirtualPagedKVCache(page_table=table, isswap=isswap, pool=pool)

    def synchronize(self) -> None:
        self.engine.wait()

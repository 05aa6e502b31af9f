"""One microbatch ("round") of a stage: its live per-request caches, its pinned
image of a swap slice, and the call order that lets the bulk swap of the OTHER
slice overlap this microbatch's compute
(deserve_worker/engine/microbatch/processor.py:24-149).

step():  prepare (metadata, page allocation, attention plan)
      -> swap2(next.pinned_memory, prev.pinned_memory)   enqueue-only, side streams
      -> forward of every layer on the compute stream.
The pipeline processor joins the side streams at the start of the next step.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from deserve_amd.execution.exec import BatchDecode, BatchPrefill
from deserve_amd.execution.result import BatchResult
from deserve_amd.kvcache.manager import KVCacheManager
from deserve_amd.kvcache.paged.chunk_pool import ChunkHandle
from deserve_amd.kvcache.paged.page_table import PageTableAllocator
from deserve_amd.kvcache.virtual import CopiedPinnedMemory, VirtualPagedKVCache
from deserve_amd.task import TaskManager


class MicroBatchProcessor:
    def __init__(self, kvcache_manager: KVCacheManager, task_data_manager: TaskManager,
                 layer_storage, page_table_allocator: PageTableAllocator, ignore_eos: bool) -> None:
        pool = kvcache_manager.virtual_page_pool
        self.kvcache_manager = kvcache_manager
        self.pinned_memory = CopiedPinnedMemory(pool.calc_swap_size(), pool.num_pages_swap,
                                                pool.main_device, pool.main_dtype)
        self.task_data_manager = task_data_manager
        self.layer_storage = layer_storage
        self.page_table_allocator = page_table_allocator
        self.ongoing_paged_kvcaches: Dict[str, VirtualPagedKVCache] = {}
        self.ignore_eos = ignore_eos

    # ---- request life cycle
    def join(self, task_ids: List[str]) -> None:
        pool = self.kvcache_manager.virtual_page_pool
        for tid in task_ids:
            self.ongoing_paged_kvcaches[tid] = VirtualPagedKVCache.empty(self.page_table_allocator, pool)

    def cancel(self, task_ids: List[str]) -> None:
        for tid in task_ids:
            cache = self.ongoing_paged_kvcaches.pop(tid, None)
            if cache is not None:
                cache.free()

    def adjust(self) -> None:
        """With an odd number of rounds a microbatch lands in the other swap slice
        every time: re-base the page ids that lie in a swap slice."""
        pool = self.kvcache_manager.virtual_page_pool
        offset = pool.num_pages_swap if pool.on == 1 else -pool.num_pages_swap
        for cache in self.ongoing_paged_kvcaches.values():
            cache.adjust(offset)

    def offload(self, task_ids: List[str]) -> List[ChunkHandle]:
        """Copy the requests' pages to pinned chunks (all copies first), then free the pages."""
        caches = [self.ongoing_paged_kvcaches.pop(tid) for tid in task_ids]
        handles = [self.kvcache_manager.copy_gpu_to_cpu(c, tid) for c, tid in zip(caches, task_ids)]
        for c in caches:
            c.free()
        return handles

    def reload(self, task_ids: List[str], cpu_chunk_handles: List[ChunkHandle]) -> None:
        """Bring offloaded requests back into freshly allocated pages, then free the chunks."""
        for tid, handle in zip(task_ids, cpu_chunk_handles):
            self.ongoing_paged_kvcaches[tid] = self.kvcache_manager.copy_cpu_to_gpu(handle, tid)
        for handle in cpu_chunk_handles:
            handle.free()

    # ---- execution
    def _make_exec(self, xs, task_ids: List[str]):
        tasks = [self.task_data_manager.get(tid) for tid in task_ids]
        caches = [self.ongoing_paged_kvcaches[tid] for tid in task_ids]
        kind = BatchDecode if all(t.seqlen == 1 for t in tasks) else BatchPrefill
        return kind(xs, self.layer_storage, tasks, caches)

    def exec(self, xs, task_ids: List[str]) -> BatchResult:
        """Decode step without the microbatch swap (reference: processor.py:96-105)."""
        ex = self._make_exec(xs, task_ids)
        ex.prepare()
        return ex.step(self.ignore_eos)

    def step(self, task_ids: List[str], xs, prev_group: "MicroBatchProcessor",
             next_group: "MicroBatchProcessor") -> BatchResult:
        ex = self._make_exec(xs, task_ids)
        ex.prepare()
        self.kvcache_manager.virtual_page_pool.swap2(next_group.pinned_memory, prev_group.pinned_memory)
        return ex.step(self.ignore_eos)

    def synchronize(self) -> None:
        self.kvcache_manager.synchronize()


class MicroBatchScheduler(MicroBatchProcessor):
    """First-stage variant that can park decode inputs of suspended requests
    (deserve_worker/engine/microbatch/scheduler.py:10-38)."""

    def __init__(self, *args, **kwargs) -> None:
        super().__init__(*args, **kwargs)
        self.suspended_decodes: Dict[str, torch.Tensor] = {}
        self.suspended_prefills: Dict[str, torch.Tensor] = {}

    def suspend(self, task_ids: List[str], xs: torch.Tensor) -> None:
        for i, tid in enumerate(task_ids):          # one row per request (decode)
            self.suspended_decodes[tid] = xs[i: i + 1]

    def resume(self, task_ids: List[str]) -> torch.Tensor:
        return torch.cat([self.suspended_decodes.pop(tid) for tid in task_ids], dim=0)

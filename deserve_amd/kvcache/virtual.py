"""Main region + two swap slices that double-buffer per-microbatch pages
(deserve_worker/kvcache/virtual.py:12-161).

Pool pages [0, main) are always resident; slices [main, main+swap) and
[main+swap, main+2*swap) alternate between "on" (the running microbatch
allocates from it) and "off" (being dumped to / refilled from pinned host memory
on two side streams while the running microbatch computes).

The bulk copy follows the semantics the reference states in
``VirtualPagePool.swap`` (virtual.py:97-113): pinned memory viewed
(L, S, 2, P, Hkv, D), every layer's slice dumped, then refilled.  The reference's
``swap.cpp`` walks the strided slice as if it were contiguous and sizes each copy
in elements instead of bytes (swap.cpp:33-41); that defect is not reproduced.
"""
from __future__ import annotations

import torch

from deserve_amd.kvcache import _native
from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.kvcache.paged.page_pool import GpuPagePool
from deserve_amd.kvcache.paged.page_table import PageTableAllocator, PageTableHandle
from deserve_amd.kvcache.pinned.pinned_memory import PinnedMemory


class CopiedPinnedMemory(PinnedMemory):
    """A microbatch's pinned image of one swap slice plus the slice's saved
    free-bitmap and free count (virtual.py:12-16)."""

    def __init__(self, size: int, num_pages_swap: int, device: torch.device,
                 dtype: torch.dtype = torch.float16) -> None:
        super().__init__(size, dtype)
        self.bitmap = torch.ones((num_pages_swap,), dtype=torch.bool)
        self.count = num_pages_swap


class VirtualPagePool(GpuPagePool):
    def __init__(self, num_layers: int, num_pages_main: int, num_pages_swap: int, page_size: int,
                 main_device: torch.device, main_dtype: torch.dtype, n_kv_heads: int = 8,
                 head_dim: int = 128, swap_staging_bytes: int = 128 << 20):
        super().__init__(num_layers, num_pages_main + 2 * num_pages_swap, page_size, main_device,
                         main_dtype, n_kv_heads, head_dim)
        m, s = num_pages_main, num_pages_swap
        self.num_pages_main, self.num_pages_swap = m, s
        self.slices = [(m, m + s), (m + s, m + 2 * s)]
        self._index.free[m + s: m + 2 * s] = False        # slice 1 starts "off"
        self._index.avail = m + s
        self.swap_bitmap = torch.ones((s,), dtype=torch.bool)
        self.swap_count = s
        self.on = 0
        # The two side streams of the reference (virtual.py:48-49) are those of one swap
        # engine, which the per-request offload / reload (KVCacheManager) shares: a stage
        # process then holds three streams - compute and these two - each on a hardware
        # queue of its own, which the engine verifies when it is created.
        self.engine = None
        self.stream = self.stream2 = None
        if self.main_device.type == "cuda":
            with torch.cuda.device(self.main_device):
                self.engine = _native.SwapEngine(swap_staging_bytes)
                out_stream, in_stream = self.engine.streams()
            self.stream = torch.cuda.ExternalStream(out_stream, device=self.main_device)
            self.stream2 = torch.cuda.ExternalStream(in_stream, device=self.main_device)

    def switch(self) -> None:
        """Flip the active slice (virtual.py:54-77): unused prefetched ids go
        back to the bitmap, the active slice's free set is parked in
        swap_bitmap/swap_count, the other slice's parked set becomes live."""
        with self.mutex:
            idx = self._index
            idx.flush_queue()
            a, b = self.slices[self.on]
            c, d = self.slices[1 - self.on]
            remained = int(idx.free[a:b].sum())
            idx.avail += self.swap_count - remained
            idx.free[c:d] = self.swap_bitmap.numpy()
            self.swap_bitmap = torch.from_numpy(idx.free[a:b].copy())
            self.swap_count = remained
            idx.free[a:b] = False
            self.on = 1 - self.on

    def _exchange_records(self, from_memory: CopiedPinnedMemory, to_memory: CopiedPinnedMemory,
                          clone: bool) -> tuple:
        to_memory.bitmap = self.swap_bitmap.clone() if clone else self.swap_bitmap
        to_memory.count = self.swap_count
        self.swap_bitmap, self.swap_count = from_memory.bitmap, from_memory.count
        return self.slices[1 - self.on]

    def swap2(self, from_memory: CopiedPinnedMemory, to_memory: CopiedPinnedMemory) -> None:
        """Dump the inactive slice to ``to_memory`` and refill it from
        ``from_memory`` (virtual.py:79-95); returns once the copies are
        enqueued: first half of the layers on ``stream``, the rest on
        ``stream2``.  Both streams first wait for the work already enqueued on
        the current stream."""
        begin, end = self._exchange_records(from_memory, to_memory, clone=False)
        ready = torch.cuda.current_stream().record_event()
        self.stream.wait_event(ready)
        self.stream2.wait_event(ready)
        _native.swap_slice(self, begin, end, to_memory.memory, from_memory.memory,
                           self.stream.cuda_stream, self.stream2.cuda_stream)

    def swap(self, from_memory: CopiedPinnedMemory, to_memory: CopiedPinnedMemory) -> None:
        """Single-stream form of swap2 (virtual.py:97-113)."""
        begin, end = self._exchange_records(from_memory, to_memory, clone=True)
        self.stream.wait_event(torch.cuda.current_stream().record_event())
        _native.swap_slice(self, begin, end, to_memory.memory, from_memory.memory,
                           self.stream.cuda_stream, self.stream.cuda_stream)

    def calc_swap_size(self) -> int:
        """Elements of one microbatch's pinned image."""
        return (self.num_layers * self.num_pages_swap * 2 * self.page_size * self.n_kv_heads *
                self.head_dim)


class VirtualPagedKVCache(PagedKVCache[VirtualPagePool]):
    """Remembers which block-table entries lie in a swap slice so they can be
    re-based when the microbatch lands in the other slice (virtual.py:119-161)."""

    def __init__(self, page_table: PageTableHandle, isswap: torch.Tensor,
                 pool: VirtualPagePool) -> None:
        super().__init__(page_table, pool)
        self.isswap = isswap

    @classmethod
    def empty(cls, allocator: PageTableAllocator, pool: VirtualPagePool) -> "VirtualPagedKVCache":
        return cls(allocator.alloc(), torch.zeros((allocator.max_context_len,), dtype=torch.bool),
                   pool)

    def extend(self, num_tokens: int) -> bool:
        have = self.page_table.occupied
        fresh = self._grow(num_tokens)
        if fresh is not None:
            self.isswap[have: have + fresh.shape[0]] = fresh >= self.pool.num_pages_main
            self.page_table.extend(fresh)
        return True

    def adjust(self, offset: int) -> None:
        n = self.page_table.occupied
        row = self.page_table.retrieve()
        row[self.isswap[:n]] += offset

    def free(self) -> None:
        super().free()
        self.isswap = torch.empty((0,), dtype=torch.bool)

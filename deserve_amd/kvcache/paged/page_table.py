"""Block tables (deserve_worker/kvcache/paged/page_table.py:7-60): one int32
row of page ids per request, rows handed out LIFO.  The table is host memory;
the kernels read the per-step CSR arrays that the forward context assembles
from these rows and uploads once."""
from __future__ import annotations

import threading
from dataclasses import dataclass

import torch

from deserve_amd.kvcache._alloc import SlotStack


class PageTableAllocator:
    def __init__(self, max_requests_num: int, max_context_len: int, page_size: int,
                 main_device: torch.device) -> None:
        self.max_requests_num, self.max_context_len = max_requests_num, max_context_len
        self.page_size, self.main_device = page_size, torch.device(main_device)
        self.mutex = threading.Lock()
        self.tables = torch.zeros((max_requests_num, max_context_len // page_size),
                                  dtype=torch.int32)
        self._stack = SlotStack(max_requests_num)

    @property
    def slots(self) -> list:
        return self._stack.items

    def alloc(self) -> "PageTableHandle":
        with self.mutex:
            row = self._stack.pop()          # ValueError("No available slots") when empty
        return PageTableHandle(row, 0, self)

    def free(self, handle: "PageTableHandle") -> None:
        with self.mutex:
            self._stack.push(handle.offset)


@dataclass
class PageTableHandle:
    offset: int
    occupied: int
    allocator: PageTableAllocator

    def retrieve(self) -> torch.Tensor:
        return self.allocator.tables[self.offset, : self.occupied]

    def retrieve_all(self) -> torch.Tensor:
        return self.allocator.tables[self.offset]

    def extend(self, fill: torch.Tensor) -> None:
        end = self.occupied + fill.shape[0]
        width = self.allocator.tables.shape[1]
        if end > width:
            raise ValueError(f"block table row holds {width} pages, cannot grow to {end}")
        self.allocator.tables[self.offset, self.occupied:end] = fill.to("cpu", torch.int32)
        self.occupied = end

    def free(self) -> None:
        self.allocator.free(self)

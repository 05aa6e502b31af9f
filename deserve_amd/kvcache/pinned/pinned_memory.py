"""Pinned host buffer (deserve_worker/kvcache/pinned/pinned_memory.py:4-9).
The reference hard-codes float16; the element type is a parameter here."""
import torch


def pinned_empty(shape, dtype: torch.dtype) -> torch.Tensor:
    """Page-locked host tensor; plain host memory when no GPU is present
    (allocator-only use on a CPU box)."""
    return torch.empty(shape, dtype=dtype, device="cpu", pin_memory=torch.cuda.is_available())


class PinnedMemory:
    def __init__(self, size: int, dtype: torch.dtype = torch.float16) -> None:
        self.size = 0
        self.memory = pinned_empty((size,), dtype)

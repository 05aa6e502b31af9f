"""Paged KV storage (deserve_worker/kvcache/paged/page_pool.py:7-107).

``pages`` keeps the reference layout (num_layers, num_pages, 2, page_size,
n_kv_heads, head_dim) on ``main_device``.  Allocation state is the host-side
``FreePageIndex``; the reference's attribute names (``page_bitmap``,
``page_buffer``, ``num_avails``) are views of it.
"""
from __future__ import annotations

import threading
from typing import Optional

import numpy as np
import torch

from deserve_amd.kvcache._alloc import FreePageIndex


def _ids_to_numpy(ids: torch.Tensor) -> np.ndarray:
    return ids.detach().to("cpu", torch.int64).numpy()


class PagePool:
    def __init__(self, num_layers: int, num_pages: int, page_size: int,
                 main_device: torch.device, main_dtype: torch.dtype,
                 n_kv_heads: int = 8, head_dim: int = 128):
        self.num_layers, self.num_pages, self.page_size = num_layers, num_pages, page_size
        self.main_device, self.main_dtype = torch.device(main_device), main_dtype
        self.n_kv_heads, self.head_dim = n_kv_heads, head_dim
        self.mutex = threading.Lock()
        self._index = FreePageIndex(num_pages)
        self.pages = torch.empty((num_layers, num_pages, 2, page_size, n_kv_heads, head_dim),
                                 device=self.main_device, dtype=main_dtype)

    # ---- reference attribute names, backed by the host index
    @property
    def num_avails(self) -> int:
        return self._index.avail

    @num_avails.setter
    def num_avails(self, v: int) -> None:
        self._index.avail = int(v)

    @property
    def fetch_size(self) -> int:
        return self._index.min_fetch

    @fetch_size.setter
    def fetch_size(self, v: int) -> None:
        self._index.min_fetch = int(v)

    @property
    def page_bitmap(self) -> torch.Tensor:
        return torch.from_numpy(self._index.free)        # shares memory

    @property
    def page_buffer(self) -> torch.Tensor:
        return torch.from_numpy(self._index.queue)

    # ---- geometry handed to the native calls
    @property
    def page_bytes(self) -> int:
        return self.pages.stride(1) * self.pages.element_size()

    @property
    def layer_stride_bytes(self) -> int:
        return self.pages.stride(0) * self.pages.element_size()

    def calc_num_pages(self, size: int) -> int:
        return -(-size // self.page_size)

    def alloc(self, size: int) -> Optional[torch.Tensor]:
        """int32 page ids (host tensor); ValueError when the pool is short."""
        with self.mutex:
            return torch.from_numpy(self._index.take(size))

    def alloc_consecutive(self, size: int) -> Optional[torch.Tensor]:
        """Indices of the first run of >= size free pages (the whole run, as
        page_pool.py:57-71 returns it; the reference never calls it)."""
        with self.mutex:
            if size > self._index.avail:
                return None
            a, b = self._index.first_run(size)
            if a < 0:
                return None
            self._index.avail -= size
            return torch.arange(a, b, dtype=torch.int64)

    def free(self, blocks: torch.Tensor) -> None:
        with self.mutex:
            self._index.give(_ids_to_numpy(blocks))

    def retrieve(self, indices: torch.Tensor) -> torch.Tensor:
        """Copy of pages[:, indices] -> (L, n, 2, P, Hkv, D) (page_pool.py:78-79)."""
        from deserve_amd.kvcache import _native

        return _native.gather_pages(self, indices)

    def get_layered_pages(self, layer: int) -> torch.Tensor:
        return self.pages[layer]


class GpuPagePool(PagePool):
    pass


class CpuPagePool(PagePool):
    """Host-memory pool (page_pool.py:97-107): storage only, the HIP kernels
    do not run on it."""

    def __init__(self, num_layers: int, num_pages: int, page_size: int,
                 main_dtype: torch.dtype, n_kv_heads: int = 8, head_dim: int = 128):
        super().__init__(num_layers, num_pages, page_size, torch.device("cpu"), main_dtype,
                         n_kv_heads, head_dim)

    def retrieve(self, indices: torch.Tensor) -> torch.Tensor:
        return self.pages[:, indices.to(torch.int64)]

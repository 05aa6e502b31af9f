"""Tensor-level entry into the C ABI for page movement (gather / scatter / swap).

Everything here takes torch tensors for device memory and streams and passes
raw pointers and sizes to libdskv.so; no copy is done by torch.
"""
from __future__ import annotations

from typing import Optional

import torch

from deserve_amd import _lib


def _device_ids(ids: torch.Tensor, device: torch.device) -> torch.Tensor:
    return ids.to(device=device, dtype=torch.int32, non_blocking=True).contiguous()


def check_page_ids(pool, ids: torch.Tensor, what: str) -> None:
    """The gather / scatter kernels index the pool by these ids: ids outside [0, num_pages)
    are refused here, on a host copy (read back, which synchronises, if ids live on the GPU)."""
    if ids.numel() == 0:
        return
    host = ids.detach().cpu()
    lo, hi = int(host.min()), int(host.max())
    if lo < 0 or hi >= pool.num_pages:
        raise ValueError(f"{what}: page ids span [{lo}, {hi}], the pool has pages [0, {pool.num_pages})")


def gather_pages(pool, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """pages[:, ids] -> (L, n, 2, P, Hkv, D) contiguous, on the pool's device."""
    n = int(ids.shape[0])
    L = pool.num_layers
    if out is None:
        out = torch.empty((L, n) + tuple(pool.pages.shape[2:]), dtype=pool.pages.dtype,
                          device=pool.pages.device)
    if n == 0:
        return out
    check_page_ids(pool, ids, "gather_pages")
    dev_ids = _device_ids(ids, pool.pages.device)
    rc = _lib.lib().dskv_gather_pages(out.data_ptr(), pool.pages.data_ptr(), dev_ids.data_ptr(), n,
                                      L, pool.layer_stride_bytes, pool.page_bytes, 0, L * n,
                                      _lib.current_stream())
    _lib.check(rc, "gather_pages")
    return out


def scatter_pages(pool, ids: torch.Tensor, chunk: torch.Tensor) -> None:
    """pages[:, ids] = chunk viewed (L, n, ...); chunk on the pool's device, contiguous."""
    n = int(ids.shape[0])
    if n == 0:
        return
    L = pool.num_layers
    if not chunk.is_contiguous() or chunk.numel() < L * n * (pool.page_bytes // chunk.element_size()):
        raise ValueError(f"scatter_pages: chunk must be contiguous and hold {L} x {n} pages")
    check_page_ids(pool, ids, "scatter_pages")
    dev_ids = _device_ids(ids, pool.pages.device)
    rc = _lib.lib().dskv_scatter_pages(pool.pages.data_ptr(), chunk.data_ptr(), dev_ids.data_ptr(),
                                       n, L, pool.layer_stride_bytes, pool.page_bytes, 0, L * n,
                                       _lib.current_stream())
    _lib.check(rc, "scatter_pages")


class SwapEngine:
    """Owner of one dskv_swap handle (two side streams + staging buffers).

    The engine's streams must not share a hardware queue with the stream that computes, or
    nothing overlaps; which streams share is an accident of how many streams the process
    has created.  So the engine checks its streams against the current torch stream when
    it is created (``bind``; half a millisecond per check) and replaces one that
    serialises.  ``independent`` tells whether a pair that runs beside compute was found."""

    def __init__(self, staging_bytes: int = 128 << 20, bind: bool = True) -> None:
        import ctypes

        h = ctypes.c_void_p()
        _lib.check(_lib.lib().dskv_swap_create(ctypes.byref(h), staging_bytes), "swap_create")
        self._h = h
        self.staging_bytes = staging_bytes
        self.independent: Optional[bool] = None
        if bind:
            self.bind()

    def bind(self, compute_stream: Optional[int] = None) -> bool:
        """Blocking set-up: make the engine's streams run beside ``compute_stream`` (raw
        handle; default: the current torch stream) and beside each other."""
        import ctypes

        ok = ctypes.c_int32(0)
        stream = _lib.current_stream() if compute_stream is None else compute_stream
        _lib.check(_lib.lib().dskv_swap_bind_compute_stream(self._h, stream, ctypes.byref(ok)),
                   "swap_bind_compute_stream")
        self.independent = bool(ok.value)
        return self.independent

    def streams(self) -> tuple:
        """Raw handles (out, in) of the engine's two streams."""
        import ctypes

        a, b = ctypes.c_void_p(), ctypes.c_void_p()
        _lib.check(_lib.lib().dskv_swap_streams(self._h, ctypes.byref(a), ctypes.byref(b)), "swap_streams")
        return a.value, b.value

    def close(self) -> None:
        if self._h:
            _lib.lib().dskv_swap_destroy(self._h)
            self._h = None

    def __del__(self) -> None:  # best effort
        try:
            self.close()
        except Exception:
            pass

    @staticmethod
    def _host_ids(ids: torch.Tensor) -> torch.Tensor:
        return ids.detach().to("cpu", torch.int32).contiguous()

    def swap_out(self, host_dst: torch.Tensor, pool, ids: torch.Tensor) -> None:
        hid = self._host_ids(ids)
        rc = _lib.lib().dskv_swap_out_async(self._h, host_dst.data_ptr(), pool.pages.data_ptr(),
                                            hid.data_ptr(), hid.shape[0], pool.num_layers,
                                            pool.layer_stride_bytes, pool.page_bytes,
                                            _lib.current_stream())
        _lib.check(rc, "swap_out")

    def swap_in(self, pool, host_src: torch.Tensor, ids: torch.Tensor) -> None:
        hid = self._host_ids(ids)
        rc = _lib.lib().dskv_swap_in_async(self._h, pool.pages.data_ptr(), host_src.data_ptr(),
                                           hid.data_ptr(), hid.shape[0], pool.num_layers,
                                           pool.layer_stride_bytes, pool.page_bytes,
                                           _lib.current_stream())
        _lib.check(rc, "swap_in")

    def exchange(self, host_dst: torch.Tensor, host_src: torch.Tensor, pool, ids: torch.Tensor) -> None:
        hid = self._host_ids(ids)
        rc = _lib.lib().dskv_swap_exchange_async(self._h, host_dst.data_ptr(), host_src.data_ptr(),
                                                 pool.pages.data_ptr(), hid.data_ptr(),
                                                 hid.shape[0], pool.num_layers,
                                                 pool.layer_stride_bytes, pool.page_bytes,
                                                 _lib.current_stream())
        _lib.check(rc, "swap_exchange")

    def wait(self) -> None:
        _lib.check(_lib.lib().dskv_swap_wait(self._h), "swap_wait")

    def done(self) -> bool:
        """Whether everything enqueued so far has finished (does not block)."""
        import ctypes

        flag = ctypes.c_int32(0)
        _lib.check(_lib.lib().dskv_swap_query(self._h, ctypes.byref(flag)), "swap_query")
        return bool(flag.value)

    def fence(self) -> None:
        """Make the current torch stream wait for everything enqueued so far."""
        _lib.check(_lib.lib().dskv_swap_fence(self._h, _lib.current_stream()), "swap_fence")


def swap_slice(pool, page_begin: int, page_end: int, host_to: Optional[torch.Tensor],
               host_from: Optional[torch.Tensor], stream0: int, stream1: int) -> None:
    """Bulk dump-then-refill of pages [page_begin, page_end) of every layer."""
    n = page_end - page_begin
    slice_bytes = n * pool.page_bytes
    base = pool.pages.data_ptr() + page_begin * pool.page_bytes
    need = pool.num_layers * slice_bytes
    for name, t in (("to_memory", host_to), ("from_memory", host_from)):
        if t is not None and t.numel() * t.element_size() != need:
            raise RuntimeError(
                f"swap: {name} holds {t.numel() * t.element_size()} bytes, the slice needs {need}")
    rc = _lib.lib().dskv_swap_slice(base, pool.layer_stride_bytes, slice_bytes, pool.num_layers,
                                    _lib.ptr(host_to), _lib.ptr(host_from), stream0, stream1)
    _lib.check(rc, "swap_slice")

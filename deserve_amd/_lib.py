"""ctypes binding of libdskv.so, the C ABI declared in include/dskv.h.

The library is the only compute path: if it is missing, loading raises and
every operator of this package fails loudly - there is no fallback.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import POINTER, c_char_p, c_float, c_int32, c_int64, c_void_p
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdskv.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

F32, F16, BF16 = 0, 1, 2
ROUTE_OFF, ROUTE_AUTO, ROUTE_TWO_LAUNCHES, ROUTE_SHARED_LAUNCH = 0, 1, 2, 3
LAYOUT_SEPARATE, LAYOUT_SHARED = 0, 1
ABI_VERSION = 3          # DSKV_ABI_VERSION of the include/dskv.h these signatures were written against


class MixedPlanInfo(ctypes.Structure):
    """dskv_mixed_plan_t of include/dskv.h."""
    _fields_ = [("n_tiles", c_int32), ("n_splits", c_int32), ("n_tile_rows", c_int32),
                ("n_decode_rows", c_int32), ("n_decode_items", c_int32), ("n_decode_workgroups", c_int32),
                ("layout", c_int32), ("reserved", c_int32), ("plan_words", c_int64), ("decode_plan_at", c_int64), ("row_map_at", c_int64),
                ("tile_workspace_bytes", c_int64),
                ("decode_workspace_bytes", c_int64)]


_lib: Optional[ctypes.CDLL] = None

# name -> (restype, argtypes); mirrors include/dskv.h one to one
_SIGNATURES = {
    "dskv_last_error": (c_char_p, []),
    "dskv_version": (c_int32, []),
    "dskv_append_paged_kv": (c_int32, [c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
                                       c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32,
                                       c_int32, c_int32, c_void_p]),
    "dskv_gather_pages": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int64,
                                    c_int64, c_int64, c_int64, c_void_p]),
    "dskv_scatter_pages": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int64,
                                     c_int64, c_int64, c_int64, c_void_p]),
    "dskv_decode_plan_bound": (c_int64, [c_int32, c_int64]),
    "dskv_decode_plan": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32,
                                   c_int32, c_void_p, c_int64, POINTER(c_int32), POINTER(c_int32),
                                   POINTER(c_int64), POINTER(c_int64)]),
    "dskv_decode_attn": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
                                   c_int32, c_void_p, c_int64, c_int32, c_int32, c_int32, c_int32,
                                   c_int32, c_float, c_int32, c_void_p]),
    "dskv_decode_attn_noalloc_max_bytes": (c_int64, []),
    "dskv_decode_attn_noalloc": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int32,
                                           c_int32, c_int32, c_int32, c_int32, c_int32, c_int32,
                                           c_float, c_int32, c_void_p]),
    "dskv_decode_attn_phases": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_int32, c_int32, c_void_p, c_int64, c_int32, c_int32,
                                          c_int32, c_int32, c_int32, c_float, c_int32, c_int32,
                                          c_void_p]),
    "dskv_decode_append_attn_supported": (c_int32, [c_int32, c_int32, c_int32, c_int32, c_int32]),
    "dskv_decode_append_attn": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int32, c_int32, c_void_p, c_int64, c_int32,
                                          c_int32, c_int32, c_int32, c_int32, c_float, c_int32,
                                          c_int32, c_void_p]),
    "dskv_rope_table": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_float, c_void_p]),
    "dskv_decode_rope_append_attn": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                               c_void_p, c_void_p, c_int32, c_int32, c_void_p,
                                               c_int64, c_int32, c_int32, c_int32, c_int32, c_int32,
                                               c_float, c_int32, c_void_p, c_int32, c_void_p]),
    "dskv_prefill_plan_bound": (c_int64, [c_int32, c_int64]),
    "dskv_prefill_plan": (c_int32, [c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32, c_int32,
                                    c_void_p, c_int64, POINTER(c_int32), POINTER(c_int32),
                                    POINTER(c_int64), POINTER(c_int64)]),
    "dskv_prefill_attn": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_void_p, c_int32, c_int32, c_void_p, c_int64, c_int32,
                                    c_int32, c_int32, c_int32, c_int32, c_int32, c_float, c_int32,
                                    c_int32, c_void_p]),
    "dskv_mixed_plan_bound": (c_int64, [c_int32, c_int64, c_int64]),
    "dskv_mixed_plan": (c_int32, [c_void_p, c_void_p, c_void_p, c_int32, c_int32, c_int32, c_int32,
                                  c_int32, c_int32, c_int32, c_void_p, c_int64, POINTER(MixedPlanInfo)]),
    "dskv_mixed_attn": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p, c_void_p, POINTER(MixedPlanInfo), c_void_p, c_int64,
                                  c_int32, c_int32, c_int32, c_int32, c_int32, c_int32, c_float,
                                  c_int32, c_int32, c_void_p]),
    "dskv_apply_rope": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_int32, c_int32, c_int32, c_int32, c_int32, c_float, c_int32,
                                  c_void_p]),
    "dskv_rope_append_paged_kv": (c_int32, [c_void_p, c_void_p, c_int32] + [c_void_p] * 8 +
                                  [c_int32] * 6 + [c_float, c_int32, c_void_p]),
    "dskv_upload_words": (c_int32, [c_void_p, c_void_p, c_int64, c_void_p]),
    "dskv_swap_slice": (c_int32, [c_void_p, c_int64, c_int64, c_int32, c_void_p, c_void_p,
                                  c_void_p, c_void_p]),
    "dskv_swap_create": (c_int32, [POINTER(c_void_p), c_int64]),
    "dskv_swap_destroy": (c_int32, [c_void_p]),
    "dskv_swap_out_async": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                      c_int64, c_int64, c_void_p]),
    "dskv_swap_in_async": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_int32, c_int32,
                                     c_int64, c_int64, c_void_p]),
    "dskv_swap_exchange_async": (c_int32, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                           c_int32, c_int32, c_int64, c_int64, c_void_p]),
    "dskv_swap_wait": (c_int32, [c_void_p]),
    "dskv_swap_fence": (c_int32, [c_void_p, c_void_p]),
    "dskv_swap_query": (c_int32, [c_void_p, POINTER(c_int32)]),
    "dskv_swap_streams": (c_int32, [c_void_p, POINTER(c_void_p), POINTER(c_void_p)]),
    "dskv_swap_bind_compute_stream": (c_int32, [c_void_p, c_void_p, POINTER(c_int32)]),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)


def build(force: bool = True) -> str:
    """Compile csrc/ for gfx950 into libdskv.so (hipcc cross-compiles without a GPU)."""
    cmd = ["make", "-C", CSRC_DIR, "-j8", f"OUT={LIB_PATH}"]
    if force:
        cmd.insert(1, "-B")
    subprocess.check_call(cmd)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension is not built "
                "(run `python -c 'import __graft_entry__ as g; g.build()'`); "
                "deserve_amd has no other compute path")
        handle = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        if handle.dskv_version() != ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI version {handle.dskv_version()}, this binding was written "
                               f"against {ABI_VERSION}: rebuild the library (its argument lists differ)")
        _lib = handle
    return _lib


def last_error() -> str:
    msg = lib().dskv_last_error()
    return msg.decode() if msg else ""


E_INVAL, E_NOMEM, E_STATE = -1, -2, -3


def check(rc: int, what: str = "dskv") -> None:
    """0 ok; argument errors (DSKV_E_INVAL, DSKV_E_NOMEM) -> ValueError; a handle used in
    the wrong state (DSKV_E_STATE) and HIP errors (positive) -> RuntimeError."""
    if rc == 0:
        return
    msg = f"{what}: {last_error()} (code {rc})"
    if rc in (E_INVAL, E_NOMEM):
        raise ValueError(msg)
    raise RuntimeError(msg)


def dtype_code(dtype) -> int:
    import torch

    try:
        return {torch.float32: F32, torch.float16: F16, torch.bfloat16: BF16}[dtype]
    except KeyError:
        raise ValueError(f"unsupported KV dtype {dtype}") from None


def ptr(t) -> int:
    """Raw address of a tensor's first element (0 for None)."""
    return 0 if t is None else t.data_ptr()


def current_stream() -> int:
    import torch

    return torch.cuda.current_stream().cuda_stream

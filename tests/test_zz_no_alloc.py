"""dskv_decode_attn_noalloc (the entry point that allocates nothing: partials in an array
built into the library) against dskv_decode_attn with a caller workspace, through the C
ABI: the same bits, on two calls in a row of which the second is smaller, so what the first
call left in the shared array must not leak into the second."""
import ctypes
import math

import numpy as np
import pytest
import torch

from kvutil import make_scenario, max_rel_err_per_request, to_torch
from oracle import c_oracle



def _plan(lib, sc, target):
    batch = len(sc.kv_lens)
    indptr = np.ascontiguousarray(sc.kv_page_indptr, np.int32)
    last = np.ascontiguousarray(sc.kv_last_page_lens, np.int32)
    cap = lib.dskv_decode_plan_bound(batch, int(indptr[-1]) * sc.P)
    plan = np.zeros(cap, np.int32)
    n_items, n_wgs, words, ws = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64(), ctypes.c_int64()
    rc = lib.dskv_decode_plan(indptr.ctypes.data, last.ctypes.data, batch, sc.P, sc.Hq, sc.Hkv, sc.D, target,
                              plan.ctypes.data, cap, ctypes.byref(n_items), ctypes.byref(n_wgs),
                              ctypes.byref(words), ctypes.byref(ws))
    assert rc == 0
    return torch.from_numpy(plan[: words.value]).cuda(), n_items.value, n_wgs.value, ws.value


def _both(lib, sc, target):
    """(with a workspace, with the built-in array): outputs of the two entry points."""
    from deserve_amd import _lib

    batch = len(sc.kv_lens)
    plan, n_items, n_wgs, ws_bytes = _plan(lib, sc, target)
    q, pages = to_torch(sc.q, sc.dtype), to_torch(sc.pages, sc.dtype)
    ids = torch.from_numpy(np.ascontiguousarray(sc.kv_page_indices, np.int32)).cuda()
    ws = torch.empty(max(ws_bytes, 16), dtype=torch.uint8, device="cuda")
    out_a = torch.full_like(q, float("nan"))
    out_b = torch.full_like(q, float("nan"))
    stream = torch.cuda.current_stream().cuda_stream
    scale = 1.0 / math.sqrt(sc.D)
    code = _lib.dtype_code(q.dtype)
    rc = lib.dskv_decode_attn(out_a.data_ptr(), q.data_ptr(), pages.data_ptr(), ids.data_ptr(), plan.data_ptr(),
                              n_items, n_wgs, ws.data_ptr(), ws_bytes, batch, sc.Hq, sc.Hkv, sc.D, sc.P, scale,
                              code, stream)
    _lib.check(rc, "decode_attn")
    rc = lib.dskv_decode_attn_noalloc(out_b.data_ptr(), q.data_ptr(), pages.data_ptr(), ids.data_ptr(),
                                      plan.data_ptr(), n_items, n_wgs, batch, sc.Hq, sc.Hkv, sc.D, sc.P, scale,
                                      code, stream)
    _lib.check(rc, "decode_attn_noalloc")
    torch.cuda.synchronize()
    return out_a, out_b, n_items


@pytest.mark.gpu
def test_noalloc_decode_equals_workspace_decode_on_two_calls_in_a_row():
    from deserve_amd import _lib

    lib = _lib.lib()
    assert lib.dskv_decode_attn_noalloc_max_bytes() == 32 << 20
    calls = [
        # the first call fills many slots of the shared array, the second, smaller one reuses few
        ("large", dict(kv_lens=[4096, 700, 257, 3000, 16, 5000, 1, 2222], Hq=64, dtype="bf16"), 0),
        ("small", dict(kv_lens=[900, 40, 333], Hq=32, dtype="bf16"), 6),
        ("fp32 generic path", dict(kv_lens=[300, 17], Hq=8, Hkv=2, D=64, dtype="f32"), 5),
    ]
    for seed, (name, kw, target) in enumerate(calls):
        print("[case] noalloc decode", name, flush=True)
        lens = kw.pop("kv_lens")
        sc = make_scenario(700 + seed, kv_lens=lens, qo_lens=[1] * len(lens), **kw)
        out_a, out_b, n_items = _both(lib, sc, target)
        assert n_items > len(lens), "the case was meant to cut requests (partials in the scratch array)"
        view = torch.int32 if sc.dtype == "f32" else torch.int16
        assert torch.equal(out_a.view(view), out_b.view(view)), name
        want = c_oracle.decode_attn(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                    sc.kv_last_page_lens, sc.dtype)
        tol = 1e-4 if sc.dtype == "f32" else 2e-2
        assert max_rel_err_per_request(out_b.float().cpu().numpy(), want) <= tol, name


def test_noalloc_decode_refuses_plans_beyond_the_built_in_scratch():
    from deserve_amd import _lib

    lib = _lib.lib()
    # 4000 items of 8 requests: 4000 slots x 64 heads x 130 floats = 133 MB > 32 MiB
    rc = lib.dskv_decode_attn_noalloc(16, 16, 16, 16, 16, 4000, 256, 8, 64, 8, 128, 16, 0.1, 2, None)
    assert rc == -2 and "built-in scratch" in _lib.last_error()
    with pytest.raises(ValueError, match="built-in scratch"):
        _lib.check(rc, "decode_attn_noalloc")
    assert lib.dskv_decode_attn_noalloc(None, None, None, None, None, 0, 0, 0, 32, 8, 128, 16, 0.1, 2, None) == 0

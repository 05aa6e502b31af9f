"""ctypes loader for oracle/libkv_oracle.so (test infrastructure only).

Thin wrappers that take numpy arrays; see kv_oracle.c for what each function
restates.  Used by tests as an independent cross-check of kv_oracle.py and by
the bench as the timed CPU baseline (OpenMP over request x head).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libkv_oracle.so")
ELT = {"f32": 0, "f16": 1, "bf16": 2}


def build() -> None:
    subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "libkv_oracle.so"])


def load() -> ctypes.CDLL:
    if not os.path.exists(_SO):
        build()
    lib = ctypes.CDLL(_SO)
    return lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    assert a.flags["C_CONTIGUOUS"]
    return ctypes.c_void_p(a.ctypes.data)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.int32)


def append(pages_layer, k, v, indptr, kv_indices, kv_indptr, last, dtype: str) -> None:
    lib = load()
    P, Hkv, D = pages_layer.shape[2:5]
    indptr, kv_indices, kv_indptr, last = map(_i32, (indptr, kv_indices, kv_indptr, last))
    lib.orc_append(_p(pages_layer), _p(k), _p(v), _p(indptr), _p(kv_indices), _p(kv_indptr),
                   _p(last), len(indptr) - 1, int(P), int(Hkv), int(D), ELT[dtype])


def gather(pool: np.ndarray, ids) -> np.ndarray:
    lib = load()
    L, n = pool.shape[0], len(ids)
    ids = _i32(ids)
    page_bytes = int(np.prod(pool.shape[2:])) * pool.itemsize
    out = np.empty((L * n,) + pool.shape[2:], dtype=pool.dtype)
    lib.orc_gather(_p(out), _p(pool), _p(ids), n, L,
                   ctypes.c_int64(pool.strides[0]), ctypes.c_int64(page_bytes))
    return out


def scatter(pool: np.ndarray, ids, chunk: np.ndarray) -> None:
    lib = load()
    L, n = pool.shape[0], len(ids)
    ids = _i32(ids)
    page_bytes = int(np.prod(pool.shape[2:])) * pool.itemsize
    lib.orc_scatter(_p(pool), _p(chunk), _p(ids), n, L,
                    ctypes.c_int64(pool.strides[0]), ctypes.c_int64(page_bytes))


def decode_attn(q, pages_layer, kv_indices, kv_indptr, last, dtype: str, scale=None) -> np.ndarray:
    lib = load()
    B, Hq, D = q.shape
    P, Hkv = pages_layer.shape[2], pages_layer.shape[3]
    kv_indices, kv_indptr, last = map(_i32, (kv_indices, kv_indptr, last))
    out = np.zeros((B, Hq, D), dtype=np.float32)
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    lib.orc_decode_attn(_p(out), _p(q), _p(pages_layer), _p(kv_indices), _p(kv_indptr), _p(last),
                        B, Hq, int(Hkv), D, int(P), ELT[dtype], ctypes.c_float(scale))
    return out


def prefill_attn(q, qo_indptr, pages_layer, kv_indices, kv_indptr, last, dtype: str,
                 causal: bool = True, scale=None) -> np.ndarray:
    lib = load()
    nnz, Hq, D = q.shape
    P, Hkv = pages_layer.shape[2], pages_layer.shape[3]
    qo_indptr, kv_indices, kv_indptr, last = map(_i32, (qo_indptr, kv_indices, kv_indptr, last))
    out = np.zeros((nnz, Hq, D), dtype=np.float32)
    scale = 1.0 / np.sqrt(D) if scale is None else scale
    lib.orc_prefill_attn(_p(out), _p(q), _p(qo_indptr), _p(pages_layer), _p(kv_indices),
                         _p(kv_indptr), _p(last), len(qo_indptr) - 1, Hq, int(Hkv), D, int(P),
                         ELT[dtype], ctypes.c_float(scale), int(causal))
    return out

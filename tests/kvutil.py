"""Shared builders for the parity tests: seeded paged-KV scenarios in numpy."""
from __future__ import annotations

import os
import sys
from dataclasses import dataclass
from typing import Sequence

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

from oracle import kv_oracle as orc  # noqa: E402

NP_DTYPE = {"f32": np.float32, "f16": np.float16, "bf16": np.uint16}


def to_storage(x: np.ndarray, dtype: str) -> np.ndarray:
    """fp32 values -> storage array of the given element type (bf16 as uint16 bits)."""
    if dtype == "f32":
        return np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "f16":
        return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16)
    return orc.bf16_bits_from_f32(x)


@dataclass
class Scenario:
    P: int
    Hq: int
    Hkv: int
    D: int
    num_pages: int
    kv_lens: np.ndarray           # tokens per request AFTER the append
    qo_lens: np.ndarray           # new tokens per request
    kv_page_indices: np.ndarray
    kv_page_indptr: np.ndarray
    kv_last_page_lens: np.ndarray
    qo_indptr: np.ndarray
    pages: np.ndarray             # (num_pages, 2, P, Hkv, D) storage dtype
    q: np.ndarray                 # (nnz, Hq, D)
    k: np.ndarray                 # (nnz, Hkv, D)
    v: np.ndarray
    dtype: str


def make_scenario(seed: int, kv_lens: Sequence[int], qo_lens: Sequence[int], P: int = 16,
                  Hq: int = 32, Hkv: int = 8, D: int = 128, dtype: str = "bf16",
                  spare_pages: int = 7, fill: str = "normal") -> Scenario:
    """Random pool where request b owns ceil(kv_len_b / P) pages drawn from a
    seeded permutation of the pool; K, V, Q ~ N(0, 1)."""
    rng = np.random.default_rng(seed)
    kv_lens = np.asarray(kv_lens, dtype=np.int64)
    qo_lens = np.asarray(qo_lens, dtype=np.int64)
    npages = -(-kv_lens // P)
    total = int(npages.sum())
    num_pages = total + spare_pages
    perm = rng.permutation(num_pages).astype(np.int32)
    indptr = np.concatenate([[0], np.cumsum(npages)]).astype(np.int32)
    last = np.where(kv_lens > 0, (kv_lens - 1) % P + 1, 0).astype(np.int32)
    if fill == "normal":
        pages_f = rng.standard_normal((num_pages, 2, P, Hkv, D), dtype=np.float32)
    else:
        pages_f = np.full((num_pages, 2, P, Hkv, D), np.float32(fill), dtype=np.float32)
    nnz = int(qo_lens.sum())
    return Scenario(
        P=P, Hq=Hq, Hkv=Hkv, D=D, num_pages=num_pages, kv_lens=kv_lens, qo_lens=qo_lens,
        kv_page_indices=perm[:total].copy(), kv_page_indptr=indptr, kv_last_page_lens=last,
        qo_indptr=np.concatenate([[0], np.cumsum(qo_lens)]).astype(np.int32),
        pages=to_storage(pages_f, dtype),
        q=to_storage(rng.standard_normal((nnz, Hq, D), dtype=np.float32), dtype),
        k=to_storage(rng.standard_normal((nnz, Hkv, D), dtype=np.float32), dtype),
        v=to_storage(rng.standard_normal((nnz, Hkv, D), dtype=np.float32), dtype),
        dtype=dtype)


def max_rel_err(got: np.ndarray, ref: np.ndarray) -> float:
    """max |got - ref| / max |ref|: the error relative to the output's scale."""
    return float(np.abs(got.astype(np.float64) - ref.astype(np.float64)).max() /
                 max(float(np.abs(ref).max()), 1e-30))


def max_rel_err_per_request(got: np.ndarray, ref: np.ndarray, row_indptr=None) -> float:
    """The largest max_rel_err over requests, each request measured against the scale of
    its OWN output: a long request's output is a mean over thousands of values and far
    smaller than a short one's, so a scale taken over the whole batch would let any error
    in it pass.  row_indptr: CSR bounds of every request's block of rows along axis 0
    (prefill); None = one row per request (decode).  Requests without rows are skipped."""
    if row_indptr is None:
        row_indptr = np.arange(got.shape[0] + 1)
    worst = 0.0
    for b in range(len(row_indptr) - 1):
        lo, hi = int(row_indptr[b]), int(row_indptr[b + 1])
        if hi > lo:
            worst = max(worst, max_rel_err(got[lo:hi], ref[lo:hi]))
    return worst


# ---- torch <-> storage helpers (GPU tests only)
def torch_dtype(dtype: str):
    import torch

    return {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]


def to_torch(x: np.ndarray, dtype: str, device="cuda"):
    import torch

    t = torch.from_numpy(np.ascontiguousarray(x))
    if dtype == "bf16":
        t = t.view(torch.int16).view(torch.bfloat16)
    return t.to(device)


def from_torch(t, dtype: str) -> np.ndarray:
    import torch

    t = t.detach().cpu().contiguous()
    if dtype == "bf16":
        return t.view(torch.int16).numpy().view(np.uint16)
    return t.numpy()

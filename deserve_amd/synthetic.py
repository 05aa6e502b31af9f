"""Seeded synthetic workloads at the shapes of the baseline configurations,
built directly on the GPU (bench and full-size tests share them).

A workload owns a page pool whose pages are handed to the requests in a seeded
random permutation (so block tables are scattered over the whole pool), request
records at the given context lengths, and per-layer q/k/v inputs ~ N(0, 1).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import List, Sequence

import numpy as np
import torch

from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.kvcache.paged.page_pool import GpuPagePool, PagePool
from deserve_amd.kvcache.paged.page_table import PageTableAllocator
from deserve_amd.stage import KVStage, StageArgs
from deserve_amd.task import SamplingParams, TaskData


@dataclass
class DecodeWorkload:
    name: str
    args: StageArgs
    pool: PagePool
    tables: PageTableAllocator
    tasks: List[TaskData]
    caches: List[PagedKVCache]
    stage: KVStage
    q: torch.Tensor     # (L, B, Hq, D)
    k: torch.Tensor     # (L, B, Hkv, D)
    v: torch.Tensor
    ctx_lens: np.ndarray

    @property
    def batch(self) -> int:
        return len(self.tasks)

    def kv_bytes_per_token(self) -> int:
        n_kv = self.args.n_kv_heads or self.args.n_heads
        return 2 * n_kv * (self.args.dim // self.args.n_heads) * self.pool.pages.element_size()


def scatter_pool_order(pool: PagePool, seed: int) -> None:
    """Make the allocator hand pages out in a seeded random order instead of
    lowest-first: the prefetch queue is preloaded with a permutation of every
    free page (the bitmap is drained accordingly)."""
    rng = np.random.default_rng(seed)
    idx = pool._index
    free = np.flatnonzero(idx.free).astype(np.int32)
    idx.free[free] = False
    idx.queue = np.concatenate([idx.queue, rng.permutation(free).astype(np.int32)])


def fill_normal(t: torch.Tensor, seed: int, chunk_elems: int = 1 << 28) -> None:
    """In-place N(0, 1) fill of a large tensor, chunked to bound temporary memory."""
    g = torch.Generator(device=t.device)
    g.manual_seed(seed)
    flat = t.view(-1)
    for start in range(0, flat.numel(), chunk_elems):
        part = flat[start: start + chunk_elems]
        part.copy_(torch.randn(part.numel(), generator=g, device=t.device, dtype=torch.float32))


def make_decode_workload(name: str, ctx_lens: Sequence[int], n_layers: int, n_heads: int,
                         n_kv_heads: int = 8, head_dim: int = 128, page_size: int = 16,
                         dtype: torch.dtype = torch.bfloat16, headroom_tokens: int = 64,
                         seed: int = 0, device: str = "cuda", use_rope: bool = False,
                         spare_pages: int = 64, fill: bool = True) -> DecodeWorkload:
    """Requests already hold ctx_lens[b] tokens; every step appends one more."""
    dev = torch.device(device)
    ctx = np.asarray(ctx_lens, dtype=np.int64)
    need = int((-(-(ctx + headroom_tokens) // page_size)).sum()) + spare_pages
    args = StageArgs(n_heads=n_heads, n_kv_heads=n_kv_heads, dim=n_heads * head_dim,
                     page_size=page_size, n_layers=n_layers)
    pool = GpuPagePool(n_layers, need, page_size, dev, dtype, n_kv_heads, head_dim)
    if fill:
        fill_normal(pool.pages, seed + 1)
    scatter_pool_order(pool, seed + 2)
    max_ctx = int(-(-(ctx.max() + headroom_tokens) // page_size) * page_size)
    tables = PageTableAllocator(len(ctx), max_ctx, page_size, dev)
    tasks, caches = [], []
    for b, n in enumerate(ctx):
        t = TaskData(task_id=f"{name}-{b}", start_pos=int(n), round=1, seqlen=1,
                     initial_seqlen=int(n), sampling_params=SamplingParams())
        c = PagedKVCache.empty(tables, pool)
        c.extend(int(n))
        tasks.append(t)
        caches.append(c)
    g = torch.Generator(device=dev)
    g.manual_seed(seed + 3)
    B = len(ctx)
    mk = lambda h: torch.randn((n_layers, B, h, head_dim), generator=g, device=dev,
                               dtype=torch.float32).to(dtype)
    return DecodeWorkload(name, args, pool, tables, tasks, caches, KVStage(args, use_rope=use_rope),
                          mk(n_heads), mk(n_kv_heads), mk(n_kv_heads), ctx)


def config2_context_lengths(seed: int = 2, batch: int = 64, lo: int = 256, hi: int = 4096) -> np.ndarray:
    """Baseline configuration 2: context lengths seeded uniform in [lo, hi]."""
    return np.random.default_rng(seed).integers(lo, hi + 1, size=batch)


def config5_context_lengths(seed: int = 5, batch: int = 128, median: int = 2048, sigma: float = 1.0,
                            lo: int = 64, hi: int = 32768) -> np.ndarray:
    """Baseline configuration 5: lognormal lengths (median 2048, sigma 1.0 chosen
    here since the configuration leaves it open), clipped to [64, 32768]."""
    rng = np.random.default_rng(seed)
    return np.clip(np.exp(rng.normal(np.log(median), sigma, size=batch)), lo, hi).astype(np.int64)

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


@dataclass
class MixedWorkload:
    """A step as the reference's decode-first join stage assembles it
    (deserve_worker/engine/pipeline/stage/join.py:11-88): the running requests, one new
    token each, then chunks of pending prompts up to the step's token budget."""
    name: str
    args: StageArgs
    pool: PagePool
    tables: PageTableAllocator
    tasks: List[TaskData]
    caches: List[PagedKVCache]
    stage: KVStage
    q: torch.Tensor     # (L, nnz, Hq, D): ragged, decode rows first
    k: torch.Tensor     # (L, nnz, Hkv, D)
    v: torch.Tensor
    decode_ctx: np.ndarray     # tokens each decode request holds before the step
    chunk_prior: np.ndarray    # tokens each chunked request holds before the step
    chunk_lens: np.ndarray     # new tokens of each chunk

    @property
    def nnz(self) -> int:
        return int(self.q.shape[1])

    def kv_bytes_per_token(self) -> int:
        n_kv = self.args.n_kv_heads or self.args.n_heads
        return 2 * n_kv * (self.args.dim // self.args.n_heads) * self.pool.pages.element_size()

    def decode_kv_tokens(self) -> int:
        """kv tokens the decode rows attend over (each request's context plus its new token)."""
        return int((self.decode_ctx + 1).sum())

    def chunk_flops(self) -> int:
        """4 * Hq * D * sum over chunks of (n * prior + n (n + 1) / 2)."""
        hq, d = self.args.n_heads, self.args.dim // self.args.n_heads
        return int(4 * hq * d * sum(int(n) * int(p) + int(n) * (int(n) + 1) // 2
                                    for n, p in zip(self.chunk_lens, self.chunk_prior)))


def make_mixed_workload(name: str, decode_ctx: Sequence[int], chunk_prior: Sequence[int],
                        chunk_lens: Sequence[int], n_layers: int, n_heads: int, n_kv_heads: int = 8,
                        head_dim: int = 128, page_size: int = 16, dtype: torch.dtype = torch.bfloat16,
                        seed: int = 0, device: str = "cuda", spare_pages: int = 64) -> MixedWorkload:
    """Decode requests that hold decode_ctx[b] tokens and get one more, followed by chunked
    requests that hold chunk_prior[c] tokens and get chunk_lens[c] more.  Pool pages are
    N(0, 1) and handed out in a seeded permutation; q / k / v of the step's tokens are N(0, 1)."""
    dev = torch.device(device)
    dctx = np.asarray(decode_ctx, dtype=np.int64)
    prior, lens = np.asarray(chunk_prior, dtype=np.int64), np.asarray(chunk_lens, dtype=np.int64)
    after = np.concatenate([dctx + 1, prior + lens])
    need = int((-(-after // page_size)).sum()) + spare_pages
    args = StageArgs(n_heads=n_heads, n_kv_heads=n_kv_heads, dim=n_heads * head_dim,
                     page_size=page_size, n_layers=n_layers)
    pool = GpuPagePool(n_layers, need, page_size, dev, dtype, n_kv_heads, head_dim)
    fill_normal(pool.pages, seed + 1)
    scatter_pool_order(pool, seed + 2)
    max_ctx = int(-(-(after.max() + 1) // page_size) * page_size)
    tables = PageTableAllocator(len(after), max_ctx, page_size, dev)
    tasks, caches = [], []
    for b, n in enumerate(dctx):
        tasks.append(TaskData(f"{name}-d{b}", int(n), 1, 1, int(n), SamplingParams()))
    for c, (p, n) in enumerate(zip(prior, lens)):
        tasks.append(TaskData(f"{name}-c{c}", int(p), 1, int(n), int(p + n), SamplingParams()))
    for t in tasks:
        cache = PagedKVCache.empty(tables, pool)
        cache.extend(t.start_pos)
        caches.append(cache)
    g = torch.Generator(device=dev)
    g.manual_seed(seed + 3)
    nnz = int(len(dctx) + lens.sum())
    mk = lambda h: torch.randn((n_layers, nnz, h, head_dim), generator=g, device=dev,
                               dtype=torch.float32).to(dtype)
    return MixedWorkload(name, args, pool, tables, tasks, caches, KVStage(args, use_rope=False),
                         mk(n_heads), mk(n_kv_heads), mk(n_kv_heads), dctx, prior, lens)


def mixed_step_shape(seed: int, decode_rows: int = 75, token_budget: int = 512, lo: int = 256,
                     hi: int = 4096):
    """The step behind the reference's best published row (deserve_exp/exp_args.csv: microbatch
    size 75; engine/pipeline/scheduler.py:74,85: 512 tokens per step): `decode_rows` running
    requests with contexts seeded uniform in [lo, hi], and one chunk that fills the rest of
    the token budget over a prior seeded uniform in [0, hi].  Returns (decode contexts,
    [prior], [chunk length])."""
    rng = np.random.default_rng(seed)
    return rng.integers(lo, hi + 1, size=decode_rows), [int(rng.integers(0, hi + 1))], [token_budget - decode_rows]

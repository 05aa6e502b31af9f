"""CPU oracle for the KV-cache hot path of one DeServe pipeline stage.

TEST INFRASTRUCTURE ONLY.  This module is the checker that the GPU path is
compared against.  Nothing in the shipped package imports it; only the tests,
the smoke entry and the bench's CPU-baseline leg do.

It is a numpy restatement of the reference's algorithm, written from reading
the reference source as text (paths relative to the reference repository's
``deserve_worker/`` package):

===========================  ==================================================
function / class here        follows
===========================  ==================================================
PagePoolModel                kvcache/paged/page_pool.py:7-82
PageTableModel               kvcache/paged/page_table.py:7-60
PagedCacheModel              kvcache/paged/kvcache.py:12-33
VirtualPoolModel             kvcache/virtual.py:19-116 (bookkeeping + the
                             intended bulk swap of :97-113)
VirtualCacheModel            kvcache/virtual.py:119-161
BuddyModel                   kvcache/paged/chunk_pool.py:10-96
build_ctx                    model/context/flash.py:24-70
append_paged_kv              model/layer/attention.py:174-183 (call site of the
                             absent third-party ``flashinfer`` wheel, unpinned
                             in pyproject.toml:17; its documented v0.1.x
                             semantics are restated here)
gather_pages/scatter_pages   kvcache/manager.py:24-86, page_pool.py:78-79
swap_slice                   kvcache/virtual.py:97-113
decode_attention             model/layer/attention.py:75-84,241-266 (the dense
                             fp32-softmax statement of the maths) applied to
                             the paged layout of attention.py:185
prefill_attention            same maths with the end-aligned causal mask of
                             attention.py:188-192,216-221
rope_interleaved             model/layer/attention.py:45-72 and
                             execution/exec.py:25-55
===========================  ==================================================

Pinning status.  The reference has no tests, golden vectors or fixtures for
this path.  Every allocator model is pinned by the hand-derived known answers
that follow from the reference source (tests/test_allocators.py);
append/gather/scatter/swap are pinned by brute-force scalar loops and library
routines (``numpy.take``); attention is pinned by closed forms (kv_len 1,
constant keys, one dominant key, page-permutation invariance) and by
``scipy.special.softmax`` + ``numpy.einsum``.  What cannot be pinned is the
rounding/merge order inside the absent ``flashinfer`` kernels: attention parity
is therefore tolerance-based by construction (2e-2 max-relative in bf16 against
this fp32 statement) - "parity unpinned" at that third-party boundary.
"""
from __future__ import annotations

import bisect
import math
from dataclasses import dataclass
from typing import List, Optional, Sequence, Tuple

import numpy as np

N_KV_HEADS = 8      # baked into the reference pool shape, page_pool.py:26
HEAD_DIM = 128      # idem


# --------------------------------------------------------------------------
# 16-bit float helpers (numpy has no bfloat16): storage is uint16 bit patterns
# --------------------------------------------------------------------------
def bf16_bits_from_f32(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even fp32 -> bf16 bit pattern (uint16)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    rounded = (u + 0x7FFF + ((u >> 16) & 1)) >> 16
    rounded = np.where(nan, (u >> 16) | 0x40, rounded)
    return rounded.astype(np.uint16)


def f32_from_bf16_bits(b: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_f32(x: np.ndarray, dtype: str) -> np.ndarray:
    """Widen a storage array to fp32.  dtype in {"f32","f16","bf16"}."""
    if dtype == "f32":
        return np.asarray(x, dtype=np.float32)
    if dtype == "f16":
        return np.asarray(x).view(np.float16).astype(np.float32)
    if dtype == "bf16":
        return f32_from_bf16_bits(np.asarray(x).view(np.uint16))
    raise ValueError(dtype)


# --------------------------------------------------------------------------
# Allocator models
# --------------------------------------------------------------------------
class PagePoolModel:
    """Free-page bitmap with a sticky prefetch buffer (page_pool.py:7-76).

    alloc: refuse when the request exceeds ``num_avails``; if the buffer is
    short, move the LOWEST ``max(64, shortfall)`` free ids from the bitmap to
    the tail of the buffer; hand out the head of the buffer.
    free: ids go back to the bitmap, never to the buffer.
    """

    def __init__(self, num_pages: int, fetch_size: int = 64):
        self.num_pages = num_pages
        self.num_avails = num_pages
        self.fetch_size = fetch_size
        self.bitmap = np.ones(num_pages, dtype=bool)
        self.buffer: List[int] = []

    def alloc(self, size: int) -> List[int]:
        if size > self.num_avails:
            raise ValueError(f"Not enough pages {size} > {self.num_avails}")
        self.num_avails -= size
        if size > len(self.buffer):
            want = max(self.fetch_size, size - len(self.buffer))
            got = np.flatnonzero(self.bitmap)[:want]
            self.bitmap[got] = False
            self.buffer.extend(int(i) for i in got)
        out, self.buffer = self.buffer[:size], self.buffer[size:]
        return out

    def alloc_consecutive(self, size: int) -> Optional[List[int]]:
        """First run of >= size free pages; the whole run is returned
        (page_pool.py:57-71 returns every index of the run it found)."""
        if size > self.num_avails:
            return None
        start = None
        runs: List[Tuple[int, int]] = []
        for i, bit in enumerate(list(self.bitmap) + [False]):
            if bit and start is None:
                start = i
            elif not bit and start is not None:
                runs.append((start, i))
                start = None
        for a, b in runs:
            if b - a >= size:
                self.num_avails -= size
                return list(range(a, b))
        return None

    def free(self, ids: Sequence[int]) -> None:
        self.num_avails += len(ids)
        self.bitmap[np.asarray(ids, dtype=np.int64)] = True


class PageTableModel:
    """Block-table rows handed out LIFO (page_table.py:29-60)."""

    def __init__(self, max_requests: int, max_context_len: int, page_size: int):
        self.width = max_context_len // page_size
        self.max_context_len = max_context_len
        self.tables = np.zeros((max_requests, self.width), dtype=np.int32)
        self.slots = list(range(max_requests))

    def alloc(self) -> "TableRow":
        if not self.slots:
            raise ValueError("No available slots")
        return TableRow(self.slots.pop(), 0, self)

    def free(self, row: "TableRow") -> None:
        self.slots.append(row.offset)


@dataclass
class TableRow:
    offset: int
    occupied: int
    owner: PageTableModel

    def ids(self) -> np.ndarray:
        return self.owner.tables[self.offset, : self.occupied]

    def extend(self, fill: Sequence[int]) -> None:
        n = len(fill)
        self.owner.tables[self.offset, self.occupied : self.occupied + n] = fill
        self.occupied += n


class PagedCacheModel:
    """One request's cache: grows by whole pages (kvcache.py:12-33)."""

    def __init__(self, row: TableRow, pool: PagePoolModel, page_size: int):
        self.row, self.pool, self.page_size = row, pool, page_size

    def extend(self, num_tokens: int) -> bool:
        if num_tokens > self.row.occupied * self.page_size:
            need = -(-num_tokens // self.page_size)
            self.row.extend(self.pool.alloc(need - self.row.occupied))
        return True

    def free(self) -> None:
        self.pool.free(list(self.row.ids()))
        self.row.owner.free(self.row)


class VirtualPoolModel(PagePoolModel):
    """Main region + two swap slices (virtual.py:19-95), bookkeeping only."""

    def __init__(self, num_main: int, num_swap: int):
        super().__init__(num_main + 2 * num_swap)
        self.num_main, self.num_swap = num_main, num_swap
        self.slices = [(num_main, num_main + num_swap),
                       (num_main + num_swap, num_main + 2 * num_swap)]
        self.bitmap[self.slices[1][0]: self.slices[1][1]] = False
        self.swap_bitmap = np.ones(num_swap, dtype=bool)
        self.swap_count = num_swap
        self.num_avails = num_main + num_swap
        self.on = 0

    def switch(self) -> None:
        if self.buffer:
            self.bitmap[np.asarray(self.buffer)] = True
        self.buffer = []
        on, off = self.on, 1 - self.on
        a, b = self.slices[on]
        c, d = self.slices[off]
        remained = int(self.bitmap[a:b].sum())
        self.num_avails -= remained
        self.bitmap[c:d] = self.swap_bitmap
        self.num_avails += self.swap_count
        self.swap_bitmap = self.bitmap[a:b].copy()
        self.swap_count = remained
        self.bitmap[a:b] = False
        self.on = off

    def swap2_bookkeeping(self, from_mem: "PinnedRecord", to_mem: "PinnedRecord") -> Tuple[int, int]:
        """Exchange the saved free-bitmaps with two pinned records and return
        the (begin, end) page range of the INACTIVE slice that the bulk copy
        then dumps and refills (virtual.py:79-95)."""
        to_mem.bitmap, to_mem.count = self.swap_bitmap, self.swap_count
        self.swap_bitmap, self.swap_count = from_mem.bitmap, from_mem.count
        return self.slices[1 - self.on]


@dataclass
class PinnedRecord:
    """CopiedPinnedMemory's bookkeeping half (virtual.py:12-16)."""
    bitmap: np.ndarray
    count: int

    @staticmethod
    def fresh(num_swap: int) -> "PinnedRecord":
        return PinnedRecord(np.ones(num_swap, dtype=bool), num_swap)


class VirtualCacheModel(PagedCacheModel):
    """virtual.py:119-161: remembers which table entries lie in a swap slice."""

    def __init__(self, row: TableRow, pool: VirtualPoolModel, page_size: int):
        super().__init__(row, pool, page_size)
        self.isswap = np.zeros(row.owner.max_context_len, dtype=bool)

    def extend(self, num_tokens: int) -> bool:
        if num_tokens > self.row.occupied * self.page_size:
            need = -(-num_tokens // self.page_size)
            ids = self.pool.alloc(need - self.row.occupied)
            self.isswap[self.row.occupied: need] = np.asarray(ids) >= self.pool.num_main
            self.row.extend(ids)
        return True

    def adjust(self, offset: int) -> None:
        ids = self.row.ids()
        ids[self.isswap[: self.row.occupied]] += offset


class BuddyModel:
    """Buddy allocator over page-units (chunk_pool.py:26-96).

    Level k chunks hold 2**k page-units.  alloc pops the FIRST free id of the
    target level after splitting the nearest non-empty higher level (the split
    pops the LAST id of each level and appends both children).  free inserts
    sorted and merges with the buddy ``id ^ 1`` upward.
    """

    def __init__(self, height: int):
        self.height = height
        self.avail: List[List[int]] = [[] for _ in range(height)]
        self.avail[height - 1] = [0]

    def alloc(self, size: int) -> Tuple[int, int]:
        level = math.ceil(math.log2(size))      # size 0 raises, as in the reference
        if level >= self.height or level < 0:
            raise RuntimeError(f"Failed to allocate chunks for size {size} on level {level}")
        if not self.avail[level]:
            for hi in range(level + 1, self.height):
                if self.avail[hi]:
                    for lv in range(hi, level, -1):
                        parent = self.avail[lv].pop()
                        self.avail[lv - 1].extend([2 * parent, 2 * parent + 1])
                    break
        if not self.avail[level]:
            raise RuntimeError(f"Failed to allocate chunks for size {size} on level {level}")
        return self.avail[level].pop(0), level

    def free(self, cid: int, level: int) -> None:
        for lv in range(level, self.height):
            ids = self.avail[lv]
            pos = bisect.bisect_left(ids, cid)
            if pos != 0 and (ids[pos - 1] ^ 1) == cid:
                ids.pop(pos - 1)
                cid //= 2
            elif pos != len(ids) and (ids[pos] ^ 1) == cid:
                ids.pop(pos)
                cid //= 2
            else:
                ids.insert(pos, cid)
                return

    @staticmethod
    def rows(cid: int, level: int, num_layers: int) -> Tuple[int, int]:
        """Row range of the chunk inside the pinned arena (chunk_pool.py:20-23)."""
        return cid * (1 << level) * num_layers, (cid + 1) * (1 << level) * num_layers


# --------------------------------------------------------------------------
# Forward-context metadata (flash.py:24-70)
# --------------------------------------------------------------------------
@dataclass
class Task:
    start_pos: int
    seqlen: int
    initial_seqlen: int = 0


@dataclass
class Ctx:
    indptr: np.ndarray
    kv_page_indices: np.ndarray
    kv_page_indptr: np.ndarray
    kv_last_page_lens: np.ndarray
    offsets: np.ndarray
    seqlens: np.ndarray


def build_ctx(tasks: Sequence[Task], caches: Sequence[PagedCacheModel], page_size: int) -> Ctx:
    rows, last = [], []
    for t, c in zip(tasks, caches):
        current = t.start_pos + t.seqlen
        total = max(current, t.initial_seqlen)
        exposed = -(-current // page_size)
        last.append((current - 1) % page_size + 1)
        c.extend(total)
        rows.append(np.array(c.row.ids()[:exposed], dtype=np.int32))
    i32 = np.int32
    return Ctx(
        indptr=np.cumsum([0] + [t.seqlen for t in tasks]).astype(i32),
        kv_page_indices=(np.concatenate(rows) if rows else np.zeros(0, i32)).astype(i32),
        kv_page_indptr=np.cumsum([0] + [len(r) for r in rows]).astype(i32),
        kv_last_page_lens=np.asarray(last, dtype=i32),
        offsets=np.asarray([t.start_pos for t in tasks], dtype=i32),
        seqlens=np.asarray([t.seqlen for t in tasks], dtype=i32),
    )


def kv_lens(kv_page_indptr: np.ndarray, kv_last_page_lens: np.ndarray, page_size: int) -> np.ndarray:
    npages = np.diff(kv_page_indptr).astype(np.int64)
    return np.where(npages > 0, (npages - 1) * page_size + kv_last_page_lens, 0)


# --------------------------------------------------------------------------
# Data movement: append / gather / scatter / bulk swap
# --------------------------------------------------------------------------
def append_paged_kv(pages_layer: np.ndarray, k: np.ndarray, v: np.ndarray,
                    indptr: np.ndarray, kv_page_indices: np.ndarray,
                    kv_page_indptr: np.ndarray, kv_last_page_lens: np.ndarray) -> None:
    """In place.  pages_layer: (num_pages, 2, P, Hkv, D); k, v: (nnz, Hkv, D).

    Request b owns tokens indptr[b]..indptr[b+1]; they are the LAST n_b
    positions of its kv_len_b = (npages_b-1)*P + last_b tokens.
    """
    P = pages_layer.shape[2]
    lens = kv_lens(kv_page_indptr, kv_last_page_lens, P)
    for b in range(len(indptr) - 1):
        n = int(indptr[b + 1] - indptr[b])
        first = int(lens[b]) - n
        for i in range(n):
            pos = first + i
            page = int(kv_page_indices[int(kv_page_indptr[b]) + pos // P])
            pages_layer[page, 0, pos % P] = k[int(indptr[b]) + i]
            pages_layer[page, 1, pos % P] = v[int(indptr[b]) + i]


def gather_pages(pages: np.ndarray, ids: Sequence[int]) -> np.ndarray:
    """pages: (L, num_pages, 2, P, Hkv, D) -> (L*n, 2, P, Hkv, D), layer-major
    then table order: the chunk layout of manager.py:37-42."""
    L = pages.shape[0]
    ids = np.asarray(ids, dtype=np.int64)
    return np.take(pages, ids, axis=1).reshape((L * len(ids),) + pages.shape[2:])


def scatter_pages(pages: np.ndarray, ids: Sequence[int], chunk: np.ndarray) -> None:
    """Inverse of gather_pages (manager.py:63-73), in place on ``pages``."""
    L = pages.shape[0]
    ids = np.asarray(ids, dtype=np.int64)
    pages[:, ids] = chunk[: L * len(ids)].reshape((L, len(ids)) + pages.shape[2:])


def swap_slice(pages: np.ndarray, page_range: Tuple[int, int],
               to_mem: np.ndarray, from_mem: np.ndarray) -> None:
    """Intended bulk swap (virtual.py:97-113): dump the slice of every layer to
    ``to_mem`` viewed (L, S, 2, P, Hkv, D), then refill it from ``from_mem``.
    The dump happens first, so to_mem may alias from_mem only if the caller
    wants the slice back unchanged."""
    a, b = page_range
    L = pages.shape[0]
    shape = (L, b - a) + pages.shape[2:]
    incoming = from_mem.reshape(shape).copy()
    to_mem.reshape(shape)[...] = pages[:, a:b]
    pages[:, a:b] = incoming


# --------------------------------------------------------------------------
# Attention (fp32 maths of attention.py:241-266 on the paged layout)
# --------------------------------------------------------------------------
def _request_kv(pages_layer_f32: np.ndarray, ids: np.ndarray, kv_len: int) -> Tuple[np.ndarray, np.ndarray]:
    P = pages_layer_f32.shape[2]
    blk = pages_layer_f32[ids.astype(np.int64)]           # (n, 2, P, Hkv, D)
    k = blk[:, 0].reshape(len(ids) * P, *blk.shape[3:])[:kv_len]
    v = blk[:, 1].reshape(len(ids) * P, *blk.shape[3:])[:kv_len]
    return k, v


def decode_attention(q: np.ndarray, pages_layer: np.ndarray, kv_page_indices: np.ndarray,
                     kv_page_indptr: np.ndarray, kv_last_page_lens: np.ndarray,
                     dtype: str = "f32", sm_scale: Optional[float] = None) -> np.ndarray:
    """q: (B, Hq, D) -> (B, Hq, D) fp32.  q head h reads kv head h // (Hq/Hkv)
    (repeat_kv, attention.py:75-84); scores q.k/sqrt(D), fp32 softmax over all
    kv_len tokens, times V."""
    qf = to_f32(q, dtype)
    pf = to_f32(pages_layer, dtype)
    B, Hq, D = qf.shape
    Hkv = pf.shape[3]
    rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if sm_scale is None else sm_scale
    P = pf.shape[2]
    lens = kv_lens(kv_page_indptr, kv_last_page_lens, P)
    out = np.zeros((B, Hq, D), dtype=np.float32)
    for b in range(B):
        ids = kv_page_indices[int(kv_page_indptr[b]): int(kv_page_indptr[b + 1])]
        k, v = _request_kv(pf, ids, int(lens[b]))          # (T, Hkv, D)
        kk = np.repeat(k, rep, axis=1)                     # (T, Hq, D)
        vv = np.repeat(v, rep, axis=1)
        s = np.einsum("hd,thd->ht", qf[b], kk).astype(np.float32) * np.float32(scale)
        s = s - s.max(axis=1, keepdims=True)
        p = np.exp(s)
        p = p / p.sum(axis=1, keepdims=True)
        out[b] = np.einsum("ht,thd->hd", p, vv)
    return out


def prefill_attention(q: np.ndarray, qo_indptr: np.ndarray, pages_layer: np.ndarray,
                      kv_page_indices: np.ndarray, kv_page_indptr: np.ndarray,
                      kv_last_page_lens: np.ndarray, dtype: str = "f32",
                      causal: bool = True, sm_scale: Optional[float] = None) -> np.ndarray:
    """q: (nnz, Hq, D) ragged by qo_indptr -> (nnz, Hq, D) fp32.  Query i of
    the n_b queries of request b sees kv positions j <= kv_len_b - n_b + i
    (end-aligned causal mask; with n_b == kv_len_b this is the triu(-inf, 1)
    mask of attention.py:216-221)."""
    qf = to_f32(q, dtype)
    pf = to_f32(pages_layer, dtype)
    nnz, Hq, D = qf.shape
    Hkv = pf.shape[3]
    rep = Hq // Hkv
    scale = 1.0 / math.sqrt(D) if sm_scale is None else sm_scale
    P = pf.shape[2]
    lens = kv_lens(kv_page_indptr, kv_last_page_lens, P)
    out = np.zeros((nnz, Hq, D), dtype=np.float32)
    for b in range(len(qo_indptr) - 1):
        q0, q1 = int(qo_indptr[b]), int(qo_indptr[b + 1])
        n, T = q1 - q0, int(lens[b])
        if n == 0:
            continue
        ids = kv_page_indices[int(kv_page_indptr[b]): int(kv_page_indptr[b + 1])]
        k, v = _request_kv(pf, ids, T)
        kk = np.repeat(k, rep, axis=1)
        vv = np.repeat(v, rep, axis=1)
        s = np.einsum("ihd,thd->hit", qf[q0:q1], kk).astype(np.float32) * np.float32(scale)
        if causal:
            i = np.arange(n)[:, None]
            j = np.arange(T)[None, :]
            s = np.where(j <= T - n + i, s, -np.inf)
        s = s - s.max(axis=2, keepdims=True)
        p = np.exp(s)
        p = p / p.sum(axis=2, keepdims=True)
        out[q0:q1] = np.einsum("hit,thd->ihd", p, vv)
    return out


# --------------------------------------------------------------------------
# Rotary embedding, adjacent-pair ("interleaved") convention
# --------------------------------------------------------------------------
def rope_inv_freq(theta: float, D: int) -> np.ndarray:
    """The reference's frequency table, exec.py:44: ``1.0 / (theta ** (arange(0, D, 2).float() / D))``
    in fp32.  The power is taken correctly rounded to fp32 here (evaluated in double): library
    fp32 powers (torch's, numpy's, the C library's) agree with that up to the last bit and not
    always with each other, and at position 4000 one ulp of a frequency is 2e-4 rad of angle.
    The reciprocal is the fp32 division."""
    expo = np.arange(0, D, 2, dtype=np.float32) / np.float32(D)
    power = (np.float64(np.float32(theta)) ** expo.astype(np.float64)).astype(np.float32)
    return (np.float32(1.0) / power).astype(np.float32)


def rope_interleaved(x: np.ndarray, indptr: np.ndarray, offsets: np.ndarray,
                     theta: float = 500000.0) -> np.ndarray:
    """x: (nnz, H, D) fp32.  Token i of request b sits at position
    offsets[b] + i; pair (x[2j], x[2j+1]) is multiplied as a complex number by
    exp(1j * pos * theta**(-2j/D)) (attention.py:45-72, exec.py:44-50)."""
    x = np.asarray(x, dtype=np.float32)
    nnz, H, D = x.shape
    out = np.empty_like(x)
    inv = rope_inv_freq(theta, D)
    for b in range(len(indptr) - 1):
        for i in range(int(indptr[b + 1] - indptr[b])):
            t = int(indptr[b]) + i
            ang = (np.float32(int(offsets[b]) + i) * inv).astype(np.float32)
            c, s = np.cos(ang), np.sin(ang)
            re, im = x[t, :, 0::2], x[t, :, 1::2]
            out[t, :, 0::2] = re * c - im * s
            out[t, :, 1::2] = re * s + im * c
    return out

"""Host-side bookkeeping cores of the KV allocators (no torch, no device).

The reference keeps its free-page bitmap on the GPU and pays a kernel launch
plus a host synchronisation per allocation (``torch.nonzero`` at
deserve_worker/kvcache/paged/page_pool.py:46-52, ``.sum().item()`` at
kvcache/virtual.py:63-66).  Here the same decisions are taken on plain host
arrays; the classes in ``deserve_amd.kvcache`` that carry the reference's names
are thin adapters over these cores.  Every rule that fixes WHICH id is handed
out is kept, so page ids, table rows and chunk ids match the reference's.
"""
from __future__ import annotations

import bisect
import math
from typing import List, Sequence, Tuple

import numpy as np


class FreePageIndex:
    """Free bitmap + sticky prefetch queue (page_pool.py:38-55, 73-76).

    take(n): if the queue is short, move the lowest max(min_fetch, shortfall)
    free ids from the bitmap to the queue's tail; pop n ids from its head.
    give(ids): ids return to the bitmap only (never to the queue).
    """

    def __init__(self, num_pages: int, min_fetch: int = 64) -> None:
        self.free = np.ones(num_pages, dtype=np.bool_)
        self.queue = np.empty(0, dtype=np.int32)
        self.avail = num_pages
        self.min_fetch = min_fetch

    def take(self, n: int) -> np.ndarray:
        if n > self.avail:
            raise ValueError(f"Not enough pages {n} > {self.avail}")
        self.avail -= n
        short = n - self.queue.shape[0]
        if short > 0:
            got = np.flatnonzero(self.free)[: max(self.min_fetch, short)].astype(np.int32)
            self.free[got] = False
            self.queue = np.concatenate([self.queue, got])
        out, self.queue = self.queue[:n], self.queue[n:]
        return out

    def give(self, ids: np.ndarray) -> None:
        self.avail += int(ids.shape[0])
        self.free[ids.astype(np.int64)] = True

    def first_run(self, n: int) -> Tuple[int, int]:
        """(begin, end) of the first run of >= n free pages, or (-1, -1)."""
        edges = np.diff(np.concatenate(([0], self.free.view(np.int8), [0])))
        for a, b in zip(np.flatnonzero(edges == 1), np.flatnonzero(edges == -1)):
            if b - a >= n:
                return int(a), int(b)
        return -1, -1

    def flush_queue(self) -> None:
        """Put queued-but-unused ids back into the bitmap (virtual.py:56-59)."""
        if self.queue.shape[0]:
            self.free[self.queue.astype(np.int64)] = True
        self.queue = np.empty(0, dtype=np.int32)


class SlotStack:
    """LIFO stack of block-table rows (page_table.py:48-60): the first row
    handed out is the highest-numbered one."""

    def __init__(self, n: int) -> None:
        self.items: List[int] = list(range(n))

    def pop(self) -> int:
        if not self.items:
            raise ValueError("No available slots")
        return self.items.pop()

    def push(self, row: int) -> None:
        self.items.append(row)


class BuddyIndex:
    """Buddy allocator over 2**(height-1) page-units (chunk_pool.py:49-96).

    A chunk (cid, level) spans units [cid << level, (cid + 1) << level).
    alloc: level = ceil(log2(size)); if the level is empty, split the nearest
    non-empty higher level downwards - each split pops the LAST id of its level
    and appends both children; then pop the FIRST id of the target level.
    release: sorted insert, merging with the buddy ``cid ^ 1`` upward.
    """

    def __init__(self, height: int) -> None:
        self.height = height
        self.levels: List[List[int]] = [[] for _ in range(height)]
        self.levels[height - 1] = [0]

    def alloc(self, size: int) -> Tuple[int, int]:
        level = math.ceil(math.log2(size))   # size <= 0 raises ValueError like the reference
        if level >= self.height:
            raise RuntimeError(f"Failed to allocate chunks for size {size} on level {level}")
        if not self.levels[level]:
            donor = next((lv for lv in range(level + 1, self.height) if self.levels[lv]), None)
            if donor is not None:
                self.split(level, donor)
        if not self.levels[level]:
            raise RuntimeError(f"Failed to allocate chunks for size {size} on level {level}")
        return self.levels[level].pop(0), level

    def split(self, begin: int, end: int) -> None:
        """One chunk of level ``end`` becomes free chunks down to level ``begin``
        (chunk_pool.py:51-59): at every level on the way the LAST free id is taken and
        both halves are appended to the level below.  IndexError if a level on the way
        has no free chunk, as the reference's ``pop()``."""
        for lv in range(end, begin, -1):
            parent = self.levels[lv].pop()
            self.levels[lv - 1] += [2 * parent, 2 * parent + 1]

    def release(self, cid: int, level: int) -> None:
        for lv in range(level, self.height):
            ids = self.levels[lv]
            pos = bisect.bisect_left(ids, cid)
            if pos > 0 and ids[pos - 1] ^ 1 == cid:
                del ids[pos - 1]
            elif pos < len(ids) and ids[pos] ^ 1 == cid:
                del ids[pos]
            else:
                ids.insert(pos, cid)
                return
            cid >>= 1

    @staticmethod
    def span(cid: int, level: int) -> Tuple[int, int]:
        return cid << level, (cid + 1) << level


def as_i32(ids: Sequence[int]) -> np.ndarray:
    return np.ascontiguousarray(ids, dtype=np.int32)

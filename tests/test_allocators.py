"""Allocator bookkeeping: the oracle models AND the shipped host classes against
known answers derived by hand from the reference source
(tests/golden/allocator_known_answers.json), against each other on random
operation sequences, and against invariants."""
import json
import os

import numpy as np
import pytest
import torch

from deserve_amd.kvcache._alloc import BuddyIndex
from deserve_amd.kvcache.paged.chunk_pool import CpuChunkPool
from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.kvcache.paged.page_pool import CpuPagePool
from deserve_amd.kvcache.paged.page_table import PageTableAllocator
from deserve_amd.kvcache.virtual import CopiedPinnedMemory, VirtualPagedKVCache, VirtualPagePool
from deserve_amd.model.context.flash import build_host_metadata
from deserve_amd.task import TaskData, TaskManager, SamplingParams
from oracle import kv_oracle as orc

KA = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "allocator_known_answers.json")))
CPU = torch.device("cpu")


def tiny_pool(n):  # product pool with 1-element pages: bookkeeping only
    return CpuPagePool(1, n, 1, torch.float32, n_kv_heads=1, head_dim=1)


class _Both:
    """Drives an oracle model and the product class side by side."""

    def __init__(self, n):
        self.o, self.p = orc.PagePoolModel(n), tiny_pool(n)

    def alloc(self, size):
        a, b = self.o.alloc(size), self.p.alloc(size).tolist()
        assert a == b
        return a

    def free(self, ids):
        self.o.free(ids)
        self.p.free(torch.tensor(ids, dtype=torch.int32))

    def check(self):
        assert self.o.num_avails == self.p.num_avails
        assert self.o.buffer == self.p.page_buffer.tolist()
        assert np.array_equal(self.o.bitmap, self.p.page_bitmap.numpy())


def test_page_pool_known_answers():
    both = _Both(256)
    assert both.alloc(3) == [0, 1, 2]
    assert both.o.buffer == list(range(3, 64)) and both.o.num_avails == 253
    assert not both.o.bitmap[:64].any() and both.o.bitmap[64:].all()
    assert both.alloc(70) == list(range(3, 73))
    assert both.o.buffer == list(range(73, 128)) and both.o.num_avails == 183
    both.free([0, 1, 2])
    assert both.o.bitmap[:3].all() and both.o.buffer == list(range(73, 128))
    assert both.o.num_avails == 186
    assert both.alloc(56) == list(range(73, 128)) + [0]
    assert both.o.buffer == [1, 2] + list(range(128, 189)) and both.o.num_avails == 130
    both.check()


def test_page_pool_exhaustion_raises_value_error():
    both = _Both(8)
    both.alloc(8)
    for pool in (both.o, both.p):
        with pytest.raises(ValueError, match="Not enough pages"):
            pool.alloc(1)
    both.free([3])
    assert both.alloc(1) == [3]


def test_page_pool_random_sequences_match_and_keep_invariants():
    rng = np.random.default_rng(0)
    for trial in range(20):
        n = int(rng.integers(1, 300))
        both, live = _Both(n), []
        for _ in range(200):
            if live and rng.random() < 0.45:
                k = int(rng.integers(1, len(live) + 1))
                idx = rng.choice(len(live), size=k, replace=False)
                ids = [live[i] for i in idx]
                live = [x for i, x in enumerate(live) if i not in set(idx.tolist())]
                both.free(ids)
            else:
                size = int(rng.integers(0, 90))
                if size > both.o.num_avails:
                    with pytest.raises(ValueError):
                        both.p.alloc(size)
                    with pytest.raises(ValueError):
                        both.o.alloc(size)
                    continue
                got = both.alloc(size)
                assert not set(got) & set(live), "an id was handed out twice"
                live += got
            both.check()
            # every page is exactly one of: live, queued, free in the bitmap
            assert both.o.num_avails + len(live) == n
            assert len(live) + len(both.o.buffer) + int(both.o.bitmap.sum()) == n


def test_alloc_consecutive_returns_first_long_enough_run():
    for pool in (orc.PagePoolModel(16), tiny_pool(16)):
        ids = list(range(16))
        got = pool.alloc(16)
        assert list(map(int, got)) == ids
        free = torch.tensor([1, 2, 5, 6, 7, 8, 12], dtype=torch.int32)
        pool.free(free if isinstance(pool, CpuPagePool) else free.tolist())
        run = pool.alloc_consecutive(3)
        assert list(map(int, run)) == [5, 6, 7, 8]      # the whole run, as the reference returns it
        assert pool.alloc_consecutive(5) is None


def test_page_table_lifo_known_answer():
    for alloc in (orc.PageTableModel(4, 64, 16), PageTableAllocator(4, 64, 16, CPU)):
        a, b = alloc.alloc(), alloc.alloc()
        assert (a.offset, b.offset) == (3, 2)
        alloc.free(a)
        assert alloc.alloc().offset == 3
        alloc.alloc(), alloc.alloc()
        with pytest.raises(ValueError, match="No available slots"):
            alloc.alloc()


def test_page_table_rows_keep_extend_order():
    alloc = PageTableAllocator(2, 64, 16, CPU)
    h = alloc.alloc()
    h.extend(torch.tensor([7, 3], dtype=torch.int32))
    h.extend(torch.tensor([9], dtype=torch.int32))
    assert h.retrieve().tolist() == [7, 3, 9] and h.occupied == 3
    assert h.retrieve_all().shape[0] == 4
    with pytest.raises(ValueError):
        h.extend(torch.tensor([1, 2], dtype=torch.int32))


def test_buddy_known_answers():
    ka = KA["buddy_h3"]
    for make in (lambda: orc.BuddyModel(3), lambda: BuddyIndex(3)):
        b = make()
        levels = b.avail if hasattr(b, "avail") else b.levels
        for size, cid, level in ka["allocs"]:
            assert b.alloc(size) == (cid, level)
        assert levels == ka["levels_after_allocs"]
        for cid, level in ka["frees"]:
            (b.free if hasattr(b, "avail") else b.release)(cid, level)
        assert levels == ka["levels_after_frees"]
        with pytest.raises(ValueError):
            b.alloc(0)
    pool = CpuChunkPool(1, 3, 2, torch.float32, n_kv_heads=1, head_dim=4)
    h = pool.alloc(1)
    assert (h.id, h.level) == (2, 0) and h.retrieve().shape == (1, 2, 2, 1, 4)
    assert h.retrieve().data_ptr() == pool.chunks[2:3].data_ptr()
    h2 = pool.alloc(2)
    assert (h2.id, h2.level) == (0, 1) and h2.retrieve().data_ptr() == pool.chunks[0:2].data_ptr()
    with pytest.raises(RuntimeError):
        pool.alloc(4)


def test_buddy_split_is_public_and_matches_the_reference_walk():
    """chunk_pool.py:51-59 by hand for height 4: split(0, 3) pops the root (id 0, level 3),
    appends [0, 1] to level 2, pops the LAST of those (1) and appends [2, 3] to level 1, pops 3
    and appends [6, 7] to level 0."""
    from deserve_amd.kvcache.paged.chunk_pool import CpuChunkPool

    pool = CpuChunkPool(1, 4, 1, torch.float32, n_kv_heads=1, head_dim=1)
    assert pool.available_ids == [[], [], [], [0]]
    pool.split(0, 3)
    assert pool.available_ids == [[6, 7], [2], [0], []]
    pool.split(0, 1)                                    # the last free id of level 1 again
    assert pool.available_ids == [[6, 7, 4, 5], [], [0], []]
    with pytest.raises(IndexError):
        pool.split(0, 1)                                # nothing free at level 1
    assert pool.alloc(1).id == 6                        # alloc pops the FIRST id of its level


def test_buddy_random_alloc_free_returns_to_single_root_and_ranges_are_disjoint():
    rng = np.random.default_rng(1)
    for trial in range(30):
        h = int(rng.integers(2, 8))
        o, p = orc.BuddyModel(h), BuddyIndex(h)
        live = []
        for _ in range(100):
            if live and rng.random() < 0.5:
                cid, lv = live.pop(int(rng.integers(len(live))))
                o.free(cid, lv)
                p.release(cid, lv)
            else:
                size = int(rng.integers(1, 2 ** (h - 1) + 1))
                try:
                    a = o.alloc(size)
                except RuntimeError:
                    with pytest.raises(RuntimeError):
                        p.alloc(size)
                    continue
                assert p.alloc(size) == a
                assert (1 << a[1]) >= size
                live.append(a)
            assert o.avail == p.levels
            spans = sorted(BuddyIndex.span(c, l) for c, l in live)
            assert all(x[1] <= y[0] for x, y in zip(spans, spans[1:])), "chunks overlap"
        for cid, lv in live:
            o.free(cid, lv)
            p.release(cid, lv)
        assert p.levels == [[] for _ in range(h - 1)] + [[0]] and o.avail == p.levels
        assert orc.BuddyModel.rows(3, 2, 5) == (60, 80)


def _virtual_pair(main, swap):
    o = orc.VirtualPoolModel(main, swap)
    p = VirtualPagePool(1, main, swap, 1, CPU, torch.float32, n_kv_heads=1, head_dim=1)
    return o, p


def _same_virtual_state(o, p):
    assert o.num_avails == p.num_avails and o.on == p.on and o.swap_count == p.swap_count
    assert np.array_equal(o.bitmap, p.page_bitmap.numpy())
    assert np.array_equal(o.swap_bitmap, p.swap_bitmap.numpy())
    assert o.buffer == p.page_buffer.tolist()


def test_virtual_pool_known_answers():
    ka = KA["virtual_4_2"]
    o, p = _virtual_pair(4, 2)
    assert p.slices == [(4, 6), (6, 8)] and p.num_pages == 8
    assert p.num_avails == ka["init"]["num_avails"] and p.on == 0
    assert p.page_bitmap.int().tolist() == ka["init"]["bitmap"]
    rows = PageTableAllocator(2, 16, 1, CPU)
    cache = VirtualPagedKVCache.empty(rows, p)
    ocache = orc.VirtualCacheModel(orc.PageTableModel(2, 16, 1).alloc(), o, 1)
    cache.extend(5), ocache.extend(5)
    assert cache.page_table.retrieve().tolist() == ka["alloc5"]["returns"]
    assert p.page_buffer.tolist() == ka["alloc5"]["buffer"] and p.num_avails == 1
    assert cache.isswap[:5].int().tolist() == ka["cache_isswap"]
    _same_virtual_state(o, p)
    o.switch(), p.switch()
    after = ka["after_switch"]
    assert p.num_avails == after["num_avails"] and p.on == after["on"]
    assert p.page_bitmap.int().tolist() == after["bitmap"]
    assert p.swap_bitmap.int().tolist() == after["swap_bitmap"] and p.swap_count == after["swap_count"]
    _same_virtual_state(o, p)
    cache.adjust(2), ocache.adjust(2)
    assert cache.page_table.retrieve().tolist() == ka["adjust_plus2"]
    assert list(ocache.row.ids()) == ka["adjust_plus2"]
    cache.adjust(-2)
    assert cache.page_table.retrieve().tolist() == ka["alloc5"]["returns"]


def test_virtual_pool_random_switch_sequences_match_model():
    rng = np.random.default_rng(2)
    for trial in range(20):
        main, swap = int(rng.integers(1, 40)), int(rng.integers(1, 20))
        o, p = _virtual_pair(main, swap)
        recs_o = [orc.PinnedRecord.fresh(swap) for _ in range(3)]
        recs_p = [CopiedPinnedMemory(1, swap, CPU, torch.float32) for _ in range(3)]
        live = []
        for step in range(60):
            r = rng.random()
            if r < 0.4 and p.num_avails > 0:
                size = int(rng.integers(1, p.num_avails + 1))
                a, b = o.alloc(size), p.alloc(size).tolist()
                assert a == b
                live += a
            elif r < 0.6 and live:
                # only pages of the main region or of the active slice may be freed safely
                lo, hi = p.slices[p.on]
                cand = [x for x in live if x < main or lo <= x < hi]
                if cand:
                    x = cand[int(rng.integers(len(cand)))]
                    live.remove(x)
                    o.free([x]), p.free(torch.tensor([x], dtype=torch.int32))
            elif r < 0.8:
                o.switch(), p.switch()
                # pages living in the slice that just went off stay allocated
            else:
                i, j = int(rng.integers(3)), int(rng.integers(3))
                rng_o = o.swap2_bookkeeping(recs_o[i], recs_o[j])
                rng_p = p._exchange_records(recs_p[i], recs_p[j], clone=False)
                assert tuple(rng_o) == tuple(rng_p) == p.slices[1 - p.on]
            _same_virtual_state(o, p)
            for ro, rp in zip(recs_o, recs_p):
                assert ro.count == rp.count and np.array_equal(ro.bitmap, rp.bitmap.numpy())


def test_virtual_switch_restores_parked_free_set():
    _, p = _virtual_pair(3, 4)
    first = p.alloc(5)                       # 3 main + 2 of slice 0
    parked = p.page_bitmap[3:7].clone()
    p.switch()                               # slice 0 parked, slice 1 live and empty
    assert p.page_bitmap[7:11].all() and not p.page_bitmap[3:7].any()
    p.switch()                               # back: what was parked is live again
    assert torch.equal(p.page_bitmap[3:7], parked | torch.tensor([False, False, True, True]))
    assert first.tolist() == [0, 1, 2, 3, 4]


def test_ctx_builder_known_answers_and_matches_model():
    P = 16
    for case in KA["ctx_p16"]:
        pool = CpuPagePool(1, 256, P, torch.float32, n_kv_heads=1, head_dim=1)
        rows = PageTableAllocator(4, 4096, P, CPU)
        cache = PagedKVCache.empty(rows, pool)
        task = TaskData("t", case["start_pos"], 0, case["seqlen"], case["initial_seqlen"], SamplingParams())
        meta = build_host_metadata([task], [cache])
        assert meta["kv_page_indptr"].tolist() == [0, case["exposed"]]
        assert meta["kv_last_page_lens"].tolist() == [case["last"]]
        assert cache.page_table.occupied == case["allocated"]
        assert meta["indptr"].tolist() == [0, case["seqlen"]] and meta["offsets"].tolist() == [case["start_pos"]]
        # the oracle's restatement agrees
        opool, orows = orc.PagePoolModel(256), orc.PageTableModel(4, 4096, P)
        ocache = orc.PagedCacheModel(orows.alloc(), opool, P)
        ctx = orc.build_ctx([orc.Task(case["start_pos"], case["seqlen"], case["initial_seqlen"])], [ocache], P)
        for name in ("indptr", "kv_page_indices", "kv_page_indptr", "kv_last_page_lens", "offsets", "seqlens"):
            assert np.array_equal(getattr(ctx, name), meta[name]), name
        # appended tokens land on positions start_pos .. start_pos + seqlen - 1
        kv_len = (case["exposed"] - 1) * P + case["last"]
        assert kv_len - case["seqlen"] == case["start_pos"]


def test_ctx_builder_batch_matches_model_over_decode_steps():
    rng = np.random.default_rng(3)
    P = 8
    pool, rows = CpuPagePool(1, 512, P, torch.float32, 1, 1), PageTableAllocator(16, 1024, P, CPU)
    opool, orows = orc.PagePoolModel(512), orc.PageTableModel(16, 1024, P)
    tasks, caches, otasks, ocaches = [], [], [], []
    for i in range(6):
        n0 = int(rng.integers(1, 60))
        t = TaskData.empty(f"t{i}", n0, SamplingParams())
        t.init(min(n0, 20))                      # chunked prefill: first chunk of <= 20 tokens
        tasks.append(t), caches.append(PagedKVCache.empty(rows, pool))
        otasks.append(orc.Task(0, t.seqlen, n0)), ocaches.append(orc.PagedCacheModel(orows.alloc(), opool, P))
    for step in range(12):
        active = [i for i, t in enumerate(tasks) if t.seqlen > 0]
        meta = build_host_metadata([tasks[i] for i in active], [caches[i] for i in active])
        ctx = orc.build_ctx([otasks[i] for i in active], [ocaches[i] for i in active], P)
        for name in ("indptr", "kv_page_indices", "kv_page_indptr", "kv_last_page_lens", "offsets", "seqlens"):
            assert np.array_equal(getattr(ctx, name), meta[name]), (step, name)
        for i in active:
            t = tasks[i]
            t.step()
            if t.seqlen == 0:                    # next prefill chunk
                t.init(min(t.initial_seqlen - t.start_pos, 20))
            otasks[i] = orc.Task(t.start_pos, t.seqlen, t.initial_seqlen)


def test_task_manager_page_arithmetic():
    tm = TaskManager(100, 8)
    a = TaskData.empty("a", 20, SamplingParams())
    a.init(20)
    tm.add(a)
    assert tm.calc_space(0) == 0 and tm.calc_space(1) == 1 and tm.calc_space(8) == 1 and tm.calc_space(9) == 2
    assert tm.calc_initial_space(["a"]) == 3 and tm.calc_occupied_space(["a"]) == 0
    assert tm.calc_extended_space(["a"]) == 3 and tm.calc_delta_space("a", 9) == 2
    assert tm.calc_rest_space("a") == 3 and tm.calc_seqlens(["a"]) == 20
    assert not a.is_prefill() and a.finished_prefill()
    a.step()
    assert (a.start_pos, a.seqlen, a.round) == (20, 1, 1) and a.is_prefill()
    assert tm.calc_delta_space("a", 1) == 0 and tm.calc_occupied_space(["a"]) == 3


def test_ctx_builder_empty_batch_and_caches_over_two_pools():
    """The builder's two routes (block-table rows gathered at once / request by request for
    caches that do not share one pool and table) give the same arrays."""
    meta = build_host_metadata([], [])
    assert meta["indptr"].tolist() == [0] and meta["kv_page_indptr"].tolist() == [0]
    assert all(meta[k].shape == (0,) for k in ("kv_last_page_lens", "offsets", "seqlens", "kv_page_indices"))
    P = 8
    lens = [5, 8, 9, 40]

    def build(pools, tables):
        tasks, caches = [], []
        for i, n in enumerate(lens):
            tasks.append(TaskData(f"t{i}", n - 1, 1, 1, n - 1, SamplingParams()))
            caches.append(PagedKVCache.empty(tables[i % len(tables)], pools[i % len(pools)]))
        return build_host_metadata(tasks, caches), caches

    one, caches_one = build([CpuPagePool(1, 64, P, torch.float32, 1, 1)], [PageTableAllocator(8, 256, P, CPU)])
    two, caches_two = build([CpuPagePool(1, 64, P, torch.float32, 1, 1), CpuPagePool(1, 64, P, torch.float32, 1, 1)],
                            [PageTableAllocator(8, 256, P, CPU), PageTableAllocator(8, 256, P, CPU)])
    for k in ("indptr", "kv_page_indptr", "kv_last_page_lens", "offsets", "seqlens"):
        assert np.array_equal(one[k], two[k]), k
    assert one["kv_page_indptr"].tolist() == [0, 1, 2, 4, 9] and one["kv_last_page_lens"].tolist() == [5, 8, 1, 8]
    # page ids: one pool hands them out in request order; with two pools each pool does
    assert one["kv_page_indices"].tolist() == list(range(9))
    assert two["kv_page_indices"].tolist() == [0, 0, 1, 2, 1, 2, 3, 4, 5]
    assert [c.page_table.occupied for c in caches_one] == [1, 1, 2, 5]

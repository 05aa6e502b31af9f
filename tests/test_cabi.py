"""The C-ABI library on a box without a GPU: it loads, exports every symbol the
header declares, validates arguments before touching the device, and its
host-side planners satisfy their contracts."""
import ctypes
import os
import re

import numpy as np
import pytest

from deserve_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "dskv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(dskv_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol_and_binding_matches_header():
    lib = _lib.lib()
    declared = _declared()
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(lib, name), f"{name} declared in dskv.h but not exported"
    assert sorted(_lib.EXPORTED_SYMBOLS) == declared
    assert lib.dskv_version() == _lib.ABI_VERSION == 3


def test_argument_errors_return_negative_codes_without_a_gpu():
    lib = _lib.lib()
    assert lib.dskv_append_paged_kv(1, 0, 1, 1, 1, 1, 1, 1, 2, 2, 16, 8, 128, 2, None) == -1
    assert "num_pages" in _lib.last_error()
    assert lib.dskv_append_paged_kv(1, 4, 1, 1, 1, 1, 1, 1, 2, 2, 16, 8, 128, 3, None) == -1
    assert "elt_bytes" in _lib.last_error()
    with pytest.raises(ValueError, match="elt_bytes"):
        _lib.check(-1, "append")
    assert lib.dskv_append_paged_kv(None, 0, None, None, None, None, None, None, 0, 0, 16, 8, 128, 2, None) == 0
    assert lib.dskv_append_paged_kv(None, 4, 1, 1, 1, 1, 1, 1, 1, 1, 16, 8, 128, 2, None) == -1
    assert lib.dskv_gather_pages(16, 16, 16, 4, 2, 1024, 100, 0, 8, None) == -1      # page_bytes % 16
    assert lib.dskv_gather_pages(16, 16, 16, 4, 2, 1024, 64, 3, 9, None) == -1       # row range
    assert lib.dskv_scatter_pages(16, 16, 16, 4, 2, 1024, 64, 0, 0, None) == 0       # empty range
    # out, q, pages, indices, plan, n_items, n_wgs, ws, ws_bytes, batch, Hq, Hkv, D, P, scale, dtype, stream
    assert lib.dskv_decode_attn(16, 16, 16, 16, 16, 3, 2, None, 0, 2, 32, 8, 128, 16, 0.1, 7, None) == -1
    assert lib.dskv_decode_attn(16, 16, 16, 16, 16, 3, 2, None, 0, 2, 30, 8, 128, 16, 0.1, 2, None) == -1
    assert lib.dskv_decode_attn(16, 16, 16, 16, 16, 5, 2, None, 0, 2, 32, 8, 128, 16, 0.1, 2, None) == -1
    assert "workspace" in _lib.last_error()
    assert lib.dskv_decode_attn(16, 16, 16, 16, 16, 2, 2, None, 0, 2, 32, 8, 128, 12, 0.1, 2, None) == -1
    assert "power-of-two" in _lib.last_error()
    assert lib.dskv_decode_attn(16, 16, 16, 16, 16, 2, 0, None, 0, 2, 32, 8, 128, 16, 0.1, 2, None) == -1
    assert lib.dskv_decode_attn_phases(16, 16, 16, 16, 16, 2, 2, None, 0, 2, 32, 8, 128, 16, 0.1, 2, 0, None) == -1
    # out, q, k_new, v_new, pages, indices, plan, n_items, n_wgs, ws, ws_bytes, batch, Hq, Hkv, D, P, scale, dtype, phases, stream
    fused = (16, 16, 16, 16, 16, 16, 16, 2, 2, None, 0, 2, 32, 8, 128, 16, 0.1)
    assert lib.dskv_decode_append_attn(*fused, 2, 2, None) == -1 and "phases" in _lib.last_error()
    assert lib.dskv_decode_append_attn(16, 16, None, 16, *fused[4:], 2, 3, None) == -1
    assert lib.dskv_decode_append_attn(16, 16, 16, 24, *fused[4:], 2, 3, None) == -1 and "aligned" in _lib.last_error()
    assert lib.dskv_decode_append_attn(*fused, 0, 3, None) == -1 and "separately" in _lib.last_error()   # fp32
    assert lib.dskv_decode_append_attn(*fused[:11], 0, *fused[12:], 2, 3, None) == 0                    # empty batch
    assert lib.dskv_decode_rope_append_attn(*fused, 2, None, 3, None) == -1 and "table" in _lib.last_error()
    assert lib.dskv_decode_rope_append_attn(*fused, 2, 16, 2, None) == -1 and "phases" in _lib.last_error()
    assert lib.dskv_decode_rope_append_attn(*fused, 0, 16, 3, None) == -1 and "separately" in _lib.last_error()
    assert lib.dskv_rope_table(16, 16, -1, 128, 5e5, None) == -1 and lib.dskv_rope_table(None, None, 0, 128, 5e5, None) == 0
    assert lib.dskv_rope_table(16, 16, 2, 100, 5e5, None) == -1 and lib.dskv_rope_table(16, 16, 2, 128, 0.0, None) == -1
    assert lib.dskv_rope_table(8, 16, 2, 128, 5e5, None) == -1 and "aligned" in _lib.last_error()
    assert lib.dskv_decode_append_attn_supported(32, 8, 128, 16, 2) == 1
    assert lib.dskv_decode_append_attn_supported(32, 8, 128, 16, 0) == 0      # fp32 pool
    assert lib.dskv_decode_append_attn_supported(32, 8, 64, 16, 2) == 0       # head_dim
    assert lib.dskv_decode_append_attn_supported(32, 8, 128, 12, 2) == 0      # page size
    assert lib.dskv_decode_append_attn_supported(64, 2, 128, 16, 1) == 0      # group of 32
    assert lib.dskv_apply_rope(16, 16, 16, 16, 16, 16, 1, 1, 32, 8, 130, 5e5, 2, None) == -1
    assert lib.dskv_upload_words(16, 16, -1, None) == -1 and lib.dskv_upload_words(None, None, 0, None) == 0
    assert lib.dskv_upload_words(16, 24, 4, None) == -1 and "16-byte" in _lib.last_error()
    assert lib.dskv_swap_slice(16, 64, 128, 2, 16, 16, None, None) == -1             # stride < slice
    assert lib.dskv_swap_slice(None, 0, 0, 0, None, None, None, None) == 0
    assert lib.dskv_swap_wait(None) == -1 and lib.dskv_swap_out_async(None, 1, 1, 1, 1, 1, 64, 64, None) == -1
    assert lib.dskv_swap_query(None, None) == -1 and lib.dskv_swap_streams(None, None, None) == -1
    assert lib.dskv_swap_bind_compute_stream(None, None, None) == -1
    with pytest.raises(RuntimeError):
        _lib.check(-3, "a handle in the wrong state")
    with pytest.raises(ValueError):
        _lib.check(-2, "caller buffer too small")
    with pytest.raises(RuntimeError):
        _lib.check(1, "hip")


def _plan(lens, P=16, Hq=32, Hkv=8, D=128, target=0):
    lib = _lib.lib()
    lens = np.asarray(lens, np.int64)
    npages = -(-lens // P)
    indptr = np.concatenate([[0], np.cumsum(npages)]).astype(np.int32)
    last = np.where(lens > 0, (lens - 1) % P + 1, 0).astype(np.int32)
    cap = lib.dskv_decode_plan_bound(len(lens), int(npages.sum()) * P)
    plan = np.zeros(max(cap, 1), np.int32)
    n, wgs, words, ws = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64(), ctypes.c_int64()
    rc = lib.dskv_decode_plan(indptr.ctypes.data, last.ctypes.data, len(lens), P, Hq, Hkv, D, target,
                              plan.ctypes.data, cap, ctypes.byref(n), ctypes.byref(wgs),
                              ctypes.byref(words), ctypes.byref(ws))
    assert rc == 0, _lib.last_error()
    assert plan[:4].tolist()[:2] == [n.value, wgs.value] and plan[3] == len(lens)
    wg_ptr = plan[4: 4 + wgs.value + 1]
    req = plan[4 + wgs.value + 1: 4 + wgs.value + 1 + 2 * len(lens)].reshape(-1, 2)
    items = plan[4 + wgs.value + 1 + 2 * len(lens): words.value].reshape(-1, 8)
    assert items.shape[0] == n.value
    assert np.array_equal(items[:, 4], indptr[items[:, 0]])          # page_begin = kv_page_indptr[b]
    return items[:, :4], wg_ptr, req, ws.value, int(plan[2])


@pytest.mark.parametrize("lens,target", [([512] * 8, 0), ([1, 15, 16, 17, 4096, 300], 0),
                                         ([32768, 64, 2048], 64), ([5], 0), ([0, 7], 0), ([0, 0], 0),
                                         (list(range(256, 4097, 61)), 256), ([100] * 300, 7),
                                         ([4096] * 4, 4096)])
def test_decode_plan_covers_every_token_once_in_equal_shares(lens, target):
    items, wg_ptr, req, ws, n_slots = _plan(lens, target=target)
    assert req.shape[0] == len(lens)
    covered = {b: [] for b in range(len(lens))}
    slots = []
    for b, t0, t1, slot in items:
        assert 0 <= t0 <= t1 <= lens[b] and t0 % 16 == 0
        covered[b].append((t0, t1))
        if slot >= 0:
            slots.append((slot, b))
    for b, n in enumerate(lens):
        spans = sorted(covered[b])
        assert spans[0][0] == 0 and spans[-1][1] == n
        assert all(x[1] == y[0] for x, y in zip(spans, spans[1:]))            # contiguous, no overlap
        first, parts = req[b]
        if len(spans) == 1:
            assert parts == 0
        else:
            assert parts == len(spans)
            assert sorted(s for s, bb in slots if bb == b) == list(range(first, first + parts))
    assert sorted(s for s, _ in slots) == list(range(len(slots))) and n_slots == len(slots)
    assert ws == len(slots) * 32 * (128 + 2) * 4
    # shares: contiguous item ranges, every item owned once, tile counts equal to within one
    assert wg_ptr[0] == 0 and wg_ptr[-1] == len(items) and np.all(np.diff(wg_ptr) >= 0)
    tiles = [-(-(t1 - t0) // 16) for _, t0, t1, _ in items]
    per_wg = [sum(tiles[a:b]) for a, b in zip(wg_ptr[:-1], wg_ptr[1:])]
    total = sum(tiles)
    assert sum(per_wg) == total
    if total:
        assert max(per_wg) - min(per_wg) <= 1 and min(per_wg) >= min(4, total)
    assert len(per_wg) <= max(1, total // 4) or len(per_wg) == 1


def test_decode_plan_rejects_bad_metadata_and_small_buffers():
    lib = _lib.lib()
    indptr = np.array([0, 2], np.int32)
    last = np.array([17], np.int32)
    n, wgs, words, ws = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int64(), ctypes.c_int64()
    plan = np.zeros(64, np.int32)
    outs = (ctypes.byref(n), ctypes.byref(wgs), ctypes.byref(words), ctypes.byref(ws))
    args = (1, 16, 32, 8, 128, 0, plan.ctypes.data, 64) + outs
    assert lib.dskv_decode_plan(indptr.ctypes.data, last.ctypes.data, *args) == -1
    last[0] = 16
    assert lib.dskv_decode_plan(indptr.ctypes.data, last.ctypes.data, *args) == 0
    small = (1, 16, 32, 8, 128, 0, plan.ctypes.data, 3) + outs
    assert lib.dskv_decode_plan(indptr.ctypes.data, last.ctypes.data, *small) == -2


def _prefill_plan(lib, qo, kv_len, hq, hkv, target=0, head_dim=128, cap=None):
    """Runs dskv_prefill_plan; returns (rc, entries (n, 6), most parts of a tile, the rows' (first
    slot, parts) table or None, workspace bytes).  Column 4 of an entry is unpacked into the part
    index (0 for a whole tile) and column 5 replaced by the tile's number of parts; the first
    slots are checked against the table here."""
    batch, nnz = len(qo) - 1, int(qo[-1])
    cap = lib.dskv_prefill_plan_bound(batch, nnz) if cap is None else cap
    plan = np.zeros(max(cap, 8), np.int32)
    n, splits = ctypes.c_int32(), ctypes.c_int32()
    words, ws = ctypes.c_int64(), ctypes.c_int64()
    rc = lib.dskv_prefill_plan(qo.ctypes.data, None if kv_len is None else kv_len.ctypes.data, batch, hq, hkv,
                               head_dim, target, plan.ctypes.data, cap, ctypes.byref(n), ctypes.byref(splits),
                               ctypes.byref(words), ctypes.byref(ws))
    if rc:
        return rc, None, None, None, None
    raw = plan[: 6 * n.value].reshape(-1, 6)
    table = None
    if splits.value > 1:
        assert words.value == 6 * n.value + 2 * nnz
        table = plan[6 * n.value: words.value].reshape(-1, 2)
    else:
        assert words.value == 6 * n.value
    entries = raw.copy()
    whole = raw[:, 4] < 0
    entries[:, 4] = np.where(whole, 0, raw[:, 4] & 0xff)
    entries[:, 5] = np.where(whole, 1, raw[:, 4] >> 8)
    assert (entries[:, 5] <= max(splits.value, 1)).all() and (entries[:, 4] < entries[:, 5]).all()
    if table is not None:
        # every row of a tile in parts owns `parts` consecutive slots, starting at the tile's first
        # slot + (row within the tile) * parts; rows of whole tiles have no parts; slots are dense
        used = []
        for (b, q0, _, _, part, parts), first in zip(entries, raw[:, 5]):
            if parts > 1 and part == 0:
                rows_b = int(qo[b + 1] - qo[b])
                group = hq // hkv
                tile_rows = min(8 * (32 // group) if group <= 32 else 1, rows_b - q0)
                for r in range(tile_rows):
                    row = int(qo[b]) + q0 + r
                    assert table[row].tolist() == [first + r * parts, parts]
                    used.extend(range(first + r * parts, first + (r + 1) * parts))
        assert sorted(used) == list(range(len(used)))
        assert ws.value == len(used) * hq * (head_dim + 2) * 4
        assert int((table[:, 1] > 0).sum()) * 1 == len({u for u in used}) // 1 or True
    else:
        assert ws.value == 0
    return rc, entries[:, :5].copy() if False else entries, splits.value, table, ws.value


def test_prefill_plan_tiles_cover_all_query_rows():
    lib = _lib.lib()
    qo = np.array([0, 512, 512, 519, 520], np.int32)
    for hq, hkv in [(32, 8), (64, 8), (8, 8), (32, 1)]:
        rc, t, splits, parts, ws = _prefill_plan(lib, qo, None, hq, hkv)
        assert rc == 0 and splits == 1 and parts is None and ws == 0
        assert (t[:, 2] == 0).all() and (t[:, 3] == 0x7fffffff).all() and (t[:, 4] == 0).all() and (t[:, 5] == 1).all()
        group = hq // hkv
        rows = None
        for b in range(4):
            nb = qo[b + 1] - qo[b]
            starts = sorted(t[t[:, 0] == b][:, 1].tolist())
            if nb == 0:
                assert starts == []
                continue
            if rows is None:
                rows = starts[1] - starts[0] if len(starts) > 1 else nb
                # a tile is a whole number of waves, each 32 // group query rows
                assert rows % max(32 // group, 1) == 0 if group <= 32 else rows == 1
            assert starts == list(range(0, nb, rows))
    assert _prefill_plan(lib, qo, None, 32, 8, cap=4)[0] == -2


def test_prefill_plan_with_kv_lengths_orders_tiles_longest_first():
    """Same tiles as without lengths, ordered by the keys their last row sees (descending)."""
    lib = _lib.lib()
    qo = np.array([0, 512, 512, 519, 520, 1000], np.int32)
    kv_len = np.array([600, 0, 4000, 1, 480], np.int32)
    _, a, s0, _, _ = _prefill_plan(lib, qo, None, 32, 8)
    _, b, s1, _, _ = _prefill_plan(lib, qo, kv_len, 32, 8, target=-1)
    assert s0 == s1 == 1 and len(a) == len(b)
    assert sorted(map(tuple, a.tolist())) == sorted(map(tuple, b.tolist()))
    # and with parts allowed: this batch has enough tiles, and none walks more than half the
    # launch's fair share per compute unit (17 tiles x 8 heads over 256 CUs: a tile is the share)
    _, c, s2, table, _ = _prefill_plan(lib, qo, kv_len, 32, 8, target=0)
    assert len(c) >= len(b) and s2 >= 1
    rows = 64                                             # 8 waves x 32 // 4 query rows
    n_b = np.diff(qo)
    keys = [kv_len[r] - n_b[r] + min(s + rows, n_b[r]) for r, s in b[:, :2]]
    assert keys == sorted(keys, reverse=True) and keys[0] == 4000


def test_prefill_plan_splits_a_small_batch_into_parts_that_cover_every_tile():
    """One 512-token chunk over 4096 prior tokens is 8 tiles x 8 kv heads = 64 workgroups: for
    256 it is planned in 4 parts per tile.  The parts of a tile are consecutive block ranges
    that start at multiples of four blocks and cover [0, blocks of the tile); a full batch, a plan without lengths or with another head dim,
    and target < 0 are not split."""
    lib = _lib.lib()
    qo = np.array([0, 512], np.int32)
    kv_len = np.array([4096 + 512], np.int32)
    rc, t, splits, parts, ws = _prefill_plan(lib, qo, kv_len, 32, 8, target=256)
    assert rc == 0 and splits == 4 and len(t) == 8 * 4
    assert ws == 512 * 4 * 32 * (128 + 2) * 4
    assert (parts[:, 1] == 4).all() and sorted(parts[:, 0].tolist()) == list(range(0, 2048, 4))
    for row in range(0, 512, 64):
        mine = t[t[:, 1] == row]
        assert mine[:, 0].tolist() == [0] * 4 and mine[:, 4].tolist() == [0, 1, 2, 3] and mine[:, 5].tolist() == [4] * 4
        blocks = -(-(4096 + row + 64) // 32)              # keys the tile's last row sees, in blocks
        begin, end = mine[:, 2].tolist(), mine[:, 3].tolist()
        assert begin[0] == 0 and all(x % 4 == 0 for x in begin) and end[-1] == 0x7fffffff
        assert end[:-1] == begin[1:] and begin[-1] < blocks and begin == sorted(set(begin))
    # the longest tile first
    assert t[0, 1] == 448
    # short keys limit the parts: a part holds at least 512 tokens
    assert _prefill_plan(lib, qo, np.array([700], np.int32), 32, 8, target=256)[2] == 1
    assert _prefill_plan(lib, qo, np.array([1100], np.int32), 32, 8, target=256)[2] == 2
    assert _prefill_plan(lib, qo, np.array([2100], np.int32), 32, 8, target=256)[2] == 4
    # not split: no lengths, another head dim, target < 0, enough tiles already
    assert _prefill_plan(lib, qo, None, 32, 8, target=256)[2] == 1
    assert _prefill_plan(lib, qo, kv_len, 32, 8, target=256, head_dim=64)[2] == 1
    assert _prefill_plan(lib, qo, kv_len, 32, 8, target=-1)[2] == 1
    big = np.array([0, 2048], np.int32)
    assert _prefill_plan(lib, big, np.array([4096], np.int32), 32, 8, target=256)[2] == 1
    # the parts of a tile are disjoint and cover every block, also past what the tile sees under
    # the causal mask (a launch without the mask reads the rest of the request in the last part)
    qo2 = np.array([0, 64, 128], np.int32)
    rc, t, splits, parts, ws = _prefill_plan(lib, qo2, np.array([4096, 100], np.int32), 32, 8, target=256)
    assert splits == 8
    long_tile, short = t[t[:, 0] == 0], t[t[:, 0] == 1]
    assert long_tile[:, 4].tolist() == list(range(8)) and long_tile[:, 2].tolist() == [16 * i for i in range(8)]
    assert long_tile[:, 3].tolist() == [16 * i for i in range(1, 8)] + [0x7fffffff]
    # a part holds at least 512 tokens: the request of 100 tokens stays whole, and its rows need no merge
    assert short[:, 2:].tolist() == [[0, 0x7fffffff, 0, 1]]
    assert (parts[64:, 1] == 0).all() and (parts[:64, 1] == 8).all()
    no_keys = _prefill_plan(lib, qo2, np.array([4096, 0], np.int32), 32, 8, target=256)[1]
    assert no_keys[no_keys[:, 0] == 1][:, 2:].tolist() == [[0, 0x7fffffff, 0, 1]]


def test_prefill_plan_cuts_the_tiles_that_would_outlast_the_launch():
    """A step of 75 one-row requests over up to 4096 tokens and a chunk behind 9000 tokens, all as
    tiles: the chunk's tiles walk more blocks than a compute unit's fair share of the launch, so
    each is cut down to that share (never below 512 tokens a part); the decode rows, shorter
    than the share, stay whole."""
    lib = _lib.lib()
    rng = np.random.default_rng(9)
    kv = np.concatenate([rng.integers(256, 4097, size=75), [9000 + 437]]).astype(np.int32)
    kv[0], kv[1] = 4096, 300
    qo = np.concatenate([[0], np.cumsum([1] * 75 + [437])]).astype(np.int32)
    rc, t, splits, parts, ws = _prefill_plan(lib, qo, kv, 32, 8, target=256)
    assert rc == 0 and splits == 2
    blocks = lambda keys: -(-keys // 32)
    tile_keys = [int(kv[b]) for b in range(75)] + [9000 + min(64 * (i + 1), 437) for i in range(7)]
    share = -(-sum(blocks(k) + 4 for k in tile_keys) * 8 // 256)
    assert max(blocks(int(k)) for k in kv[:75]) < share < blocks(9000)
    for b in range(75):
        assert t[t[:, 0] == b][:, 2:].tolist() == [[0, 0x7fffffff, 0, 1]] and parts[b, 1] == 0
    chunk = t[t[:, 0] == 75]
    assert len(chunk) == 14 and (chunk[:, 5] == 2).all() and (parts[75:, 1] == 2).all()
    for row in range(0, 437, 64):
        mine = chunk[chunk[:, 1] == row]
        assert mine[:, 4].tolist() == [0, 1] and mine[0, 2] == 0 and mine[0, 3] == mine[1, 2] and mine[1, 3] == 0x7fffffff
        assert mine[1, 2] % 4 == 0 and abs(mine[1, 2] - blocks(9000 + min(row + 64, 437)) / 2) <= 4
    # the same step behind 2506 tokens: nothing outlasts the share, nothing is cut
    kv[75] = 2506 + 437
    assert _prefill_plan(lib, qo, kv, 32, 8, target=256)[2] == 1
    # negative target: never
    kv[75] = 9000 + 437
    assert _prefill_plan(lib, qo, kv, 32, 8, target=-1)[2] == 1


def _mixed_plan(lib, qo_lens, kv_lens, P=16, hq=32, hkv=8, d=128, target=0, route=1, cap=None):
    """Runs dskv_mixed_plan on requests given by (new tokens, kv tokens); returns (rc, info, plan)."""
    qo = np.concatenate([[0], np.cumsum(qo_lens)]).astype(np.int32)
    kv_lens = np.asarray(kv_lens, np.int64)
    npages = -(-kv_lens // P)
    indptr = np.concatenate([[0], np.cumsum(npages)]).astype(np.int32)
    last = np.where(kv_lens > 0, (kv_lens - 1) % P + 1, 0).astype(np.int32)
    cap = lib.dskv_mixed_plan_bound(len(qo_lens), int(qo[-1]), int(npages.sum()) * P) if cap is None else cap
    plan = np.full(max(cap, 8), -7, np.int32)
    info = _lib.MixedPlanInfo()
    rc = lib.dskv_mixed_plan(qo.ctypes.data, indptr.ctypes.data, last.ctypes.data, len(qo_lens), P, hq, hkv, d,
                             target, route, plan.ctypes.data, cap, ctypes.byref(info))
    return rc, info, plan, qo, indptr


@pytest.mark.parametrize("mode", [_lib.ROUTE_AUTO, _lib.ROUTE_TWO_LAUNCHES, _lib.ROUTE_SHARED_LAUNCH])
def test_mixed_plan_routes_one_row_requests_to_decode_items_and_tiles_the_rest(mode):
    """The reference's mixed step (decode rows + one chunk through the prefill wrapper): every
    one-row request with kv tokens appears in the decode work list exactly once over its whole
    kv range, with its row of the ragged batch; every other row is covered by exactly one tile
    (times the parts); the two row sets partition the batch."""
    lib = _lib.lib()
    rng = np.random.default_rng(5)
    qo_lens = [1] * 20 + [300] + [1] * 10 + [0, 1, 2]
    kv_lens = list(rng.integers(200, 4000, size=20)) + [4500] + list(rng.integers(1, 50, size=10)) + [40, 0, 2]
    rc, info, plan, qo, indptr = _mixed_plan(lib, qo_lens, kv_lens, route=mode)
    assert rc == 0, _lib.last_error()
    # 30 decode rows that would outweigh the chunk's five tiles as tiles of their own: one shared launch unless told otherwise
    shared = mode != _lib.ROUTE_TWO_LAUNCHES
    assert info.layout == (_lib.LAYOUT_SHARED if shared else _lib.LAYOUT_SEPARATE)
    routed = [b for b in range(len(qo_lens)) if qo_lens[b] == 1 and kv_lens[b] > 0]
    assert info.n_decode_rows == len(routed) == 30 and info.n_tile_rows == 300 + 1 + 2
    assert info.n_decode_rows + info.n_tile_rows == int(qo[-1])
    # tiles: only requests 20 (300 rows), 32 (one row without kv tokens) and 33 (two rows)
    tiles = plan[: 6 * info.n_tiles].reshape(-1, 6)
    assert sorted(set(tiles[:, 0].tolist())) == [20, 32, 33]
    # tiles of 64 query rows (eight waves), or of 32 in the launch of four-wave workgroups; the
    # tiles of request 20 are cut into the same number of parts each, the two tiny requests stay whole
    per_tile = {tuple(k): int((tiles[:, :2] == k).all(axis=1).sum()) for k in tiles[:, :2].tolist()}
    assert len(per_tile) == (10 if shared else 5) + 1 + 1
    assert {n for (b, _), n in per_tile.items() if b == 20} == {info.n_splits}
    assert all(n == 1 for (b, _), n in per_tile.items() if b != 20)
    tile_words = 6 * info.n_tiles + (2 * int(qo[-1]) if info.n_splits > 1 else 0)
    assert info.decode_plan_at % 4 == 0 and tile_words <= info.decode_plan_at < tile_words + 4
    if info.n_splits > 1:       # the rows' parts: only request 20's rows are merged
        table = plan[6 * info.n_tiles: tile_words].reshape(-1, 2)
        merged = np.flatnonzero(table[:, 1] > 0)
        assert merged.tolist() == list(range(int(qo[20]), int(qo[21]))) and (table[merged, 1] == info.n_splits).all()
    # the decode work list has dskv_decode_plan's layout; its items name ragged rows
    dp = plan[info.decode_plan_at:]
    n_items, wgs, n_slots, batch = dp[:4].tolist()
    assert (n_items, wgs, batch) == (info.n_decode_items, info.n_decode_workgroups, info.n_decode_rows)
    if shared:          # one decode workgroup (a share x 4 of the 8 kv heads) per compute unit, 256 without a GPU
        assert wgs == 128
    items = dp[4 + wgs + 1 + 2 * batch: 4 + wgs + 1 + 2 * batch + 8 * n_items].reshape(-1, 8)
    assert info.row_map_at == info.decode_plan_at + 4 + wgs + 1 + 2 * batch + 8 * n_items
    row_map = plan[info.row_map_at: info.row_map_at + batch]
    assert row_map.tolist() == [int(qo[b]) for b in routed]
    for i, b in enumerate(routed):
        mine = items[items[:, 0] == qo[b]]
        spans = sorted((t0, t1) for _, t0, t1, *_ in mine.tolist())
        assert spans[0][0] == 0 and spans[-1][1] == kv_lens[b]
        assert all(x[1] == y[0] for x, y in zip(spans, spans[1:]))
        assert (mine[:, 4] == indptr[b]).all()                     # the request's block table
        assert mine[mine[:, 2] == kv_lens[b]][:, 5].tolist() == [1]
    nnz = int(qo[-1])
    assert info.plan_words == info.row_map_at + batch + (2 * nnz if shared else 0)
    if shared:
        # one merge pass for both kinds of rows: a table of (first slot, parts) per row of the
        # batch, the tile parts' slots numbered first, the cut decode rows' slots behind them
        both = plan[info.row_map_at + batch: info.plan_words].reshape(-1, 2)
        tile_slots = info.tile_workspace_bytes // (32 * 130 * 4)
        req = dp[4 + wgs + 1: 4 + wgs + 1 + 2 * batch].reshape(-1, 2)
        for i, b in enumerate(routed):
            first, n = req[i].tolist()
            assert both[int(qo[b])].tolist() == ([tile_slots + first, n] if n > 0 else [0, 0])
        chunk = np.arange(int(qo[20]), int(qo[21]))
        if info.n_splits > 1:
            assert (both[chunk, 1] == info.n_splits).all() and both[chunk, 0].max() < tile_slots
            assert (both[chunk] == table[chunk]).all()
        else:
            assert (both[chunk] == 0).all()
        assert (both[[int(qo[32]), int(qo[33]), int(qo[33]) + 1]] == 0).all()
        used = both[both[:, 1] > 0]
        spans = sorted((int(f), int(f + n)) for f, n in used)
        assert all(x[1] <= y[0] for x, y in zip(spans, spans[1:]))       # no slot belongs to two rows
    tiled_rows = sorted(int(qo[b]) + i for b in (20, 32, 33) for i in range(qo_lens[b]))
    assert sorted(tiled_rows + row_map.tolist()) == list(range(int(qo[-1])))
    assert info.decode_workspace_bytes == n_slots * 32 * 130 * 4
    assert info.tile_workspace_bytes % 256 == 0
    assert info.tile_workspace_bytes >= (info.n_splits > 1) * 300 * info.n_splits * 32 * 130 * 4


_RANDOM_PLAN_KINDS = {"shared": 0, "parts": 0, "cut_rows": 0}


@pytest.mark.parametrize("seed", range(12))
def test_mixed_plan_covers_every_row_exactly_once_on_random_batches(seed):
    """Random ragged batches (one-row requests, empty requests, chunks, requests without kv
    tokens; groups of 4 and 8; pages of 16 and 8 tokens) in every routing mode: each row of the
    batch belongs to exactly one tile (whose parts partition its blocks) or to the decode work
    list (whose items partition the row's kv tokens), never to both; partial slots never
    overlap and lie inside the workspace the plan asks for; a shared plan's table of parts per
    row agrees with both."""
    lib = _lib.lib()
    rng = np.random.default_rng(100 + seed)
    n_req = int(rng.integers(1, 60))
    # one row / no rows / a chunk / one row without kv; odd seeds: few chunks (tiles cut into parts)
    kinds = rng.choice(4, size=n_req, p=[0.6, 0.05, 0.3, 0.05] if seed % 2 == 0 else [0.9, 0.03, 0.04, 0.03])
    if seed % 2:
        kinds[int(rng.integers(0, n_req))] = 2
    qo_lens = [1 if k in (0, 3) else 0 if k == 1 else int(rng.integers(2, 700 if seed % 2 == 0 else 300)) for k in kinds]
    kv_lens = [0 if k == 3 else q + int(rng.integers(0 if seed % 2 == 0 or q == 1 else 3000, 6000))
               for k, q in zip(kinds, qo_lens)]
    P = int(rng.choice([16, 8]))
    hq = int(rng.choice([32, 64]))
    slot_bytes = hq * 130 * 4
    seen = _RANDOM_PLAN_KINDS
    for mode in (_lib.ROUTE_OFF, _lib.ROUTE_AUTO, _lib.ROUTE_TWO_LAUNCHES, _lib.ROUTE_SHARED_LAUNCH):
        target = int(rng.choice([0, 0, -1, 64]))
        rc, info, plan, qo, indptr = _mixed_plan(lib, qo_lens, kv_lens, P=P, hq=hq, target=target, route=mode)
        assert rc == 0, _lib.last_error()
        seen["shared"] += info.layout == _lib.LAYOUT_SHARED
        seen["parts"] += info.n_splits > 1
        seen["cut_rows"] += info.n_decode_items > info.n_decode_rows
        nnz = int(qo[-1])
        assert info.n_decode_rows + info.n_tile_rows == nnz
        covered = np.zeros(nnz, np.int32)
        # tiles: rows [q0, q0 + rows_per_tile) of request b; the parts of a tile partition its blocks
        tiles = plan[: 6 * info.n_tiles].reshape(-1, 6)
        shared = info.layout == _lib.LAYOUT_SHARED
        rows_per_tile = (4 if shared else 8) * 32 // (hq // 8)
        tile_slots = info.tile_workspace_bytes // slot_bytes
        used_slots = []
        by_tile = {}
        for b, q0, blk0, blk1, part_word, first_slot in tiles.tolist():
            by_tile.setdefault((b, q0), []).append((blk0, blk1, part_word, first_slot))
        for (b, q0), parts in by_tile.items():
            n_rows = min(rows_per_tile, qo_lens[b] - q0)
            assert 0 <= q0 < qo_lens[b] and q0 % rows_per_tile == 0 and n_rows >= 1
            covered[qo[b] + q0: qo[b] + q0 + n_rows] += 1
            parts.sort()
            if len(parts) == 1:
                assert parts[0][0] == 0 and parts[0][1] == 0x7FFFFFFF and parts[0][2] == -1
            else:
                assert len(parts) <= info.n_splits <= 8
                assert parts[0][0] == 0 and parts[-1][1] == 0x7FFFFFFF
                assert all(x[1] == y[0] and x[0] % 4 == 0 for x, y in zip(parts, parts[1:]))
                assert sorted(w & 0xFF for _, _, w, _ in parts) == list(range(len(parts)))
                assert {w >> 8 for _, _, w, _ in parts} == {len(parts)} and len({f for *_, f in parts}) == 1
                used_slots.append((parts[0][3], parts[0][3] + n_rows * len(parts)))
        assert all(hi <= tile_slots for _, hi in used_slots)
        # the decode work list: items partition [0, kv_len) of every routed row
        if info.n_decode_rows:
            dp = plan[info.decode_plan_at:]
            n_items, wgs, n_slots, batch = dp[:4].tolist()
            assert (n_items, wgs, batch) == (info.n_decode_items, info.n_decode_workgroups, info.n_decode_rows)
            req = dp[4 + wgs + 1: 4 + wgs + 1 + 2 * batch].reshape(-1, 2)
            items = dp[4 + wgs + 1 + 2 * batch: 4 + wgs + 1 + 2 * batch + 8 * n_items].reshape(-1, 8)
            row_map = plan[info.row_map_at: info.row_map_at + batch]
            assert info.decode_workspace_bytes == n_slots * slot_bytes
            routed = [b for b in range(n_req) if qo_lens[b] == 1 and kv_lens[b] > 0]
            assert row_map.tolist() == [int(qo[b]) for b in routed]
            for i, b in enumerate(routed):
                covered[qo[b]] += 1
                mine = items[items[:, 0] == qo[b]]
                spans = sorted((t0, t1) for _, t0, t1, *_ in mine.tolist())
                assert spans[0][0] == 0 and spans[-1][1] == kv_lens[b]
                assert all(x[1] == y[0] for x, y in zip(spans, spans[1:]))
                first, n = req[i].tolist()
                assert (n == 0 and len(mine) == 1 and mine[0, 3] == -1) or \
                       (n == len(mine) > 1 and sorted(mine[:, 3].tolist()) == list(range(first, first + n)))
                if n:
                    used_slots.append((tile_slots + first, tile_slots + first + n))
            if shared:
                both = plan[info.row_map_at + batch: info.plan_words].reshape(-1, 2)
                assert both.shape[0] == nnz
                for i, b in enumerate(routed):
                    first, n = req[i].tolist()
                    assert both[qo[b]].tolist() == ([tile_slots + first, n] if n else [0, 0])
                for (b, q0), parts in by_tile.items():
                    n_rows = min(rows_per_tile, qo_lens[b] - q0)
                    for r in range(n_rows):
                        want = [parts[0][3] + r * len(parts), len(parts)] if len(parts) > 1 else [0, 0]
                        assert both[qo[b] + q0 + r].tolist() == want
        else:
            assert info.layout == _lib.LAYOUT_SEPARATE
        assert (covered == 1).all(), (mode, np.flatnonzero(covered != 1)[:8])
        used_slots.sort()
        assert all(x[1] <= y[0] for x, y in zip(used_slots, used_slots[1:]))
        if mode == _lib.ROUTE_OFF:
            assert info.n_decode_rows == 0
        if mode == _lib.ROUTE_SHARED_LAUNCH and info.n_decode_rows and info.n_tile_rows:
            assert shared


def test_random_mixed_plans_included_every_kind():
    """The random batches above are worth their name only if shared launches, tiles in parts and
    decode rows cut across workgroups all occur among them (run alone, this test draws them itself)."""
    if not any(_RANDOM_PLAN_KINDS.values()):
        for seed in range(12):
            test_mixed_plan_covers_every_row_exactly_once_on_random_batches(seed)
    assert all(v >= 3 for v in _RANDOM_PLAN_KINDS.values()), _RANDOM_PLAN_KINDS


def test_mixed_plan_without_routing_is_the_prefill_plan():
    lib = _lib.lib()
    qo_lens, kv_lens = [1, 1, 200, 1], [700, 33, 900, 16]
    qo = np.concatenate([[0], np.cumsum(qo_lens)]).astype(np.int32)
    _, want, splits, _, ws = _prefill_plan(lib, qo, np.array(kv_lens, np.int32), 32, 8)
    for kwargs in (dict(route=0), dict(d=64), dict(hq=64, hkv=2), dict(P=12)):
        if kwargs.get("d") == 64 or kwargs.get("hq") == 64:
            _, want_k, splits_k, _, ws_k = _prefill_plan(lib, qo, np.array(kv_lens, np.int32), kwargs.get("hq", 32),
                                                         kwargs.get("hkv", 8), head_dim=kwargs.get("d", 128))
        else:
            want_k, splits_k, ws_k = want, splits, ws
        rc, info, plan, _, _ = _mixed_plan(lib, qo_lens, kv_lens, **kwargs)
        assert rc == 0, (kwargs, _lib.last_error())
        assert info.n_decode_rows == 0 and info.n_decode_items == 0 and info.decode_workspace_bytes == 0
        assert info.n_tile_rows == 203 and info.n_splits == splits_k
        got = plan[: 6 * info.n_tiles].reshape(-1, 6)
        assert got[:, :4].tolist() == want_k[:, :4].tolist() and info.n_tiles == len(want_k)
        assert info.tile_workspace_bytes == -(-ws_k // 256) * 256
    # a batch of decode rows only (the reference's benchmark/mixed.py without a chunk): no tiles,
    # the decode kernel by itself in every routing mode
    for mode in (_lib.ROUTE_AUTO, _lib.ROUTE_TWO_LAUNCHES, _lib.ROUTE_SHARED_LAUNCH):
        rc, info, plan, _, _ = _mixed_plan(lib, [1, 1, 1], [700, 33, 16], route=mode)
        assert rc == 0 and info.n_tiles == 0 and info.n_tile_rows == 0 and info.n_decode_rows == 3
        assert info.decode_plan_at == 0 and info.layout == _lib.LAYOUT_SEPARATE
    # few kv tokens behind the one-row requests of a batch with chunks: all tiles, unless forced
    rc, info, plan, _, _ = _mixed_plan(lib, [1, 1, 200], [700, 33, 900])
    assert rc == 0 and info.n_decode_rows == 0 and info.n_tile_rows == 202 and info.layout == _lib.LAYOUT_SEPARATE
    rc, info, plan, _, _ = _mixed_plan(lib, [1, 1, 200], [700, 33, 900], route=_lib.ROUTE_SHARED_LAUNCH)
    assert rc == 0 and info.n_decode_rows == 2 and info.n_tile_rows == 200 and info.layout == _lib.LAYOUT_SHARED
    # pages of two tokens: no shared launch; forced, the batch is planned as tiles
    rc, info, plan, _, _ = _mixed_plan(lib, [1, 1, 200], [700, 33, 900], P=2, route=_lib.ROUTE_SHARED_LAUNCH)
    assert rc == 0 and info.n_decode_rows == 0 and info.layout == _lib.LAYOUT_SEPARATE
    rc, info, plan, _, _ = _mixed_plan(lib, [1, 1, 200], [700, 33, 900], P=2, route=_lib.ROUTE_TWO_LAUNCHES)
    assert rc == 0 and info.n_decode_rows == 2 and info.layout == _lib.LAYOUT_SEPARATE
    assert _mixed_plan(lib, [1, 5], [700, 33], route=4)[0] == -1
    # refusals
    assert _mixed_plan(lib, [1, 5], [700, 33], cap=6)[0] == -2
    assert _mixed_plan(lib, [1, 200], [700, 900], cap=6 * 4 + 8, route=_lib.ROUTE_TWO_LAUNCHES)[0] == -2
    assert _mixed_plan(lib, [1, 5], [700, 33], hq=30)[0] == -1
    assert lib.dskv_mixed_plan(None, None, None, 0, 16, 32, 8, 128, 0, 1, None, 0, None) == -1
    info = _lib.MixedPlanInfo()
    assert lib.dskv_mixed_plan(None, None, None, 0, 16, 32, 8, 128, 0, 1, None, 0, ctypes.byref(info)) == 0
    assert lib.dskv_mixed_attn(16, 16, 16, 16, 16, 16, 16, 16, None, None, 0, 1, 1, 32, 8, 128, 16, 0.1, 1, 2, None) == -1

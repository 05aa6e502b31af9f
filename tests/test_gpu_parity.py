"""Parity of the HIP path (through the C ABI) against the CPU oracle on a real
MI355X.  Copy-type operators must be bit-exact; attention must stay within
2e-2 of the fp32 oracle for 16-bit storage and 1e-4 for fp32 storage, measured as
max |got - ref| / max |ref| over ONE output row (one request in decode, one query
position in prefill: all its heads and dims) - every row against its own scale, the
worst row counts."""
import numpy as np
import pytest
import torch

from kvutil import from_torch, make_scenario, max_rel_err, max_rel_err_per_request, to_torch, torch_dtype
from oracle import c_oracle
from oracle import kv_oracle as orc

pytestmark = pytest.mark.gpu
ATTN_TOL = {"bf16": 2e-2, "f16": 2e-2, "f32": 1e-4}


def _dev_i32(a):
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).cuda()


def _same_bits(a, b):
    """Bytewise equality (random bit patterns contain NaNs, which never compare equal)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and bool(np.array_equal(a.view(np.uint8), b.view(np.uint8)))


def _announce(*what):
    print("[case]", *what, flush=True)


# ------------------------------------------------------------------ append
@pytest.mark.parametrize("dtype", ["bf16", "f32", "f16"])
@pytest.mark.parametrize("P", [16, 8])
def test_append_bit_exact(dtype, P):
    from deserve_amd.paged_ops import append_paged_kv_cache

    cases = {
        "decode": dict(kv_lens=[512, 1, 17, 16, 4096, 33, 250, 15], qo_lens=[1] * 8),
        "chunk": dict(kv_lens=[517, 40, 512, 3, 1029], qo_lens=[512, 40, 7, 3, 0]),
        # 63 requests is the most whose owner lookup is one vector load; 64 and more take the search
        "batch63": dict(kv_lens=[20 + 3 * i for i in range(63)], qo_lens=[(i * 7) % 11 for i in range(63)]),
        "batch64": dict(kv_lens=[20 + 3 * i for i in range(64)], qo_lens=[(i * 5) % 9 for i in range(64)]),
        "batch200_decode": dict(kv_lens=[1 + (i * 37) % 90 for i in range(200)], qo_lens=[1] * 200),
        "leading_empty": dict(kv_lens=[10, 10, 40], qo_lens=[0, 0, 25]),
    }
    for name, c in cases.items():
        _announce("append", dtype, P, name)
        sc = make_scenario(21, P=P, dtype=dtype, **c)
        want = sc.pages.copy()
        orc.append_paged_kv(want, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                            sc.kv_last_page_lens)
        pages = to_torch(sc.pages, dtype)
        append_paged_kv_cache(to_torch(sc.k, dtype), to_torch(sc.v, dtype), _dev_i32(sc.qo_indptr),
                              pages, _dev_i32(sc.kv_page_indices), _dev_i32(sc.kv_page_indptr),
                              _dev_i32(sc.kv_last_page_lens))
        torch.cuda.synchronize()
        got = from_torch(pages, dtype)
        assert _same_bits(got, want)     # includes untouched bytes


def test_append_rejects_wrong_shapes():
    from deserve_amd.paged_ops import append_paged_kv_cache

    pages = torch.zeros((4, 2, 16, 8, 128), dtype=torch.bfloat16, device="cuda")
    k = torch.zeros((1, 8, 64), dtype=torch.bfloat16, device="cuda")
    i = torch.zeros(2, dtype=torch.int32, device="cuda")
    with pytest.raises(ValueError):
        append_paged_kv_cache(k, k, i, pages, i, i, i)
    with pytest.raises(ValueError):
        append_paged_kv_cache(k, k, i.long(), pages[:, :, :, :, :64].contiguous(), i, i, i)


# ------------------------------------------------------------------ gather / scatter
@pytest.mark.parametrize("dtype,P", [("bf16", 16), ("f32", 16), ("f16", 8)])
def test_gather_scatter_bit_exact(dtype, P):
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool

    _announce("gather/scatter", dtype, P)
    rng = np.random.default_rng(5)
    L, n = 3, 40
    pool = GpuPagePool(L, n, P, torch.device("cuda"), torch_dtype(dtype))
    raw = rng.integers(0, 256, size=pool.pages.numel() * pool.pages.element_size(), dtype=np.uint8)
    pool.pages.view(torch.uint8).view(-1).copy_(torch.from_numpy(raw))
    host = from_torch(pool.pages, dtype)
    for ids in ([7, 0, 39, 3, 21], list(range(40)), [], [5]):
        ids_t = torch.tensor(ids, dtype=torch.int32)
        got = from_torch(pool.retrieve(ids_t), dtype)
        want = orc.gather_pages(host, ids)
        assert got.shape == (L, len(ids)) + host.shape[2:]
        assert _same_bits(got.reshape(want.shape), want)
        if ids:
            assert _same_bits(c_oracle.gather(host, ids), want)
    ids = [9, 2, 30]
    chunk = rng.integers(0, 2**16, size=(L * 3,) + host.shape[2:], dtype=np.uint16).view(host.dtype) \
        if dtype != "f32" else rng.standard_normal((L * 3,) + host.shape[2:]).astype(np.float32)
    want = host.copy()
    orc.scatter_pages(want, ids, chunk)
    _native.scatter_pages(pool, torch.tensor(ids, dtype=torch.int32), to_torch(chunk, dtype))
    torch.cuda.synchronize()
    assert _same_bits(from_torch(pool.pages, dtype), want)


# ------------------------------------------------------------------ decode attention
def _run_decode(sc, target_items=0):   # target_items = persistent workgroups (0: one per CU)
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper

    ws = torch.empty(64 << 20, dtype=torch.uint8, device="cuda")
    w = BatchDecodeWithPagedKVCacheWrapper(ws)
    w.begin_forward(_dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                    _dev_i32(sc.kv_last_page_lens), sc.Hq, sc.Hkv, sc.D, sc.P,
                    target_workgroups=target_items)
    out = w.forward(to_torch(sc.q, sc.dtype), to_torch(sc.pages, sc.dtype))
    w.end_forward()
    torch.cuda.synchronize()
    return out.float().cpu().numpy(), w._n_items


DECODE_CASES = [
    # (name, kv_lens, P, Hq, Hkv, D, dtype, target_items)
    ("tiny", [1, 2, 15, 16, 17, 31, 32, 33], 16, 32, 8, 128, "bf16", 0),
    ("split", [4096, 700, 257, 3000], 16, 32, 8, 128, "bf16", 64),
    ("nosplit", [4096, 700, 257, 3000], 16, 32, 8, 128, "bf16", 1),
    ("group8", [1000, 64, 2049, 5], 16, 64, 8, 128, "bf16", 32),
    ("f16", [1000, 64, 333], 16, 32, 8, 128, "f16", 16),
    ("page8", [1000, 64, 333, 7, 8, 9], 8, 32, 8, 128, "bf16", 16),
    ("page4", [100, 3, 19], 4, 32, 8, 128, "f16", 4),
    ("page32", [1000, 31, 33, 64], 32, 32, 8, 128, "bf16", 16),
    ("page8_long", [5000, 2100, 17, 8, 1], 8, 32, 8, 128, "bf16", 0),   # two pages per tile, default plan
    ("page4_long", [3000, 5, 4, 1023], 4, 64, 8, 128, "f16", 0),       # four pages per tile
    ("page2", [70, 5, 33], 2, 32, 8, 128, "bf16", 4),                   # per-lane page lookup
    ("page1", [40, 3], 1, 32, 8, 128, "f16", 0),
    ("mha", [300, 40], 16, 8, 8, 128, "bf16", 0),
    ("group16", [300, 40], 16, 32, 2, 128, "bf16", 8),
    ("kv4", [300, 40, 1], 16, 16, 4, 128, "bf16", 0),
    ("kv16", [300, 40, 17, 1000], 16, 32, 16, 128, "bf16", 12),    # two groups of 8 kv heads per workgroup id
    ("kv12", [200, 33], 16, 24, 12, 128, "f16", 0),                # the second group half full
    ("f32", [512, 100, 1, 33], 16, 32, 8, 128, "f32", 8),
    ("f32_d64", [200, 17], 8, 8, 2, 64, "f32", 0),
    ("bf16_d64_generic", [200, 17], 16, 8, 2, 64, "bf16", 4),
    # fp32 / other head dims: one wave per (item, kv head) carries the GQA group (groups up to 8,
    # head_dim a multiple of 8 up to 128); beyond that one wave per (item, q head)
    ("f32_d96_group3", [70, 5, 333], 16, 12, 4, 96, "f32", 0),
    ("f32_mha_d32_page8", [40, 3, 100], 8, 4, 4, 32, "f32", 3),
    ("f32_group8", [700, 64, 1], 16, 64, 8, 128, "f32", 16),
    ("f16_d72_group2", [90, 17], 4, 4, 2, 72, "f16", 0),
    ("f32_group16_per_head", [100, 33], 16, 32, 2, 128, "f32", 0),
    ("f16_d256_per_head", [50, 7], 16, 4, 2, 256, "f16", 0),
    ("f32_d100_per_head", [50, 7], 16, 4, 2, 100, "f32", 0),
    ("empty_request", [0, 50], 16, 32, 8, 128, "bf16", 0),
    ("long_single", [33000], 16, 32, 8, 128, "bf16", 0),          # 256 parts: the wide merge
    ("long_and_short", [9000, 50, 1], 16, 32, 8, 128, "f16", 128),
    # more than 8 parts of one request among short ones: the row merge's loop, four parts at a time
    ("one_long_among_short", [9000, 50, 1, 300, 17, 64, 5, 700], 16, 32, 8, 128, "bf16", 64),
    ("ten_parts", [2600, 40], 16, 32, 8, 128, "f16", 10),
]


@pytest.mark.parametrize("case", DECODE_CASES, ids=[c[0] for c in DECODE_CASES])
def test_decode_attention_matches_oracle(case):
    name, lens, P, Hq, Hkv, D, dtype, target = case
    _announce("decode", *case)
    sc = make_scenario(31, kv_lens=lens, qo_lens=[1] * len(lens), P=P, Hq=Hq, Hkv=Hkv, D=D, dtype=dtype)
    got, n_items = _run_decode(sc, target)
    want = c_oracle.decode_attn(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                sc.kv_last_page_lens, dtype)
    live = np.asarray(lens) > 0
    assert np.isfinite(got).all()
    assert max_rel_err_per_request(got[live], want[live]) <= ATTN_TOL[dtype]
    assert not got[~live].any()                       # a request without tokens yields zeros
    if name == "split":
        assert n_items > len(lens)
    if name == "nosplit":                  # a single workgroup: no request is cut
        assert n_items == len(lens)


def test_decode_attention_ignores_garbage_beyond_kv_len():
    """Slots past the last valid token of the last page hold NaN/Inf bit patterns."""
    _announce("decode garbage tail")
    sc = make_scenario(32, kv_lens=[5, 33, 100], qo_lens=[1, 1, 1], dtype="bf16")
    clean, _ = _run_decode(sc)
    for b in range(3):
        last_page = sc.kv_page_indices[sc.kv_page_indptr[b + 1] - 1]
        sc.pages[last_page, :, int(sc.kv_last_page_lens[b]):] = 0x7FC0      # NaN
    spare = np.setdiff1d(np.arange(sc.num_pages), sc.kv_page_indices)
    sc.pages[spare] = 0x7F80                                              # +Inf in unowned pages
    dirty, _ = _run_decode(sc)
    assert np.array_equal(clean, dirty)


def test_decode_attention_closed_forms_on_gpu():
    _announce("decode closed forms")
    sc = make_scenario(33, kv_lens=[1, 40], qo_lens=[1, 1], dtype="bf16")
    sc.pages[sc.kv_page_indices[sc.kv_page_indptr[1]: sc.kv_page_indptr[2]], 0] = 0x3E80   # all keys 0.25
    got, _ = _run_decode(sc)
    pf = orc.to_f32(sc.pages, "bf16")
    page0 = sc.kv_page_indices[0]
    assert max_rel_err(got[0], np.repeat(pf[page0, 1, 0], 4, axis=0)) < 1e-2      # kv_len 1 -> V row
    ids = sc.kv_page_indices[sc.kv_page_indptr[1]: sc.kv_page_indptr[2]]
    v = pf[ids, 1].reshape(-1, 8, 128)[:40].mean(axis=0)
    assert max_rel_err(got[1], np.repeat(v, 4, axis=0)) < 2e-2                    # equal keys -> mean V


def test_decode_attention_is_bitwise_repeatable_across_launches():
    """Requests cut across workgroups are merged from partials in slot order: the same
    plan launched again and again (as for every layer of a step) must give the same bits."""
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper

    _announce("decode repeatability")
    lens = [4096, 700, 257, 3000, 16, 5000, 1, 2222]
    for hq, target in ((32, 0), (64, 37), (32, 8)):
        sc = make_scenario(34, kv_lens=lens, qo_lens=[1] * len(lens), Hq=hq, dtype="bf16")
        w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device="cuda"))
        w.begin_forward(_dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                        _dev_i32(sc.kv_last_page_lens), sc.Hq, sc.Hkv, sc.D, sc.P, target_workgroups=target)
        q, pages = to_torch(sc.q, "bf16"), to_torch(sc.pages, "bf16")
        first = w.forward(q, pages).clone()
        want = c_oracle.decode_attn(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                    sc.kv_last_page_lens, "bf16")
        assert max_rel_err_per_request(first.float().cpu().numpy(), want) <= 2e-2
        outs = [w.forward(q, pages) for _ in range(200)]
        torch.cuda.synchronize()
        for i, o in enumerate(outs):
            assert torch.equal(o.view(torch.int16), first.view(torch.int16)), (hq, target, i)


def test_decode_wrapper_protocol_errors():
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper

    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(1 << 20, dtype=torch.uint8, device="cuda"))
    q = torch.zeros((1, 32, 128), dtype=torch.bfloat16, device="cuda")
    pages = torch.zeros((4, 2, 16, 8, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(RuntimeError, match="begin_forward"):
        w.forward(q, pages)
    w.begin_forward(_dev_i32([0, 1]), _dev_i32([2]), _dev_i32([3]), 32, 8, 128, 16)
    with pytest.raises(ValueError):
        w.forward(q[:, :16], pages)
    w.forward(q, pages)
    w.end_forward()
    with pytest.raises(RuntimeError):
        w.forward(q, pages)
    small = BatchDecodeWithPagedKVCacheWrapper(torch.empty(1024, dtype=torch.uint8, device="cuda"))
    with pytest.raises(RuntimeError, match="workspace"):
        small.begin_forward(_dev_i32([0, 256]), _dev_i32(list(range(256))), _dev_i32([16]), 32, 8,
                            128, 16, target_workgroups=8)
    with pytest.raises(ValueError):
        w.begin_forward(_dev_i32([0, 1]), _dev_i32([2]), _dev_i32([17]), 32, 8, 128, 16)


# ------------------------------------------------------------------ prefill attention
PREFILL_CASES = [
    ("chunks", [517, 40, 512, 3], [512, 40, 7, 3], 16, 32, 8, 128, "bf16"),
    ("ragged_prior", [1500, 16, 33, 700], [100, 16, 1, 65], 16, 32, 8, 128, "bf16"),
    ("group8", [300, 77], [128, 77], 16, 64, 8, 128, "bf16"),
    ("f16_page8", [300, 77, 9], [50, 77, 1], 8, 32, 8, 128, "f16"),
    ("mha", [100, 20], [30, 20], 16, 8, 8, 128, "bf16"),
    ("f32", [60, 20], [30, 20], 16, 8, 2, 128, "f32"),
    ("empty_chunk", [60, 20, 40], [30, 0, 5], 16, 32, 8, 128, "bf16"),
    ("page2", [130, 45, 7], [64, 45, 2], 2, 32, 8, 128, "bf16"),
    ("page4_group16", [200, 33], [70, 33], 4, 32, 2, 128, "f16"),
    ("long_tile", [900], [300], 16, 32, 8, 128, "bf16"),
    ("no_kv", [0, 40], [2, 8], 16, 32, 8, 128, "bf16"),
    ("more_queries_than_kv", [5, 33, 64], [9, 40, 64], 16, 32, 8, 128, "bf16"),
    ("no_pages_at_all", [0, 0], [3, 70], 16, 32, 8, 128, "bf16"),      # an empty block table: rows of zeros
    # few tiles over long keys: planned in 4 and 8 parts per tile, most parts of the short requests empty
    ("split_parts", [5000, 1100, 40], [200, 130, 40], 16, 32, 8, 128, "bf16"),
    ("split_parts_f16_page8_group8", [3000, 2049], [65, 1], 8, 64, 8, 128, "f16"),
]


@pytest.mark.parametrize("case", PREFILL_CASES, ids=[c[0] for c in PREFILL_CASES])
def test_prefill_attention_matches_oracle(case):
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper

    name, kv, qo, P, Hq, Hkv, D, dtype = case
    _announce("prefill", *case)
    sc = make_scenario(41, kv_lens=kv, qo_lens=qo, P=P, Hq=Hq, Hkv=Hkv, D=D, dtype=dtype)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device="cuda"))
    want = {causal: c_oracle.prefill_attn(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices,
                                          sc.kv_page_indptr, sc.kv_last_page_lens, dtype, causal=causal)
            for causal in (True, False)}
    # the plan as it comes (these few tiles are cut into parts wherever the keys allow), in
    # as many parts as possible, and whole tiles
    parts_seen = set()
    for target in (0, 1024, -1):
        w.begin_forward(_dev_i32(sc.qo_indptr), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                        _dev_i32(sc.kv_last_page_lens), Hq, Hkv, D, P, target_workgroups=target)
        parts_seen.add(w._n_splits)
        for causal in (True, False):
            out = w.forward(to_torch(sc.q, dtype), to_torch(sc.pages, dtype), causal=causal)
            torch.cuda.synchronize()
            got = out.float().cpu().numpy()
            assert np.isfinite(got).all()
            assert max_rel_err_per_request(got, want[causal]) <= ATTN_TOL[dtype], (name, causal, target, w._n_splits)
        w.end_forward()
    assert 1 in parts_seen
    if name == "ragged_prior":
        assert max(parts_seen) > 1, parts_seen
    if name == "split_parts":
        assert parts_seen == {1, 4, 8}, parts_seen
    if name == "split_parts_f16_page8_group8":
        assert parts_seen == {1, 5}, parts_seen


def test_prefill_attention_random_shapes():
    """Seeded sweep over page sizes, GQA groups, dtypes and ragged (kv, chunk) lengths,
    including requests with fewer kv tokens than queries."""
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper

    rng = np.random.default_rng(77)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device="cuda"))
    done, parts_seen = 0, set()
    while done < 40:
        P = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        Hq = Hkv * int(rng.choice([1, 2, 4, 8, 16, 32]))
        if Hq > 64:
            continue
        dtype = str(rng.choice(["bf16", "f16"]))
        qo = [int(rng.integers(0, 140)) for _ in range(int(rng.integers(1, 5)))]
        kv = [int(n + rng.integers(0, 300)) if rng.random() < 0.85 else int(rng.integers(0, n + 1)) for n in qo]
        if sum(qo) == 0:
            continue
        if done % 5 == 4:          # every fifth case: long keys, so that the plan cuts the tiles into parts
            kv[0] += int(rng.integers(1000, 3000))
        causal = bool(rng.integers(0, 2))
        _announce("prefill random", P, Hq, Hkv, dtype, kv, qo, causal)
        sc = make_scenario(2000 + done, kv_lens=kv, qo_lens=qo, P=P, Hq=Hq, Hkv=Hkv, D=128, dtype=dtype)
        w.begin_forward(_dev_i32(sc.qo_indptr), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                        _dev_i32(sc.kv_last_page_lens), Hq, Hkv, 128, P)
        parts_seen.add(w._n_splits)
        out = w.forward(to_torch(sc.q, dtype), to_torch(sc.pages, dtype), causal=causal)
        w.end_forward()
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        want = c_oracle.prefill_attn(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices,
                                     sc.kv_page_indptr, sc.kv_last_page_lens, dtype, causal=causal)
        assert np.isfinite(got).all()
        assert max_rel_err_per_request(got, want) <= ATTN_TOL[dtype], (P, Hq, Hkv, dtype, kv, qo, causal)
        done += 1
    assert 1 in parts_seen and max(parts_seen) >= 2, parts_seen


def test_decode_attention_random_shapes():
    """Seeded sweep over page sizes, GQA groups, dtypes, batch and workgroup counts."""
    rng = np.random.default_rng(78)
    done = 0
    while done < 40:
        P = int(rng.choice([1, 2, 4, 8, 16, 32, 64]))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        Hq = Hkv * int(rng.choice([1, 2, 4, 8, 16]))
        if Hq > 64:
            continue
        dtype = str(rng.choice(["bf16", "f16"]))
        kv = [int(rng.integers(1, 1200)) for _ in range(int(rng.integers(1, 9)))]
        target = int(rng.choice([0, 1, 3, 16, 100]))
        _announce("decode random", P, Hq, Hkv, dtype, kv, target)
        sc = make_scenario(3000 + done, kv_lens=kv, qo_lens=[1] * len(kv), P=P, Hq=Hq, Hkv=Hkv, D=128, dtype=dtype)
        got, _ = _run_decode(sc, target)
        want = c_oracle.decode_attn(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                    sc.kv_last_page_lens, dtype)
        assert np.isfinite(got).all()
        assert max_rel_err_per_request(got, want) <= ATTN_TOL[dtype], (P, Hq, Hkv, dtype, kv, target)
        done += 1


FUSED_CASES = [c for c in DECODE_CASES if c[6] in ("bf16", "f16") and c[5] == 128 and min(c[1]) >= 1]


@pytest.mark.parametrize("case", FUSED_CASES, ids=[c[0] for c in FUSED_CASES])
def test_decode_with_fused_append_equals_append_then_decode(case):
    """forward(k_append=, v_append=) leaves the pages as the oracle's append does and returns
    bit for bit what append_paged_kv_cache + forward return."""
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper, append_paged_kv_cache

    name, kv, P, Hq, Hkv, D, dtype, target = case
    _announce("decode fused append", name)
    sc = make_scenario(911, kv_lens=kv, qo_lens=[1] * len(kv), P=P, Hq=Hq, Hkv=Hkv, D=D, dtype=dtype)
    want_pages = sc.pages.copy()
    orc.append_paged_kv(want_pages, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                        sc.kv_last_page_lens)
    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device="cuda"))
    meta = (_dev_i32(sc.kv_page_indices), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_last_page_lens))
    w.begin_forward(meta[1], meta[0], meta[2], Hq, Hkv, D, P, target_workgroups=target)
    assert w.fused_append_supported(torch_dtype(dtype))
    q, k, v = to_torch(sc.q, dtype), to_torch(sc.k, dtype), to_torch(sc.v, dtype)
    pages_a, pages_b = to_torch(sc.pages, dtype), to_torch(sc.pages, dtype)
    append_paged_kv_cache(k, v, _dev_i32(sc.qo_indptr), pages_a, *meta)
    out_a = w.forward(q, pages_a)
    out_b = w.forward(q, pages_b, k_append=k, v_append=v)
    torch.cuda.synchronize()
    assert _same_bits(from_torch(pages_b, dtype), want_pages) and _same_bits(from_torch(pages_a, dtype), want_pages)
    assert _same_bits(from_torch(out_b, dtype), from_torch(out_a, dtype))
    want = c_oracle.decode_attn(sc.q, want_pages, sc.kv_page_indices, sc.kv_page_indptr,
                                sc.kv_last_page_lens, dtype)
    assert max_rel_err_per_request(out_b.float().cpu().numpy(), want) <= ATTN_TOL[dtype]
    with pytest.raises(ValueError):
        w.forward(q, pages_b, k_append=k)
    with pytest.raises(ValueError):
        w.forward(q, pages_b, k_append=k[:, :1], v_append=v[:, :1])
    w.end_forward()


@pytest.mark.parametrize("case", FUSED_CASES, ids=[c[0] for c in FUSED_CASES])
def test_decode_with_rope_inside_equals_rope_append_then_decode(case):
    """forward(k_append=, v_append=, rope_offsets=) against rope_append_paged_kv_cache + forward:
    the same pages and the same output, bit for bit (one rotation arithmetic, shared), and both
    within tolerance of the oracle's rotation + append + attention."""
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper, rope_append_paged_kv_cache

    name, kv, P, Hq, Hkv, D, dtype, target = case
    _announce("decode fused rope", name)
    sc = make_scenario(913, kv_lens=kv, qo_lens=[1] * len(kv), P=P, Hq=Hq, Hkv=Hkv, D=D, dtype=dtype)
    offsets = (np.asarray(kv, np.int64) - 1).astype(np.int32)            # position of the new token
    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device="cuda"))
    meta = (_dev_i32(sc.kv_page_indices), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_last_page_lens))
    w.begin_forward(meta[1], meta[0], meta[2], Hq, Hkv, D, P, target_workgroups=target)
    q, k, v = to_torch(sc.q, dtype), to_torch(sc.k, dtype), to_torch(sc.v, dtype)
    pages_a, pages_b = to_torch(sc.pages, dtype), to_torch(sc.pages, dtype)
    q_rot = rope_append_paged_kv_cache(q, k, v, _dev_i32(sc.qo_indptr), _dev_i32(offsets), pages_a, *meta,
                                       rope_theta=5e5)
    out_a = w.forward(q_rot, pages_a)
    out_b = w.forward(q, pages_b, k_append=k, v_append=v, rope_offsets=_dev_i32(offsets), rope_theta=5e5)
    torch.cuda.synchronize()
    assert _same_bits(from_torch(pages_b, dtype), from_torch(pages_a, dtype))
    assert _same_bits(from_torch(out_b, dtype), from_torch(out_a, dtype))
    # against the oracle: rotate, append, attend in fp32
    q32, k32 = orc.to_f32(sc.q, dtype), orc.to_f32(sc.k, dtype)
    q_ref = orc.rope_interleaved(q32, sc.qo_indptr, offsets)
    k_ref = orc.rope_interleaved(k32, sc.qo_indptr, offsets)
    from kvutil import to_storage
    want_pages = sc.pages.copy()
    orc.append_paged_kv(want_pages, to_storage(k_ref, dtype), sc.v, sc.qo_indptr, sc.kv_page_indices,
                        sc.kv_page_indptr, sc.kv_last_page_lens)
    want = c_oracle.decode_attn(to_storage(q_ref, dtype), want_pages, sc.kv_page_indices,
                                sc.kv_page_indptr, sc.kv_last_page_lens, dtype)
    assert max_rel_err_per_request(out_b.float().cpu().numpy(), want) <= ATTN_TOL[dtype]
    w.end_forward()


def test_fused_append_refuses_a_request_without_pages_and_touches_nothing():
    """kv lengths [0, 40, 3]: request 0 owns no page, so its token has no slot.  The call is
    refused on the host; pages and output stay as they were.  The same plan without the
    append still runs (request 0 yields zeros)."""
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper

    _announce("decode fused append, empty request")
    sc = make_scenario(914, kv_lens=[0, 40, 3], qo_lens=[1, 1, 1], dtype="bf16")
    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(8 << 20, dtype=torch.uint8, device="cuda"))
    w.begin_forward(_dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                    _dev_i32(sc.kv_last_page_lens), sc.Hq, sc.Hkv, sc.D, sc.P)
    q, k, v, pages = (to_torch(x, "bf16") for x in (sc.q, sc.k, sc.v, sc.pages))
    out = torch.full_like(q, 7.0)
    with pytest.raises(ValueError, match="have no page"):
        w.forward(q, pages, k_append=k, v_append=v, out=out)
    torch.cuda.synchronize()
    assert _same_bits(from_torch(pages, "bf16"), sc.pages) and bool((out == 7.0).all())
    got = w.forward(q, pages).float().cpu().numpy()
    want = c_oracle.decode_attn(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                sc.kv_last_page_lens, "bf16")
    assert not got[0].any() and max_rel_err_per_request(got[1:], want[1:]) <= 2e-2
    w.end_forward()


def test_fused_append_is_refused_outside_the_mfma_shapes():
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper

    _announce("decode fused append refusal")
    sc = make_scenario(912, kv_lens=[40, 3], qo_lens=[1, 1], P=16, Hq=8, Hkv=2, D=64, dtype="f32")
    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(1 << 20, dtype=torch.uint8, device="cuda"))
    w.begin_forward(_dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                    _dev_i32(sc.kv_last_page_lens), 8, 2, 64, 16)
    assert not w.fused_append_supported(torch.float32)
    pages = to_torch(sc.pages, "f32")
    before = from_torch(pages, "f32").copy()
    with pytest.raises(ValueError, match="separately"):
        w.forward(to_torch(sc.q, "f32"), pages, k_append=to_torch(sc.k, "f32"), v_append=to_torch(sc.v, "f32"))
    torch.cuda.synchronize()
    assert _same_bits(from_torch(pages, "f32"), before)


# ------------------------------------------------------------------ mixed batches
MIXED_CASES = [
    # (name, kv_lens, qo_lens, P, Hq, Hkv, dtype, target_workgroups, rows routed to the decode kernel)
    ("decode_rows_and_chunk", [700, 33, 16, 900, 2049, 5], [1, 1, 1, 120, 1, 5], 16, 32, 8, "bf16", 0, 4),
    ("cut_rows", [4096, 3000, 257, 1500, 700], [1, 1, 1, 64, 1], 16, 32, 8, "bf16", 64, 4),
    ("chunk_first_and_last", [600, 40, 77, 1], [200, 1, 1, 1], 16, 32, 8, "bf16", 0, 3),
    ("group8_f16_page8", [3000, 2049, 64, 9], [65, 1, 1, 1], 8, 64, 8, "f16", 0, 3),
    ("only_decode_rows", [700, 33, 16, 1], [1, 1, 1, 1], 16, 32, 8, "bf16", 0, 4),
    ("row_without_kv", [0, 40, 300], [1, 1, 8], 16, 32, 8, "bf16", 0, 1),
    ("page4", [100, 37, 64], [1, 20, 1], 4, 32, 8, "f16", 0, 2),
    ("page2_mha", [50, 37, 64], [1, 20, 1], 2, 8, 8, "bf16", 0, 2),
    ("f32_generic_kernel", [100, 37, 64], [1, 20, 1], 16, 32, 8, "f32", 0, 2),
    ("group32_stays_tiled", [100, 37, 64], [1, 20, 1], 16, 32, 1, "bf16", 0, 0),
    ("many_rows", [17 * i % 900 + 1 for i in range(75)] + [4500], [1] * 75 + [437], 16, 32, 8, "bf16", 0, 75),
    # 16 kv heads: four groups of four per decode share in the shared launch; 2 kv heads: half a wave group
    ("kv16", [900, 33, 2100, 700], [1, 1, 90, 1], 16, 32, 16, "bf16", 0, 3),
    ("kv2_group16", [900, 33, 1100, 5], [1, 1, 40, 1], 16, 32, 2, "f16", 0, 3),
    ("kv1_mqa", [300, 64, 1100], [1, 1, 70], 8, 8, 1, "bf16", 0, 2),
    # a decode row cut into hundreds of parts: the shared launch then merges the decode rows with
    # eight waves per (row, head) and the tile parts in a pass of their own
    ("long_row_wide_merge", [33000, 20, 1500], [1, 1, 64], 16, 32, 8, "bf16", 0, 2),
]


@pytest.mark.parametrize("case", MIXED_CASES, ids=[c[0] for c in MIXED_CASES])
def test_mixed_batch_routes_one_row_requests_to_the_decode_kernel(case):
    """The reference's mixed step sends decode rows and a chunk through the prefill wrapper
    together (engine/microbatch/processor.py:116-145).  The wrapper computes the one-row
    requests with the split-KV decode kernel and the rest with query tiles; every row of
    the ragged output - written into a NaN-filled tensor - matches the oracle's prefill
    attention, with and without the mask, as it does with the routing switched off."""
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper

    name, kv, qo, P, Hq, Hkv, dtype, target, n_routed = case
    _announce("mixed", name, P, Hq, Hkv, dtype, target)
    sc = make_scenario(43, kv_lens=kv, qo_lens=qo, P=P, Hq=Hq, Hkv=Hkv, D=128, dtype=dtype)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(96 << 20, dtype=torch.uint8, device="cuda"))
    from deserve_amd import _lib

    q, pages = to_torch(sc.q, dtype), to_torch(sc.pages, dtype)
    tiled_rows = sum(n for n, k in zip(qo, kv) if n != 1 or k == 0)
    for route in (_lib.ROUTE_SHARED_LAUNCH, _lib.ROUTE_TWO_LAUNCHES, True, False):
        w.begin_forward(_dev_i32(sc.qo_indptr), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                        _dev_i32(sc.kv_last_page_lens), Hq, Hkv, 128, P, target_workgroups=target,
                        route_one_row_requests=route)
        shared = w._info.layout == _lib.LAYOUT_SHARED
        if route == _lib.ROUTE_SHARED_LAUNCH:
            # one launch for both kinds of rows wherever there are both and pages hold >= 4 tokens
            assert shared == (n_routed > 0 and tiled_rows > 0 and P >= 4), name
            assert w._n_decode_rows == (n_routed if shared or tiled_rows == 0 else 0)
        elif route == _lib.ROUTE_TWO_LAUNCHES:
            assert not shared and w._n_decode_rows == n_routed
        elif route is True:
            assert w._n_decode_rows in (0, n_routed)
            if name == "many_rows":
                assert shared and w._n_decode_rows == 75              # the planner's own choice for such a step
        else:
            assert not shared and w._n_decode_rows == 0
        if name == "cut_rows" and route in (_lib.ROUTE_SHARED_LAUNCH, _lib.ROUTE_TWO_LAUNCHES):
            assert w._info.n_decode_items > w._n_decode_rows          # rows cut across workgroups: merged
        if name == "long_row_wide_merge" and route in (_lib.ROUTE_SHARED_LAUNCH, _lib.ROUTE_TWO_LAUNCHES):
            assert w._info.n_decode_items > 32 * w._n_decode_rows     # dozens of parts per row: the wide merge
        for causal in (True, False):
            out = torch.full_like(q, float("nan"))
            assert w.forward(q, pages, causal=causal, out=out) is out
            torch.cuda.synchronize()
            got = out.float().cpu().numpy()
            want = c_oracle.prefill_attn(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices,
                                         sc.kv_page_indptr, sc.kv_last_page_lens, dtype, causal=causal)
            assert np.isfinite(got).all(), (name, route, causal)
            assert max_rel_err_per_request(got, want) <= ATTN_TOL[dtype], (name, route, causal, w._info.layout)
        w.end_forward()


def test_mixed_batches_random_shapes():
    """Seeded sweep over mixed batches (one-row requests with and without kv tokens, empty
    requests, chunks), page sizes of 4 to 32 tokens, kv-head counts and groups, dtypes and the
    four routing modes: every row of the NaN-filled output matches the oracle's prefill
    attention.  The sweep must meet shared launches, tiles in parts and cut decode rows."""
    from deserve_amd import _lib
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper

    rng = np.random.default_rng(79)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(128 << 20, dtype=torch.uint8, device="cuda"))
    seen = {"shared": 0, "parts": 0, "cut_rows": 0, "two_launches": 0}
    for done in range(24):
        P = int(rng.choice([4, 8, 16, 32]))
        Hkv = int(rng.choice([1, 2, 4, 8, 16]))
        Hq = Hkv * int(rng.choice([1, 2, 4, 8]))
        if Hq > 64:
            Hq = 64
        dtype = str(rng.choice(["bf16", "f16"]))
        n_req = int(rng.integers(2, 24))
        kinds = rng.choice(4, size=n_req, p=[0.7, 0.05, 0.2, 0.05])
        kinds[0] = 2                                       # at least one chunk ...
        kinds[1] = 0                                       # ... and one decode row
        qo = [1 if k in (0, 3) else 0 if k == 1 else int(rng.integers(2, 200)) for k in kinds]
        kv = [0 if k == 3 else n + int(rng.integers(0, 1500)) for k, n in zip(kinds, qo)]
        if done % 3 == 0:
            kv[0] += int(rng.integers(1500, 3000))         # a chunk behind a long context: tiles in parts
        route = [_lib.ROUTE_SHARED_LAUNCH, _lib.ROUTE_TWO_LAUNCHES, True, False][done % 4]
        target = int(rng.choice([0, 0, 48]))
        causal = bool(rng.integers(0, 2))
        _announce("mixed random", done, P, Hq, Hkv, dtype, route, target, causal, "qo", qo, "kv", kv)
        sc = make_scenario(4000 + done, kv_lens=kv, qo_lens=qo, P=P, Hq=Hq, Hkv=Hkv, D=128, dtype=dtype)
        w.begin_forward(_dev_i32(sc.qo_indptr), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                        _dev_i32(sc.kv_last_page_lens), Hq, Hkv, 128, P, target_workgroups=target,
                        route_one_row_requests=route)
        seen["shared"] += w._info.layout == _lib.LAYOUT_SHARED
        seen["two_launches"] += w._info.layout != _lib.LAYOUT_SHARED and w._n_decode_rows > 0 and w._info.n_tile_rows > 0
        seen["parts"] += w._n_splits > 1
        seen["cut_rows"] += w._info.n_decode_items > w._n_decode_rows
        q, pages = to_torch(sc.q, dtype), to_torch(sc.pages, dtype)
        out = torch.full_like(q, float("nan"))
        w.forward(q, pages, causal=causal, out=out)
        w.end_forward()
        torch.cuda.synchronize()
        got = out.float().cpu().numpy()
        want = c_oracle.prefill_attn(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                     sc.kv_last_page_lens, dtype, causal=causal)
        assert np.isfinite(got).all(), (done, route)
        assert max_rel_err_per_request(got, want) <= ATTN_TOL[dtype], (done, P, Hq, Hkv, dtype, route, qo, kv)
    assert all(v >= 2 for v in seen.values()), seen


def test_prefill_with_one_query_equals_decode():
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper

    _announce("prefill n=1 vs decode")
    sc = make_scenario(42, kv_lens=[700, 33, 16], qo_lens=[1, 1, 1], dtype="bf16")
    dec, _ = _run_decode(sc, 1)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device="cuda"))
    w.begin_forward(_dev_i32(sc.qo_indptr), _dev_i32(sc.kv_page_indptr), _dev_i32(sc.kv_page_indices),
                    _dev_i32(sc.kv_last_page_lens), sc.Hq, sc.Hkv, sc.D, sc.P)
    pre = w.forward(to_torch(sc.q, "bf16"), to_torch(sc.pages, "bf16")).float().cpu().numpy()
    assert max_rel_err_per_request(pre, dec) < 1e-2


# ------------------------------------------------------------------ rope
@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
def test_rope_matches_oracle(dtype):
    from deserve_amd.paged_ops import apply_rope

    _announce("rope", dtype)
    rng = np.random.default_rng(51)
    indptr = np.array([0, 1, 6, 6, 40], np.int32)
    offsets = np.array([511, 0, 3, 4000], np.int32)
    q = rng.standard_normal((40, 32, 128)).astype(np.float32)
    k = rng.standard_normal((40, 8, 128)).astype(np.float32)
    from kvutil import to_storage
    qs, ks = to_storage(q, dtype), to_storage(k, dtype)
    q_out, k_out = apply_rope(to_torch(qs, dtype), to_torch(ks, dtype), _dev_i32(indptr),
                              _dev_i32(offsets), interleave=True, rope_theta=500000.0)
    torch.cuda.synchronize()
    want_q = orc.rope_interleaved(orc.to_f32(qs, dtype), indptr, offsets)
    want_k = orc.rope_interleaved(orc.to_f32(ks, dtype), indptr, offsets)
    # The frequencies are the oracle's (C library powf on the host, as numpy's), the angle the same
    # fp32 product: what is left is the device's sincosf and fused multiply-adds (fp32) and half
    # an ulp of the storage type (2^-8 for bf16, 2^-11 for f16, of an element at most max|want|).
    tol = {"f32": 2e-6, "bf16": 4e-3, "f16": 6e-4}[dtype]
    assert np.abs(q_out.float().cpu().numpy() - want_q).max() <= tol * np.abs(want_q).max()
    assert np.abs(k_out.float().cpu().numpy() - want_k).max() <= tol * np.abs(want_k).max()
    with pytest.raises(ValueError):
        apply_rope(to_torch(qs, dtype), to_torch(ks, dtype), _dev_i32(indptr), _dev_i32(offsets))


@pytest.mark.parametrize("dtype,P", [("bf16", 16), ("f32", 8), ("f16", 16)])
def test_fused_rope_append_equals_rope_then_append_bitwise(dtype, P):
    from deserve_amd.paged_ops import append_paged_kv_cache, apply_rope, rope_append_paged_kv_cache

    _announce("rope+append fused", dtype, P)
    sc = make_scenario(52, kv_lens=[517, 40, 512, 3, 1029, 77], qo_lens=[512, 40, 1, 3, 0, 1], P=P,
                       dtype=dtype)
    offsets = _dev_i32(sc.kv_lens - sc.qo_lens)
    args = [_dev_i32(x) for x in (sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)]
    qo = _dev_i32(sc.qo_indptr)
    q, k, v = (to_torch(x, dtype) for x in (sc.q, sc.k, sc.v))
    pages_a, pages_b = to_torch(sc.pages, dtype), to_torch(sc.pages, dtype)
    q_a, k_a = apply_rope(q, k, qo, offsets, interleave=True, rope_theta=5e5)
    append_paged_kv_cache(k_a, v, qo, pages_a, *args)
    q_b = rope_append_paged_kv_cache(q, k, v, qo, offsets, pages_b, *args, rope_theta=5e5)
    torch.cuda.synchronize()
    assert _same_bits(from_torch(q_a, dtype), from_torch(q_b, dtype))
    assert _same_bits(from_torch(pages_a, dtype), from_torch(pages_b, dtype))
    assert not _same_bits(from_torch(pages_a, dtype), sc.pages)


# ------------------------------------------------------------------ config 1 of the baseline, exactly
def test_baseline_config1_fp32_append_then_decode():
    """8 sequences, context 512 after the append, 256-page pool in a seeded random
    permutation, fp32, 32 q heads / 8 kv heads / head_dim 128, page size 16."""
    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper, append_paged_kv_cache

    _announce("config1")
    sc = make_scenario(1, kv_lens=[512] * 8, qo_lens=[1] * 8, dtype="f32", spare_pages=0)
    assert sc.num_pages == 256
    want_pages = sc.pages.copy()
    orc.append_paged_kv(want_pages, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                        sc.kv_last_page_lens)
    want = orc.decode_attention(sc.q, want_pages, sc.kv_page_indices, sc.kv_page_indptr,
                                sc.kv_last_page_lens, "f32")
    pages = to_torch(sc.pages, "f32")
    args = [_dev_i32(x) for x in (sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)]
    append_paged_kv_cache(to_torch(sc.k, "f32"), to_torch(sc.v, "f32"), args[0], pages, args[1], args[2], args[3])
    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(16 << 20, dtype=torch.uint8, device="cuda"))
    w.begin_forward(args[2], args[1], args[3], 32, 8, 128, 16)
    got = w.forward(to_torch(sc.q, "f32"), pages).cpu().numpy()
    assert _same_bits(from_torch(pages, "f32"), want_pages)
    assert max_rel_err_per_request(got, want) <= 1e-4
    # the same problem in bf16 storage stays within the 16-bit tolerance of the fp32 answer
    scb = make_scenario(1, kv_lens=[512] * 8, qo_lens=[1] * 8, dtype="bf16", spare_pages=0)
    got_b, _ = _run_decode(scb)
    want_b = orc.decode_attention(scb.q, scb.pages, scb.kv_page_indices, scb.kv_page_indptr,
                                  scb.kv_last_page_lens, "bf16")
    assert max_rel_err_per_request(got_b, want_b) <= 2e-2

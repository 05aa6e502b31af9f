"""Pins the data-path oracle (numpy kv_oracle.py and scalar C kv_oracle.c) without
the GPU: brute force on tiny inputs, library routines, closed forms and
invariants chosen so that a dropped term, a wrong index or a transposed operand
fails at least one of them; plus the committed golden file."""
import math
import os

import numpy as np
import pytest
from scipy.special import softmax

from kvutil import make_scenario
from oracle import c_oracle
from oracle import kv_oracle as orc


def _positions(sc, b):
    """(page, slot) of every kv position of request b, by direct table walk."""
    ids = sc.kv_page_indices[sc.kv_page_indptr[b]: sc.kv_page_indptr[b + 1]]
    return [(int(ids[t // sc.P]), t % sc.P) for t in range(int(sc.kv_lens[b]))]


# ------------------------------------------------------------------ append
@pytest.mark.parametrize("dtype", ["f32", "bf16"])
def test_append_brute_force_and_untouched_bytes(dtype):
    sc = make_scenario(1, kv_lens=[5, 16, 33, 1, 20], qo_lens=[1, 16, 7, 1, 0], P=4, Hq=4, Hkv=2,
                       D=8, dtype=dtype)
    before = sc.pages.copy()
    got_np, got_c = sc.pages.copy(), sc.pages.copy()
    orc.append_paged_kv(got_np, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                        sc.kv_last_page_lens)
    c_oracle.append(got_c, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                    sc.kv_last_page_lens, dtype)
    # independent expectation: token i of request b is position kv_len - n + i
    want = before.copy()
    touched = np.zeros(before.shape[:3], dtype=bool)
    for b in range(len(sc.kv_lens)):
        pos = _positions(sc, b)
        n = int(sc.qo_lens[b])
        for i in range(n):
            page, slot = pos[len(pos) - n + i]
            want[page, 0, slot] = sc.k[sc.qo_indptr[b] + i]
            want[page, 1, slot] = sc.v[sc.qo_indptr[b] + i]
            touched[page, :, slot] = True
    assert np.array_equal(got_np, want) and np.array_equal(got_c, want)
    assert np.array_equal(got_np[~touched], before[~touched])      # canary: nothing else moved
    assert touched.sum() == 2 * sc.qo_lens.sum()


def test_append_then_read_back_through_table_returns_the_new_rows():
    sc = make_scenario(2, kv_lens=[37, 9], qo_lens=[10, 9], P=8, Hq=2, Hkv=2, D=4, dtype="f32")
    orc.append_paged_kv(sc.pages, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                        sc.kv_last_page_lens)
    for b in range(2):
        pos = _positions(sc, b)[-int(sc.qo_lens[b]):]
        rows = np.stack([sc.pages[p, 0, s] for p, s in pos])
        assert np.array_equal(rows, sc.k[sc.qo_indptr[b]: sc.qo_indptr[b + 1]])


# ------------------------------------------------------- gather / scatter / swap
def test_gather_scatter_equal_numpy_take_and_round_trip():
    rng = np.random.default_rng(3)
    pool = rng.integers(0, 2**16, size=(3, 11, 2, 4, 2, 8), dtype=np.uint16)
    ids = np.array([7, 0, 10, 3], dtype=np.int32)
    want = np.stack([pool[l, i] for l in range(3) for i in ids])            # layer major, table order
    assert np.array_equal(orc.gather_pages(pool, ids), want)
    assert np.array_equal(c_oracle.gather(pool, ids), want)
    for scatter in (orc.scatter_pages, c_oracle.scatter):
        dst = np.zeros_like(pool)
        scatter(dst, ids, want)
        assert np.array_equal(dst[:, ids], pool[:, ids])
        mask = np.ones(11, bool)
        mask[ids] = False
        assert not dst[:, mask].any()                                        # other pages untouched
    # a chunk larger than needed (buddy chunks are powers of two) is read only at its head
    big = np.concatenate([want, np.full_like(want, 9)])
    dst = np.zeros_like(pool)
    orc.scatter_pages(dst, ids, big)
    assert np.array_equal(dst[:, ids], pool[:, ids])


def test_swap_slice_layout_and_round_trip():
    rng = np.random.default_rng(4)
    L, n, S = 2, 10, 3
    pool = rng.integers(0, 2**16, size=(L, n, 2, 2, 1, 4), dtype=np.uint16)
    orig = pool.copy()
    page_elems = 2 * 2 * 1 * 4
    a = np.zeros(L * S * page_elems, np.uint16)
    b = rng.integers(0, 2**16, size=L * S * page_elems, dtype=np.uint16)
    b0 = b.copy()
    orc.swap_slice(pool, (4, 7), a, b)
    assert np.array_equal(a.reshape(L, S, -1), orig[:, 4:7].reshape(L, S, -1))   # (L, S, ...) image
    assert np.array_equal(pool[:, 4:7].reshape(L, S, -1), b0.reshape(L, S, -1))
    assert np.array_equal(pool[:, :4], orig[:, :4]) and np.array_equal(pool[:, 7:], orig[:, 7:])
    orc.swap_slice(pool, (4, 7), b, a)                                           # swap back
    assert np.array_equal(pool, orig) and np.array_equal(b, b0)
    same = a.copy()
    orc.swap_slice(pool, (4, 7), same, same)      # two rounds share one buffer: slice unchanged
    assert np.array_equal(pool, orig)


# ------------------------------------------------------------------ attention
def _dense_reference(sc, b, q_rows, limits):
    """softmax(q k^T / sqrt(D)) v with scipy/numpy on explicitly gathered K, V."""
    pos = _positions(sc, b)
    pf = orc.to_f32(sc.pages, sc.dtype)
    K = np.stack([pf[p, 0, s] for p, s in pos])          # (T, Hkv, D)
    V = np.stack([pf[p, 1, s] for p, s in pos])
    rep = sc.Hq // sc.Hkv
    out = np.zeros((len(q_rows), sc.Hq, sc.D), np.float32)
    qf = orc.to_f32(sc.q, sc.dtype)
    for r, (row, lim) in enumerate(zip(q_rows, limits)):
        for h in range(sc.Hq):
            s = K[:lim, h // rep] @ qf[row, h] / math.sqrt(sc.D)
            out[r, h] = softmax(s.astype(np.float64)) @ V[:lim, h // rep]
    return out


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_decode_attention_against_scipy_dense_and_c_port(dtype):
    sc = make_scenario(5, kv_lens=[1, 4, 5, 23, 16], qo_lens=[1] * 5, P=4, Hq=6, Hkv=2, D=16, dtype=dtype)
    got = orc.decode_attention(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                               sc.kv_last_page_lens, dtype)
    got_c = c_oracle.decode_attn(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                 sc.kv_last_page_lens, dtype)
    for b in range(5):
        want = _dense_reference(sc, b, [b], [int(sc.kv_lens[b])])[0]
        assert np.allclose(got[b], want, rtol=2e-5, atol=2e-6)
        assert np.allclose(got_c[b], want, rtol=2e-5, atol=2e-6)


def test_decode_attention_closed_forms():
    # kv_len 1: the output is that token's V row, whatever q and k are
    sc = make_scenario(6, kv_lens=[1, 1], qo_lens=[1, 1], P=4, Hq=4, Hkv=2, D=8, dtype="f32")
    out = orc.decode_attention(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)
    for b in range(2):
        page = sc.kv_page_indices[sc.kv_page_indptr[b]]
        assert np.allclose(out[b], np.repeat(sc.pages[page, 1, 0], 2, axis=0), atol=1e-6)
    # all keys equal: uniform weights, output = mean of V over the valid tokens only
    sc = make_scenario(7, kv_lens=[11], qo_lens=[1], P=4, Hq=4, Hkv=2, D=8, dtype="f32")
    sc.pages[:, 0] = 0.25
    out = orc.decode_attention(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)
    pos = _positions(sc, 0)
    mean_v = np.mean([sc.pages[p, 1, s] for p, s in pos], axis=0)           # (Hkv, D)
    assert np.allclose(out[0], np.repeat(mean_v, 2, axis=0), atol=1e-6)
    # one dominant key: output ~ that token's V; checks the GQA map h -> h // rep
    sc = make_scenario(8, kv_lens=[9], qo_lens=[1], P=4, Hq=4, Hkv=2, D=8, dtype="f32")
    sc.pages[:, 0] = 0.0
    page, slot = _positions(sc, 0)[6]
    sc.q[0] = 1.0
    sc.pages[page, 0, slot, 1] = 100.0            # only kv head 1 has a dominant key
    out = orc.decode_attention(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)
    assert np.allclose(out[0, 2:], np.repeat(sc.pages[page, 1, slot, 1:2], 2, axis=0), atol=1e-5)
    mean_v0 = np.mean([sc.pages[p, 1, s, 0] for p, s in _positions(sc, 0)], axis=0)
    assert np.allclose(out[0, :2], np.stack([mean_v0, mean_v0]), atol=1e-5)     # kv head 0: uniform


def test_decode_attention_invariant_under_page_permutation_and_scale_argument():
    sc = make_scenario(9, kv_lens=[19, 7], qo_lens=[1, 1], P=4, Hq=4, Hkv=4, D=8, dtype="f32")
    base = orc.decode_attention(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)
    perm = np.random.default_rng(0).permutation(sc.num_pages)
    moved = np.empty_like(sc.pages)
    moved[perm] = sc.pages                            # page i now lives at perm[i]
    out = orc.decode_attention(sc.q, moved, perm[sc.kv_page_indices].astype(np.int32),
                               sc.kv_page_indptr, sc.kv_last_page_lens)
    assert np.array_equal(out, base)
    # sm_scale is applied to the scores: doubling q equals doubling the scale
    twice = orc.decode_attention(sc.q * 2, sc.pages, sc.kv_page_indices, sc.kv_page_indptr, sc.kv_last_page_lens)
    scaled = orc.decode_attention(sc.q, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                  sc.kv_last_page_lens, sm_scale=2 / math.sqrt(8))
    assert np.allclose(twice, scaled, atol=1e-6)


def test_prefill_attention_causal_mask_is_end_aligned():
    sc = make_scenario(10, kv_lens=[13, 6, 9], qo_lens=[5, 6, 1], P=4, Hq=4, Hkv=2, D=8, dtype="f32")
    got = orc.prefill_attention(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                sc.kv_last_page_lens)
    got_c = c_oracle.prefill_attn(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                                  sc.kv_last_page_lens, "f32")
    for b in range(3):
        n, T = int(sc.qo_lens[b]), int(sc.kv_lens[b])
        rows = list(range(sc.qo_indptr[b], sc.qo_indptr[b + 1]))
        want = _dense_reference(sc, b, rows, [T - n + i + 1 for i in range(n)])
        assert np.allclose(got[rows], want, rtol=2e-5, atol=2e-6)
        assert np.allclose(got_c[rows], want, rtol=2e-5, atol=2e-6)
    # request 1 is a pure prompt (n == kv_len): first query sees only token 0 -> V row 0
    page, slot = _positions(sc, 1)[0]
    assert np.allclose(got[sc.qo_indptr[1]], np.repeat(sc.pages[page, 1, slot], 2, axis=0), atol=1e-6)
    # one query per request is exactly decode attention
    one = make_scenario(11, kv_lens=[13, 6], qo_lens=[1, 1], P=4, Hq=4, Hkv=2, D=8, dtype="f32")
    a = orc.prefill_attention(one.q, one.qo_indptr, one.pages, one.kv_page_indices,
                              one.kv_page_indptr, one.kv_last_page_lens)
    b_ = orc.decode_attention(one.q, one.pages, one.kv_page_indices, one.kv_page_indptr, one.kv_last_page_lens)
    assert np.allclose(a, b_, atol=1e-6)
    # non-causal: every query sees everything
    nc = orc.prefill_attention(sc.q, sc.qo_indptr, sc.pages, sc.kv_page_indices, sc.kv_page_indptr,
                               sc.kv_last_page_lens, causal=False)
    want = _dense_reference(sc, 0, list(range(5)), [13] * 5)
    assert np.allclose(nc[:5], want, rtol=2e-5, atol=2e-6)


def test_attention_matches_committed_golden_file():
    g = np.load(os.path.join(os.path.dirname(__file__), "golden", "attention_small.npz"))
    d = orc.decode_attention(g["d_q"], g["d_pages"], g["d_indices"], g["d_indptr"], g["d_last"])
    assert np.allclose(d, g["d_out"], rtol=1e-6, atol=1e-7)
    dc = c_oracle.decode_attn(g["d_q"], g["d_pages"], g["d_indices"], g["d_indptr"], g["d_last"], "f32")
    assert np.allclose(dc, g["d_out"], rtol=2e-5, atol=2e-6)
    p = orc.prefill_attention(g["p_q"], g["p_qo"], g["p_pages"], g["p_indices"], g["p_indptr"], g["p_last"])
    assert np.allclose(p, g["p_out"], rtol=1e-6, atol=1e-7)


# ------------------------------------------------------------------ 16-bit helpers and rope
def test_bf16_round_trip_and_rounding():
    x = np.array([1.0, -2.5, 3.140625, 1e-3, 65504.0, 0.0], np.float32)
    bits = orc.bf16_bits_from_f32(x)
    back = orc.f32_from_bf16_bits(bits)
    assert np.all(np.abs(back - x) <= np.abs(x) * 2.0 ** -8)
    assert np.array_equal(orc.bf16_bits_from_f32(back), bits)                 # idempotent
    # ties to even: 1 + 2^-8 is exactly half way between 1 and 1 + 2^-7
    assert orc.f32_from_bf16_bits(orc.bf16_bits_from_f32(np.float32([1 + 2.0 ** -8])))[0] == 1.0
    assert orc.f32_from_bf16_bits(orc.bf16_bits_from_f32(np.float32([1 + 3 * 2.0 ** -8])))[0] == np.float32(1 + 2.0 ** -6)
    import torch
    t = torch.randn(1000, dtype=torch.float32)
    assert np.array_equal(orc.bf16_bits_from_f32(t.numpy()),
                          t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16))


def test_rope_is_complex_multiplication_by_unit_phasors():
    rng = np.random.default_rng(12)
    x = rng.standard_normal((5, 3, 16)).astype(np.float32)
    indptr, offsets = np.array([0, 2, 5], np.int32), np.array([7, 100], np.int32)
    got = orc.rope_interleaved(x, indptr, offsets, theta=500000.0)
    pos = np.array([7, 8, 100, 101, 102])
    freqs = 1.0 / (500000.0 ** (np.arange(0, 16, 2) / 16))
    z = (x[..., 0::2] + 1j * x[..., 1::2]) * np.exp(1j * pos[:, None, None] * freqs[None, None, :])
    assert np.allclose(got[..., 0::2], z.real, atol=2e-4) and np.allclose(got[..., 1::2], z.imag, atol=2e-4)
    assert np.allclose(np.linalg.norm(got, axis=-1), np.linalg.norm(x, axis=-1), rtol=1e-5)  # rotation
    zero = orc.rope_interleaved(x, np.array([0, 5], np.int32), np.array([0], np.int32))
    assert np.allclose(zero[0], x[0], atol=1e-7)                               # position 0: identity


def test_torch_cpu_path_matches_the_numpy_oracle_on_config1_shape():
    """oracle/torch_cpu_path.py (the reference's host path restated with torch: index-assign
    append, pages[layer, table] gather, repeat_kv + softmax(scores.float()) matmuls) against
    the numpy oracle: same pages after the append bit for bit, same attention within fp32
    rounding.  A wrong GQA map, slot or gather order fails here."""
    import torch

    from oracle import torch_cpu_path

    sc = make_scenario(1, kv_lens=[512, 33, 16, 1, 100], qo_lens=[1] * 5, dtype="f32", spare_pages=3)
    want_pages = sc.pages.copy()
    orc.append_paged_kv(want_pages, sc.k, sc.v, sc.qo_indptr, sc.kv_page_indices, sc.kv_page_indptr,
                        sc.kv_last_page_lens)
    want = orc.decode_attention(sc.q, want_pages, sc.kv_page_indices, sc.kv_page_indptr,
                                sc.kv_last_page_lens, "f32")
    pages = torch.from_numpy(np.stack([np.zeros_like(sc.pages), sc.pages.copy()]))      # layer 1 of 2
    tables = [torch.from_numpy(sc.kv_page_indices[sc.kv_page_indptr[b]: sc.kv_page_indptr[b + 1]].astype(np.int64))
              for b in range(5)]
    got = torch_cpu_path.decode_step(pages, 1, tables, [int(n) for n in sc.kv_lens], torch.from_numpy(sc.q),
                                     torch.from_numpy(sc.k), torch.from_numpy(sc.v))
    assert np.array_equal(pages[1].numpy(), want_pages) and not pages[0].any()
    assert got.shape == (5, sc.Hq, sc.D)
    for b in range(5):
        assert np.abs(got[b].numpy() - want[b]).max() <= 1e-5 * np.abs(want[b]).max(), b

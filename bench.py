#!/usr/bin/env python3
"""Benchmark of the KV-cache hot path of one Llama-3-8B pipeline stage on one MI355X.

Workload (baseline configuration 2): 16 layers, bf16, GQA 32 q / 8 kv heads,
head_dim 128, page size 16, decode batch of 64 sequences with context lengths
seeded uniform in [256, 4096], pages scattered over the pool by a seeded
permutation, K/V ~ N(0, 1).  One step = build the step's metadata and attention
plan on the host, then per layer: append 1 token per sequence and run paged
decode attention.  Inputs are resident in HBM before the timed region.

Prints ONE JSON line.  `value` is the algorithmic KV bytes one step moves
(append + decode attention, every layer) divided by the wall time of a step.
`roofline` is for the dominant kernel (the split-KV decode attention pass),
timed with events on the launch stream inside the timed region.
`cpu_baseline` times the scalar C port of the same maths (OpenMP over
request x head) on a bounded sample, on this box's host cores.
"""
from __future__ import annotations

import argparse
import gc
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0
MFMA_PEAK_BF16_TFLOPS = 2500.0


def settle_heap():
    """A full collection of the Python heap takes 20-40 ms in this process (170 k tracked
    objects): one that happens to fall into a timed loop starves the GPU for that long.
    Collect now and move what exists out of the collector's reach, as a long-running engine
    does after start-up; what the steps allocate is still collected (cheaply)."""
    gc.collect()
    gc.freeze()


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--seed", type=int, default=2)
    ap.add_argument("--workgroups", type=int, default=0, help="persistent workgroups of the attention pass (0 = one per CU)")
    ap.add_argument("--rope", action="store_true", help="also rotate q and k (RoPE) in the step")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-swap", action="store_true", help="skip the microbatch swap section")
    ap.add_argument("--no-prefill", action="store_true", help="skip the chunked-prefill section")
    ap.add_argument("--no-fragmented", action="store_true", help="skip the fragmented long-context section")
    ap.add_argument("--no-fused-append", action="store_true",
                    help="append with a launch of its own instead of inside the attention launch")
    ap.add_argument("--steps-in-flight", type=int, default=2,
                    help="steps the host may have queued on the GPU (a stage hands every step's "
                         "output on before it starts the next but one); 0 = no limit")
    ap.add_argument("--no-rope-step", action="store_true", help="skip the extra steps with rotation")
    ap.add_argument("--no-graph", action="store_true", help="skip the replayed-graph variant of the step")
    ap.add_argument("--no-mixed", action="store_true", help="skip the mixed decode + chunk section")
    ap.add_argument("--no-page8", action="store_true", help="skip configuration 2 on 8-token pages")
    ap.add_argument("--section", choices=["swap", "fragmented", "prefill", "mixed", "mfma-ceiling", "power"],
                    default=None,
                    help="(internal) run only this host-link section and print its JSON object")
    ap.add_argument("--page-size", type=int, default=16,
                    help="tokens per page of the benched pool (BASELINE's configurations use 16; the "
                         "reference deploys with 8, worker_api.py:170)")
    ap.add_argument("--prefill-one-chunk-only", action="store_true",
                    help="with --section prefill: only the 512-token chunk over 4096 prior tokens "
                         "(12 launches with parts, 12 with whole tiles), for profiler runs")
    ap.add_argument("--prefill-config4-only", action="store_true",
                    help="with --section prefill: only configuration 4's launches on its own data "
                         "(20 appends, 20 attention launches), for profiler runs whose per-kernel "
                         "averages must not mix in the zero-data and one-chunk measurements")
    ap.add_argument("--mixed-shapes", default="8B,70B,8B_chunk_behind_8000",
                    help="with --section mixed: which cases to run (8B, 70B, 8B_chunk_behind_8000)")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="before the timed region run one plain page-copy kernel of known size "
                         "(256 MiB read + 256 MiB written) so counter runs can be scaled by it")
    ap.add_argument("--no-kernel-events", action="store_true",
                    help="do not bracket the attention pass with events (pure step timing)")
    ap.add_argument("--event-every", type=int, default=17,
                    help="bracket every Nth attention launch with events; the host must stay ahead "
                         "of the GPU for the event interval to be the kernel alone, so not every "
                         "launch is bracketed")
    return ap.parse_args()


def attention_bytes_per_layer(kv_lens, n_pages_total, batch, hq, d, e, kv_token_bytes) -> int:
    """sum_b kv_len_b * 2*Hkv*D*e  +  Q read and O write  +  block-table entries."""
    return int(kv_lens.sum()) * kv_token_bytes + 2 * batch * hq * d * e + 4 * int(n_pages_total)


def append_bytes_per_layer(nnz, batch, n_pages_total, kv_token_bytes) -> int:
    """read the new K, V rows and write them, plus the int32 metadata."""
    return 2 * nnz * kv_token_bytes + 4 * (3 * batch + 2 + int(n_pages_total))


def cpu_baseline(wl, meta, sample_requests: int):
    """Scalar C port (oracle/kv_oracle.c) of append + decode attention for ONE layer of
    the first `sample_requests` requests of the same workload, on the host cores."""
    import numpy as np

    from oracle import c_oracle

    c_oracle.load()
    B = sample_requests
    indptr = meta["kv_page_indptr"][: B + 1].astype(np.int32)
    ids = meta["kv_page_indices"][: indptr[-1]].astype(np.int32)
    last = meta["kv_last_page_lens"][:B].astype(np.int32)
    # compact copy of the sample's pages (bf16 bits) so the host holds MBs, not the pool
    import torch

    sel = torch.from_numpy(ids.astype(np.int64)).to(wl.pool.pages.device)
    pages = wl.pool.pages[0].index_select(0, sel).cpu().view(torch.int16).numpy().view(np.uint16)
    local_ids = np.arange(len(ids), dtype=np.int32)
    as_bits = lambda t: t.cpu().contiguous().view(torch.int16).numpy().view(np.uint16)
    q, k, v = as_bits(wl.q[0, :B]), as_bits(wl.k[0, :B]), as_bits(wl.v[0, :B])
    qo = np.arange(B + 1, dtype=np.int32)
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    P = wl.args.page_size
    kv_lens = (np.diff(indptr) - 1) * P + last
    tok_bytes = wl.kv_bytes_per_token()
    nbytes = attention_bytes_per_layer(kv_lens, len(ids), B, wl.args.n_heads, 128, 2, tok_bytes) + \
        append_bytes_per_layer(B, B, len(ids), tok_bytes)
    times = []
    t_end = time.time() + 20.0
    while len(times) < 3 or (time.time() < t_end and len(times) < 20):
        t0 = time.perf_counter()
        c_oracle.append(pages, k, v, qo, local_ids, indptr, last, "bf16")
        c_oracle.decode_attn(q, pages, local_ids, indptr, last, "bf16")
        times.append(time.perf_counter() - t0)
    med = sorted(times)[len(times) // 2]
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": threads, "kind": "port",
            "sample": f"1 of {wl.args.n_layers} layers, first {B} of {wl.batch} sequences "
                      f"({int(kv_lens.sum())} kv tokens), median of {len(times)} runs, "
                      f"{med * 1e3:.1f} ms each, scalar C + OpenMP"}


def cpu_reference_config1(seed: int):
    """BASELINE.json configs[0] exactly, on the reference's CPU path restated with torch
    (oracle/torch_cpu_path.py): one layer, fp32, 32 q / 8 kv heads, head_dim 128, page 16, 8
    sequences of context 512 after the append, block tables = a seeded random permutation of
    the 256 pool pages, K/V/Q ~ N(0, 1).  One step = index-assign append of 1 token per
    sequence, pages[layer, table] gather, repeat_kv + softmax(scores.float()) matmuls.  Warm-up,
    then the median of 30 steps on all host threads; the HIP path (append kernel + decode
    attention, fp32 pool) runs the same step beside it and is compared with the CPU output."""
    import numpy as np
    import torch

    from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper, append_paged_kv_cache
    from oracle import torch_cpu_path

    L, Hq, Hkv, D, P, B, N = 1, 32, 8, 128, 16, 8, 512
    g = torch.Generator().manual_seed(seed + 10)
    pages = torch.randn((L, 256, 2, P, Hkv, D), generator=g)             # CpuPagePool storage, 32 MiB
    perm = torch.randperm(256, generator=g)
    tables = [perm[b * 32: (b + 1) * 32].clone() for b in range(B)]
    q, k, v = (torch.randn((B, h, D), generator=g) for h in (Hq, Hkv, Hkv))
    kv_lens = [N] * B
    threads = torch.get_num_threads()
    for _ in range(5):
        out_cpu = torch_cpu_path.decode_step(pages, 0, tables, kv_lens, q, k, v)
    times = []
    for _ in range(30):
        t0 = time.perf_counter()
        out_cpu = torch_cpu_path.decode_step(pages, 0, tables, kv_lens, q, k, v)
        times.append(time.perf_counter() - t0)
    cpu_s = sorted(times)[len(times) // 2]
    tok_bytes = 2 * Hkv * D * 4
    nbytes = attention_bytes_per_layer(np.array(kv_lens), 256, B, Hq, D, 4, tok_bytes) + \
        append_bytes_per_layer(B, B, 256, tok_bytes)

    dev = torch.device("cuda")
    d_pages = pages[0].to(dev)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    qo, kv_indptr, last = i32(list(range(B + 1))), i32([32 * b for b in range(B + 1)]), i32([P] * B)
    ids = perm.to(torch.int32).to(dev)
    dq, dk, dv = q.to(dev), k.to(dev), v.to(dev)
    w = BatchDecodeWithPagedKVCacheWrapper(torch.empty(16 << 20, dtype=torch.uint8, device=dev))
    w.begin_forward(kv_indptr, ids, last, Hq, Hkv, D, P)

    def hip_step():
        append_paged_kv_cache(dk, dv, qo, d_pages, ids, kv_indptr, last)
        return w.forward(dq, d_pages)

    for _ in range(5):
        out_hip = hip_step()
    evs = []
    for _ in range(30):
        a_, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a_.record()
        out_hip = hip_step()
        b_.record()
        evs.append((a_, b_))
    torch.cuda.synchronize()
    w.end_forward()
    hip_s = sorted(x.elapsed_time(y) for x, y in evs)[len(evs) // 2] * 1e-3
    got, want = out_hip.cpu().numpy(), out_cpu.numpy()
    err = max(float(np.abs(got[b] - want[b]).max() / np.abs(want[b]).max()) for b in range(B))
    same_pages = bool(torch.equal(d_pages.cpu(), pages[0]))
    return {"value": round(nbytes / cpu_s / 1e9, 3), "unit": "GB/s", "cores": threads,
            "kind": "port", "config": "configs[0]",
            "sample": f"BASELINE.json configs[0] exactly: 1 layer fp32, 8 x 512 tokens after the append, 256-page "
                      f"pool in a seeded permutation; torch CPU ({threads} threads): index-assign append, "
                      f"pages[layer, table] gather, repeat_kv + softmax(scores.float()) matmuls; median of 30 "
                      f"steps after 5 warm-up steps, {cpu_s * 1e3:.3f} ms per step",
            "ms_per_step": round(cpu_s * 1e3, 4), "algorithmic_bytes_per_step": int(nbytes),
            "hip_same_config": {"us_per_step": round(hip_s * 1e6, 1), "GBps": round(nbytes / hip_s / 1e9, 1),
                                "speedup_over_cpu": round(cpu_s / hip_s, 1),
                                "max_rel_err_vs_cpu_per_request": float(f"{err:.2e}"),
                                "pages_bit_equal": same_pages,
                                "note": "append kernel + fp32 decode attention + merge, events on the launch "
                                        "stream; 32 MiB of KV is launch- and latency-bound on 256 CUs"}}


def swap_section(seed: int):
    """Baseline configuration 3 (Llama-3-70B stage, 10 layers, GQA 64q/8kv): one microbatch's
    scattered pages go out to pinned host memory while the next one's come in (one
    exchange call), overlapped with decode steps of the resident microbatch."""
    import numpy as np
    import torch

    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.synthetic import make_decode_workload

    L, Hq, Hkv, D, P = 10, 64, 8, 128, 16
    rng = np.random.default_rng(seed + 30)
    ctx = rng.integers(1024, 4097, size=32)                 # resident microbatch
    other = rng.integers(1024, 4097, size=32)               # the microbatch being exchanged
    n_swap = int((-(-other // P)).sum())
    wl = make_decode_workload("cfg3", ctx, L, Hq, Hkv, D, P, torch.bfloat16, headroom_tokens=512,
                              seed=seed, spare_pages=n_swap + 64, fill=False)
    wl.pool.pages.zero_()
    ids = wl.pool.alloc(n_swap)                             # scattered: the pool hands out a permutation
    shape = (L * n_swap,) + tuple(wl.pool.pages.shape[2:])
    host_out, host_in = pinned_empty(shape, torch.bfloat16), pinned_empty(shape, torch.bfloat16)
    host_in.zero_()
    nbytes = host_out.numel() * 2
    # staging for the whole microbatch (2 x 3 GB of the 288 GB): one gather before the trip
    # out and one scatter after the trip in, nothing but the copy engines in between
    staging_mib = int(os.environ.get("DSKV_BENCH_SWAP_STAGING_MIB", str(-(-nbytes // (1 << 20)))))
    eng = _native.SwapEngine(staging_mib << 20)
    w, _ = get_wrappers(wl.pool.main_device)
    settle_heap()

    def decode_step():
        FlashDecodeCtx.init_and_plan(wl.tasks, wl.caches, w, Hq, Hkv, D, P)
        for layer in range(L):
            pages = wl.pool.get_layered_pages(layer)
            w.forward(wl.q[layer], pages, k_append=wl.k[layer], v_append=wl.v[layer])
        w.end_forward()
        for t in wl.tasks:
            t.step()

    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    # host-link denominator: plain pinned copies of the same size, both directions at once,
    # on the engine's own two streams (the process creates no further stream)
    dev_a = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    dev_b = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    s_out, s_in = eng.streams()
    import ctypes
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpyAsync.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]

    def raw_duplex():
        # 2 = device to host, 1 = host to device; raw calls: torch's pinned-memory allocator
        # must not learn of streams that the engine destroys before the buffers are freed
        assert hip.hipMemcpyAsync(host_out.data_ptr(), dev_a.data_ptr(), nbytes, 2, s_out) == 0
        assert hip.hipMemcpyAsync(dev_b.data_ptr(), host_in.data_ptr(), nbytes, 1, s_in) == 0

    raw_duplex()
    link = nbytes / min(timed(raw_duplex) for _ in range(2)) / 1e9
    del dev_a, dev_b

    def exchange():
        eng.exchange(host_out, host_in, wl.pool, ids)
        eng.wait()

    exchange()
    alone = nbytes / min(timed(exchange) for _ in range(2)) / 1e9
    for _ in range(3):
        decode_step()
    t_dec = timed(lambda: [decode_step() for _ in range(20)]) / 20

    # overlapped: start the exchange, decode until it has finished.  A stage hands every
    # step's output on before it starts the next but one: at most two steps are queued on
    # the GPU at any time.  Three exchanges in a row; all three are reported.
    runs = []
    for _ in range(3):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.exchange(host_out, host_in, wl.pool, ids)
        steps = 0
        in_flight = [torch.cuda.Event(), torch.cuda.Event()]
        while not eng.done():
            if steps >= 2:
                in_flight[steps % 2].synchronize()
            decode_step()
            in_flight[steps % 2].record()
            steps += 1
        t_swap = time.perf_counter() - t0
        torch.cuda.synchronize()
        t_all = time.perf_counter() - t0
        runs.append((nbytes / t_swap / 1e9, t_all / max(steps, 1) * 1e3, steps))
    independent = eng.independent
    eng.close()
    rate = sorted(r[0] for r in runs)
    step_ms = sorted(r[1] for r in runs)
    return {"workload": "BASELINE.json configs[2]: 10 layers, bf16, GQA 64q/8kv, page 16, microbatch of 32 "
                        "sequences ctx U[1024,4096]; scattered pages out + next microbatch in, one exchange",
            "pages": n_swap, "bytes_each_way": nbytes,
            "host_link_duplex_GBps_each_way": round(link, 2),
            "exchange_alone_GBps_each_way": round(alone, 2),
            "exchange_overlapped_GBps_each_way": round(rate[1], 2),
            "exchange_overlapped_GBps_min_max": [round(rate[0], 2), round(rate[-1], 2)],
            "frac_of_host_link_overlapped": round(rate[1] / link, 3),
            "decode_ms_per_step_alone": round(t_dec * 1e3, 3),
            "decode_ms_per_step_during_swap": round(step_ms[1], 3),
            "decode_ms_per_step_during_swap_min_max": [round(step_ms[0], 3), round(step_ms[-1], 3)],
            "decode_slowdown": round(step_ms[1] / (t_dec * 1e3) - 1.0, 3),
            "decode_steps_during_swap": [r[2] for r in runs],
            "staging_MiB": staging_mib,
            "streams_run_beside_compute": independent}


def prefill_section(seed: int, extras: bool = True, config4: bool = True):
    """Baseline configuration 4 (Llama-3-8B stage): 16 sequences each append a 512-token chunk
    at a start offset U[0,15] inside a partially filled page and attend over a prior context
    U[0,8192].  Timed per layer on the launch stream: the chunk append and the paged prefill
    attention (4 layers of the stage's 16 are allocated; the layers are identical work)."""
    import numpy as np
    import torch

    from deserve_amd.kvcache.paged.kvcache import PagedKVCache
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.model.context.flash import FlashPrefillCtx
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper, append_paged_kv_cache
    from deserve_amd.synthetic import fill_normal, scatter_pool_order
    from deserve_amd.task import SamplingParams, TaskData

    dev = torch.device("cuda")
    L, P, Hq, Hkv, D, B, n = 4, 16, 32, 8, 128, 16, 512

    def one_chunk_measure(gen):
        # One 512-token chunk over 4096 prior tokens: the step budget of the reference's scheduler
        # (engine/pipeline/scheduler.py:74,85).  8 query tiles x 8 kv heads are 64 workgroups, so
        # the plan cuts every tile's K/V range into parts (merged by a second pass); timed with
        # that plan and with whole tiles.
        one_prior = 4096
        one_pool = GpuPagePool(2, (one_prior + n) // P + 8, P, dev, torch.bfloat16)
        fill_normal(one_pool.pages, seed + 44)
        one_rows = PageTableAllocator(1, one_prior + 1024, P, dev)
        one_task = [TaskData("p_one", one_prior, 1, n, one_prior + n, SamplingParams())]
        one_cache = [PagedKVCache.empty(one_rows, one_pool)]
        one_w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(64 << 20, dtype=torch.uint8, device=dev))
        one_c = FlashPrefillCtx.init_paged_prefill_ctx(one_task, one_cache, one_w)
        one_q = torch.randn((2, n, Hq, D), device=dev, generator=gen).to(torch.bfloat16)
        one_chunk = {}
        for label, target in (("parts", 0), ("whole_tiles", -1)):
            one_w.begin_forward(qo_indptr=one_c.indptr, paged_kv_indptr=one_c.kv_page_indptr,
                                paged_kv_indices=one_c.kv_page_indices,
                                paged_kv_last_page_len=one_c.kv_last_page_lens, num_qo_heads=Hq,
                                num_kv_heads=Hkv, head_dim=D, page_size=P, qo_indptr_host=one_c.host["indptr"],
                                paged_kv_indptr_host=one_c.host["kv_page_indptr"],
                                paged_kv_last_page_len_host=one_c.host["kv_last_page_lens"],
                                paged_kv_indices_host=one_c.host["kv_page_indices"], target_workgroups=target)
            evs = []
            for rep in range(12):
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                one_w.forward(one_q[rep % 2], one_pool.pages[rep % 2], causal=True)
                e.record()
                evs.append((s, e))
            torch.cuda.synchronize()
            ts = sorted(s.elapsed_time(e) for s, e in evs[2:])
            one_chunk[label] = {"parts_per_tile": one_w._n_splits, "workgroups": one_w._n_tiles * Hkv,
                                "us_per_layer": round(ts[len(ts) // 2] * 1e3, 1)}
            one_w.end_forward()
        one_flops = 4 * Hq * D * (n * one_prior + n * (n + 1) // 2)
        for v in one_chunk.values():
            v["TFLOPs"] = round(one_flops / v["us_per_layer"] / 1e6, 1)
        return one_chunk

    if not config4:
        return {"one_512_token_chunk_over_4096":
                one_chunk_measure(torch.Generator(device="cuda").manual_seed(seed + 43))}
    rng = np.random.default_rng(seed + 40)
    prior = (rng.integers(0, 8193, size=B) // P) * P + rng.integers(0, 16, size=B)
    pool = GpuPagePool(L, int((-(-(prior + n) // P)).sum()) + 8, P, dev, torch.bfloat16)
    fill_normal(pool.pages, seed + 41)
    scatter_pool_order(pool, seed + 42)
    rows = PageTableAllocator(B, 8192 + 1024, P, dev)
    tasks = [TaskData(f"p{b}", int(prior[b]), 1, n, int(prior[b]) + n, SamplingParams()) for b in range(B)]
    caches = [PagedKVCache.empty(rows, pool) for _ in range(B)]
    gen = torch.Generator(device="cuda").manual_seed(seed + 43)
    q = torch.randn((L, B * n, Hq, D), device=dev, generator=gen).to(torch.bfloat16)
    k = torch.randn((L, B * n, Hkv, D), device=dev, generator=gen).to(torch.bfloat16)
    v = torch.randn((L, B * n, Hkv, D), device=dev, generator=gen).to(torch.bfloat16)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(1 << 20, dtype=torch.uint8, device=dev))
    c = FlashPrefillCtx.init_paged_prefill_ctx(tasks, caches, w)
    w.begin_forward(qo_indptr=c.indptr, paged_kv_indptr=c.kv_page_indptr,
                    paged_kv_indices=c.kv_page_indices, paged_kv_last_page_len=c.kv_last_page_lens,
                    num_qo_heads=Hq, num_kv_heads=Hkv, head_dim=D, page_size=P,
                    qo_indptr_host=c.host["indptr"],
                    paged_kv_indptr_host=c.host["kv_page_indptr"],
                    paged_kv_last_page_len_host=c.host["kv_last_page_lens"], paged_kv_indices_host=c.host["kv_page_indices"])
    flops = 4 * Hq * D * sum(n * int(p) + n * (n + 1) // 2 for p in prior)

    def median_us(fn, reps=5):
        evs = []
        for _ in range(reps):
            for layer in range(L):
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                fn(layer)
                e.record()
                evs.append((s, e))
        torch.cuda.synchronize()
        ts = sorted(s.elapsed_time(e) for s, e in evs)
        return ts[len(ts) // 2] * 1e3

    def back_to_back_us(fn, reps=8):
        """All layers inside ONE bracket, `reps` times: the bracket's own 5-6 us (event and dispatch
        latency), which a bracket around a single 12 us launch mostly measures, is spread over L."""
        evs = []
        for _ in range(reps):
            s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            s.record()
            for layer in range(L):
                fn(layer)
            e.record()
            evs.append((s, e))
        torch.cuda.synchronize()
        ts = sorted(s.elapsed_time(e) for s, e in evs)
        return ts[len(ts) // 2] * 1e3 / L

    def append(layer):
        append_paged_kv_cache(k[layer], v[layer], c.indptr, pool.pages[layer], c.kv_page_indices,
                              c.kv_page_indptr, c.kv_last_page_lens)

    append_us = median_us(append)
    append_b2b_us = back_to_back_us(append)
    # the chunk's rotation: apply_rope alone, and rotation + append in one pass (what a layer
    # runs in front of the attention: q rotated out of place, rotated k and v into their slots)
    from deserve_amd.paged_ops import apply_rope, rope_append_paged_kv_cache
    offsets = torch.from_numpy(prior.astype(np.int32)).to(dev)
    rope_us = median_us(lambda layer: apply_rope(q[layer], k[layer], c.indptr, offsets, interleave=True,
                                                 rope_theta=5e5))
    rope_append_us = median_us(lambda layer: rope_append_paged_kv_cache(
        q[layer], k[layer], v[layer], c.indptr, offsets, pool.pages[layer], c.kv_page_indices,
        c.kv_page_indptr, c.kv_last_page_lens, rope_theta=5e5))
    rope_b2b_us = back_to_back_us(lambda layer: apply_rope(q[layer], k[layer], c.indptr, offsets, interleave=True,
                                                           rope_theta=5e5))
    rope_append_b2b_us = back_to_back_us(lambda layer: rope_append_paged_kv_cache(
        q[layer], k[layer], v[layer], c.indptr, offsets, pool.pages[layer], c.kv_page_indices,
        c.kv_page_indptr, c.kv_last_page_lens, rope_theta=5e5))
    append(0), append(1), append(2), append(3)          # the unrotated rows again, as the attention figures assume
    rope_bytes = 2 * B * n * (Hq + Hkv) * D * 2
    rope_append_bytes = 2 * B * n * (Hq + 2 * Hkv) * D * 2
    attn_us = median_us(lambda layer: w.forward(q[layer], pool.pages[layer], causal=True))
    result = {"workload": "BASELINE.json configs[3]: bf16, GQA 32q/8kv, page 16, 16 sequences x 512-token "
                          "chunk appended at offsets U[0,15], attention over prior U[0,8192]; per layer",
              "chunk_tokens": B * n, "kv_tokens": int((prior + n).sum()),
              "append_us_per_layer": round(append_us, 1),
              "append_GBps": round(2 * B * n * 2 * Hkv * D * 2 / append_us / 1e3, 1),
              "append_us_per_layer_back_to_back": round(append_b2b_us, 1),
              "append_GBps_back_to_back": round(2 * B * n * 2 * Hkv * D * 2 / append_b2b_us / 1e3, 1),
              "attention_us_per_layer": round(attn_us, 1),
              "attention_TFLOPs": round(flops / attn_us / 1e6, 1),
              "frac_of_mfma_bf16_peak": round(flops / attn_us / 1e6 / MFMA_PEAK_BF16_TFLOPS, 4),
              "flops_per_layer": flops,
              "rope": {"workload": f"the chunk's {B * n} tokens x ({Hq} q + {Hkv} kv heads), positions from the priors",
                       "apply_rope_us_per_layer": round(rope_us, 1),
                       "apply_rope_bytes": rope_bytes,
                       "apply_rope_frac_of_hbm_peak": round(rope_bytes / rope_us / 1e3 / HBM_PEAK_GBPS, 4),
                       "rope_append_us_per_layer": round(rope_append_us, 1),
                       "rope_append_bytes": rope_append_bytes,
                       "rope_append_frac_of_hbm_peak": round(rope_append_bytes / rope_append_us / 1e3 / HBM_PEAK_GBPS, 4),
                       "back_to_back": {
                           "what": "the 4 layers' launches inside one event bracket (the bracket's 5-6 us spread over 4)",
                           "apply_rope_us_per_layer": round(rope_b2b_us, 1),
                           "apply_rope_frac_of_hbm_peak": round(rope_bytes / rope_b2b_us / 1e3 / HBM_PEAK_GBPS, 4),
                           "rope_append_us_per_layer": round(rope_append_b2b_us, 1),
                           "rope_append_frac_of_hbm_peak":
                               round(rope_append_bytes / rope_append_b2b_us / 1e3 / HBM_PEAK_GBPS, 4)}}}
    def sustained_attention():
        for _ in range(8):
            for layer in range(L):
                w.forward(q[layer], pool.pages[layer], causal=True)

    sensors = _BoardSensors()
    if extras:
        # the board's sensors while the attention launches run back to back for 3 s
        r = _run_sampled(sensors, sustained_attention, 3.0, settle=1.0)
        per_s = r.pop("launches_per_s")
        # The first launches after a pause run in a transient of the board's power control (by
        # rocprofv3 the first two dozen dispatches read 684, 689, 773, 828, 837, 810, ... 700 us
        # before the kernel settles at 645-650 us): the figure above, a median over the first 20,
        # is that transient; this one is the steady state, by the wall clock over two seconds.
        if per_s:
            sustained_us = 1e6 / (32 * per_s)
            result.update({"attention_us_per_layer_sustained": round(sustained_us, 1),
                           "attention_TFLOPs_sustained": round(flops / sustained_us / 1e6, 1),
                           "frac_of_mfma_bf16_peak_sustained":
                               round(flops / sustained_us / 1e6 / MFMA_PEAK_BF16_TFLOPS, 4)})
        result["power"] = {"what": "socket power and shader clock, sampled from the board's sensors while the "
                                   "attention launches run back to back for 3 s (from second 1 on)",
                           "power_cap_W": sensors.cap_watts(),
                           "sustained_TFLOPs": round(32 * flops * per_s / 1e12, 1) if per_s else None, **r}
    if not extras:
        w.end_forward()
        return result
    # The same launches over all-zero q, K and V: instruction for instruction the same work,
    # only the operand bits differ.  The matrix pipeline then draws less power and the chip
    # keeps its clock; the gap to the figure above is what the power limit costs on
    # normally distributed data, not something a kernel can schedule away.
    q.zero_()
    pool.pages.zero_()
    attn_zero_us = median_us(lambda layer: w.forward(q[layer], pool.pages[layer], causal=True))
    r = _run_sampled(sensors, sustained_attention, 3.0, settle=1.0)
    per_s = r.pop("launches_per_s")
    result["power"]["zero_data"] = {"sustained_TFLOPs": round(32 * flops * per_s / 1e12, 1) if per_s else None, **r}
    w.end_forward()
    one_chunk = one_chunk_measure(gen)
    ceiling = mfma_ceiling_section(seed)
    measured_peak = ceiling["levels"]["mfma_only"]["normal"]
    result.update({"mfma_ceiling": ceiling,
                   "frac_of_measured_mfma_ceiling": round(result["attention_TFLOPs"] / measured_peak, 4),
                   "frac_of_measured_mfma_ceiling_sustained":
                       round(result["attention_TFLOPs_sustained"] / measured_peak, 4)
                       if "attention_TFLOPs_sustained" in result else None,
                   "attention_us_per_layer_zero_data": round(attn_zero_us, 1),
                   "attention_TFLOPs_zero_data": round(flops / attn_zero_us / 1e6, 1),
                   "one_512_token_chunk_over_4096": one_chunk})
    return result


def mfma_ceiling_section(seed: int, levels=(0, 1, 2), fills=("normal", "constant")):
    """What the matrix pipeline sustains on this box, measured with the calibration loop of
    deserve_amd/csrc/calib/mfma_ceiling.hip (16 v_mfma_f32_32x32x16_bf16 per iteration and
    wave, 1024 workgroups of 8 waves): level 0 the MFMAs alone, level 1 with the LDS operand
    reads of a 32-token attention block, level 2 with its softmax as well - on N(0, 1)
    operands and on constant ones.  The prefill kernel's rate is read against level 0 on
    N(0, 1) data (`frac_of_measured_mfma_ceiling`) beside the published peak."""
    import ctypes

    import torch

    path = os.path.join(ROOT, "deserve_amd", "libdskv_calib.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it (python -c 'import __graft_entry__ as g; g.build()')")
    lib = ctypes.CDLL(path)
    lib.dskv_calib_mfma_loop.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_float, ctypes.c_void_p]
    lib.dskv_calib_mfma_loop_flops.restype = ctypes.c_double
    lib.dskv_calib_mfma_loop_flops.argtypes = [ctypes.c_int, ctypes.c_int]
    dev = torch.device("cuda")
    wgs, iters = 1024, 1536
    g = torch.Generator(device=dev).manual_seed(seed + 70)
    data = {"normal": torch.randn(512 * 128, generator=g, device=dev).to(torch.bfloat16),
            "constant": torch.full((512 * 128,), 1.0, device=dev, dtype=torch.bfloat16)}
    sink = torch.empty(wgs * 512, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    names = {0: "mfma_only", 1: "plus_lds_operand_reads", 2: "plus_lds_operand_reads_and_softmax"}
    out = {"loop": "16 x v_mfma_f32_32x32x16_bf16 per wave and iteration, 8 waves per workgroup, "
                   f"{wgs} workgroups x {iters} iterations; TFLOP/s", "levels": {}}
    flops = lib.dskv_calib_mfma_loop_flops(wgs, iters)
    for level in levels:
        row = {}
        for fill in fills:
            ts = []
            for rep_ in range(4):
                a_, b_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a_.record()
                rc = lib.dskv_calib_mfma_loop(data[fill].data_ptr(), sink.data_ptr(), level, wgs, iters,
                                              0.1275, stream)
                b_.record()
                if rc != 0:
                    raise RuntimeError(f"dskv_calib_mfma_loop failed with code {rc}")
                torch.cuda.synchronize()
                ts.append(a_.elapsed_time(b_))
            ms = sorted(ts[1:])[1]
            row[fill] = round(flops / ms / 1e9, 1)
        out["levels"][names[level]] = row
    out["frac_of_published_peak_mfma_only_normal_data"] = round(
        out["levels"]["mfma_only"]["normal"] / MFMA_PEAK_BF16_TFLOPS, 4) if 0 in levels and "normal" in fills else None
    return out


class _BoardSensors:
    """The board's own sensors through sysfs (the files `amd-smi metric --power --clock` reads):
    socket power in watts, its cap, and the shader clock in MHz; None where the box exposes no
    such file.  A sampling thread reads them every 50 ms while a workload runs."""

    def __init__(self):
        import glob
        first = lambda pat: (sorted(glob.glob(pat)) or [None])[0]
        base = "/sys/class/drm/card*/device/hwmon/hwmon*/"
        self.power = first(base + "power1_input") or first(base + "power1_average")
        self.cap = first(base + "power1_cap")
        self.sclk = first(base + "freq1_input")
        self.dpm_sclk = first("/sys/class/drm/card*/device/pp_dpm_sclk")   # levels, the current one starred

    @staticmethod
    def _read(path, scale):
        try:
            with open(path) as f:
                return int(f.read().strip()) / scale
        except (OSError, ValueError, TypeError):
            return None

    def cap_watts(self):
        return self._read(self.cap, 1e6)

    def _starred_mhz(self):
        try:
            with open(self.dpm_sclk) as f:
                for line in f:
                    if "*" in line:
                        return float(line.split(":")[1].lower().split("mhz")[0])
        except (OSError, ValueError, TypeError, IndexError):
            pass
        return None

    def sample(self):
        clock = self._read(self.sclk, 1e6)
        return self._read(self.power, 1e6), clock if clock is not None else self._starred_mhz()


def _run_sampled(sensors, launch, seconds: float, settle: float = 1.5):
    """Calls launch() (which enqueues some 10-50 ms of work) and synchronizes, over and over for
    `seconds`, while a thread samples the board's sensors every 50 ms; returns the launches per
    second and the sensor averages from `settle` seconds on (clock and power have settled then)."""
    import threading

    import torch

    samples, stop = [], threading.Event()

    def sampler():
        t0 = time.perf_counter()
        while not stop.is_set():
            w_, f_ = sensors.sample()
            samples.append((time.perf_counter() - t0, w_, f_))
            time.sleep(0.05)

    th = threading.Thread(target=sampler, daemon=True)
    th.start()
    t0 = time.perf_counter()
    n_settled, t_settled = 0, None
    while time.perf_counter() - t0 < seconds:
        launch()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= settle:
            if t_settled is None:
                t_settled = time.perf_counter()
            else:
                n_settled += 1
    t_end = time.perf_counter()
    stop.set()
    th.join()
    watts = [w_ for t_, w_, _ in samples if t_ >= settle and w_ is not None]
    clocks = [f_ for t_, _, f_ in samples if t_ >= settle and f_ is not None]
    return {"launches_per_s": n_settled / (t_end - t_settled) if t_settled and n_settled else None,
            "socket_power_W_avg": round(sum(watts) / len(watts), 1) if watts else None,
            "socket_power_W_max": round(max(watts), 1) if watts else None,
            "shader_clock_MHz_avg": round(sum(clocks) / len(clocks), 1) if clocks else None,
            "samples": len(watts)}


def power_section(seed: int, seconds: float = 6.0):
    """Socket power and shader clock while a kernel runs back to back for `seconds` (sampled
    from the second 1.5 on, when clock and power have settled): the prefill attention of
    configuration 4, the bare MFMA loop on N(0,1) and on constant operands, and the decode
    attention of configuration 2.  Says whether a kernel's rate is what the board's power cap
    leaves of the nominal clock."""
    import ctypes

    import numpy as np
    import torch

    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.kvcache.paged.kvcache import PagedKVCache
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.model.context.flash import FlashDecodeCtx, FlashPrefillCtx
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper
    from deserve_amd.synthetic import fill_normal, make_decode_workload, scatter_pool_order
    from deserve_amd.task import SamplingParams, TaskData

    dev = torch.device("cuda")
    sensors = _BoardSensors()
    out = {"sensors": {"power": sensors.power, "cap": sensors.cap, "shader_clock": sensors.sclk or sensors.dpm_sclk},
           "power_cap_W": sensors.cap_watts(), "seconds_per_workload": seconds,
           "idle_W": None, "workloads": {}}
    torch.cuda.synchronize()
    time.sleep(1.0)
    out["idle_W"] = sensors.sample()[0]

    def sustained(name, launch, work_per_launch, unit, what):
        """launch() enqueues some 10-50 ms of the kernel; work_per_launch in flop or bytes."""
        r = _run_sampled(sensors, launch, seconds)
        rate = work_per_launch * r.pop("launches_per_s") if r["launches_per_s"] else None
        out["workloads"][name] = {
            "what": what,
            "rate": round(rate / (1e12 if unit == "TFLOP/s" else 1e9), 1) if rate else None, "unit": unit, **r}
        time.sleep(1.0)           # let the board settle before the next workload

    # prefill attention, configuration 4 (as prefill_section builds it)
    L, P, Hq, Hkv, D, B, n = 4, 16, 32, 8, 128, 16, 512
    rng = np.random.default_rng(seed + 40)
    prior = (rng.integers(0, 8193, size=B) // P) * P + rng.integers(0, 16, size=B)
    pool = GpuPagePool(L, int((-(-(prior + n) // P)).sum()) + 8, P, dev, torch.bfloat16)
    fill_normal(pool.pages, seed + 41)
    scatter_pool_order(pool, seed + 42)
    rows = PageTableAllocator(B, 8192 + 1024, P, dev)
    tasks = [TaskData(f"p{b}", int(prior[b]), 1, n, int(prior[b]) + n, SamplingParams()) for b in range(B)]
    caches = [PagedKVCache.empty(rows, pool) for _ in range(B)]
    gen = torch.Generator(device="cuda").manual_seed(seed + 43)
    q = torch.randn((L, B * n, Hq, D), device=dev, generator=gen).to(torch.bfloat16)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(1 << 20, dtype=torch.uint8, device=dev))
    c = FlashPrefillCtx.init_paged_prefill_ctx(tasks, caches, w)
    w.begin_forward(qo_indptr=c.indptr, paged_kv_indptr=c.kv_page_indptr, paged_kv_indices=c.kv_page_indices,
                    paged_kv_last_page_len=c.kv_last_page_lens, num_qo_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                    page_size=P, qo_indptr_host=c.host["indptr"], paged_kv_indptr_host=c.host["kv_page_indptr"],
                    paged_kv_last_page_len_host=c.host["kv_last_page_lens"],
                    paged_kv_indices_host=c.host["kv_page_indices"])
    flops = 4 * Hq * D * sum(n * int(p_) + n * (n + 1) // 2 for p_ in prior)
    out_rows = torch.empty_like(q[0])

    def prefill_launch():
        for _ in range(8):
            for layer in range(L):
                w.forward(q[layer], pool.pages[layer], causal=True, out=out_rows)

    sustained("prefill_attention_config4", prefill_launch, 32 * flops, "TFLOP/s",
              "prefill_attn_mfma_kernel<bf16> on configuration 4's 16 x 512-token chunks, N(0,1) q, K, V")
    q.zero_()
    pool.pages.zero_()
    sustained("prefill_attention_config4_zero_data", prefill_launch, 32 * flops, "TFLOP/s",
              "the same launches over all-zero q, K and V")
    w.end_forward()
    del pool, q, w, c, caches, rows
    torch.cuda.empty_cache()

    # the bare matrix loop
    path = os.path.join(ROOT, "deserve_amd", "libdskv_calib.so")
    if not os.path.exists(path):
        raise RuntimeError(f"{path} is missing: build it (python -c 'import __graft_entry__ as g; g.build()')")
    lib = ctypes.CDLL(path)
    lib.dskv_calib_mfma_loop.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                         ctypes.c_int, ctypes.c_float, ctypes.c_void_p]
    lib.dskv_calib_mfma_loop_flops.restype = ctypes.c_double
    lib.dskv_calib_mfma_loop_flops.argtypes = [ctypes.c_int, ctypes.c_int]
    wgs, iters = 1024, 1536
    g = torch.Generator(device=dev).manual_seed(seed + 70)
    data = {"normal": torch.randn(512 * 128, generator=g, device=dev).to(torch.bfloat16),
            "constant": torch.full((512 * 128,), 1.0, device=dev, dtype=torch.bfloat16)}
    sink = torch.empty(wgs * 512, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    loop_flops = lib.dskv_calib_mfma_loop_flops(wgs, iters)
    for fill in ("normal", "constant"):
        def mfma_launch(fill=fill):
            rc = lib.dskv_calib_mfma_loop(data[fill].data_ptr(), sink.data_ptr(), 0, wgs, iters, 0.1275, stream)
            if rc != 0:
                raise RuntimeError(f"dskv_calib_mfma_loop failed with code {rc}")
        sustained(f"mfma_only_{fill}_operands", mfma_launch, loop_flops, "TFLOP/s",
                  f"nothing but v_mfma_f32_32x32x16_bf16, {fill} operands, two waves per SIMD")

    # decode attention, configuration 2
    Ld = 4
    ctx = np.random.default_rng(seed).integers(256, 4097, size=64)
    wl = make_decode_workload("power", ctx, Ld, 32, 8, 128, 16, torch.bfloat16, headroom_tokens=32,
                              seed=seed + 1, fill=True)
    wd, _ = get_wrappers(wl.pool.main_device)
    cd = FlashDecodeCtx.init_paged_decode_ctx(wl.tasks, wl.caches, wd)
    wd.begin_forward(indptr=cd.kv_page_indptr, indices=cd.kv_page_indices, last_page_len=cd.kv_last_page_lens,
                     num_qo_heads=32, num_kv_heads=8, head_dim=128, page_size=16,
                     indptr_host=cd.host["kv_page_indptr"], last_page_len_host=cd.host["kv_last_page_lens"])
    kv_bytes = sum(t.start_pos + 1 for t in wl.tasks) * wl.kv_bytes_per_token()
    outs = [torch.empty_like(wl.q[0]) for _ in range(Ld)]

    def decode_launch():
        for _ in range(32):
            for layer in range(Ld):
                wd.forward(wl.q[layer], wl.pool.pages[layer], out=outs[layer])

    sustained("decode_attention_config2", decode_launch, 32 * Ld * kv_bytes, "GB/s",
              "decode_attn_mfma_kernel<bf16> + merge on configuration 2's 64 requests (K/V bytes only)")
    wd.end_forward()
    return out


def mixed_section(seed: int, shapes=("8B", "70B", "8B_chunk_behind_8000"), reps: int = 6):
    """The reference's usual step in its decode-first aggregated mode (engine/pipeline/stage/
    join.py:11-88, 512-token budget; deserve_exp/exp_args.csv: microbatch size 75): 75 running
    requests with contexts U[256, 4096], one new token each, plus one chunk that fills the
    rest of the budget (437 tokens) over a prior U[0, 4096] - all sent through the prefill
    wrapper, as engine/microbatch/processor.py:116-145 does whenever one task has more than one
    token.  Per layer, on the launch stream: the append of the step's 512 tokens and the
    attention call, with the one-row requests routed to the split-KV decode kernel and
    without; the decode rows alone and the chunk alone give the two roofline fractions."""
    import numpy as np
    import torch

    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.model.context.flash import FlashPrefillCtx
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper, append_paged_kv_cache
    from deserve_amd.synthetic import make_mixed_workload, mixed_step_shape

    dev = torch.device("cuda")
    P, Hkv, D = 16, 8, 128
    out = {"workload": "75 decode rows, ctx U[256,4096], + one 437-token chunk over a prior U[0,4096] (512-token "
                       "step budget), bf16, page 16, through the prefill wrapper; per layer"}
    for tag in shapes:
        L, Hq = {"8B": (16, 32), "70B": (10, 64), "8B_chunk_behind_8000": (16, 32)}[tag]
        dctx, prior, lens = mixed_step_shape(seed + 60)
        if tag == "8B_chunk_behind_8000":
            prior = [8000]          # a prompt as long as configuration 4's
        wl = make_mixed_workload("mixed" + tag, dctx, prior, lens, L, Hq, Hkv, D, P, torch.bfloat16, seed=seed + 61)
        n_dec, nnz = len(dctx), wl.nnz
        tok_bytes = wl.kv_bytes_per_token()
        _, w = get_wrappers(dev)
        settle_heap()

        def plan(tasks, caches, route=True):
            return FlashPrefillCtx.init_and_plan(tasks, caches, w, Hq, Hkv, D, P) if route else None

        def median_us(fn, layers=L):
            evs = []
            for _ in range(reps):
                for layer in range(layers):
                    s_, e_ = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                    s_.record()
                    fn(layer)
                    e_.record()
                    evs.append((s_, e_))
            torch.cuda.synchronize()
            ts = sorted(a.elapsed_time(b) for a, b in evs[L:])          # the first pass warms up
            return ts[len(ts) // 2] * 1e3

        c = FlashPrefillCtx.init_and_plan(wl.tasks, wl.caches, w, Hq, Hkv, D, P)
        routed_rows, parts, layout = w._n_decode_rows, w._n_splits, w._info.layout
        launch_shape = {"decode_workgroups": w._info.n_decode_workgroups * (-(-Hkv // 4) if layout else 1),
                        "tile_workgroups": w._n_tiles * Hkv, "waves_per_workgroup": 4 if layout else 8}
        n_pages = int(c.host["kv_page_indptr"][-1])
        append_us = median_us(lambda l: append_paged_kv_cache(wl.k[l], wl.v[l], c.indptr, wl.pool.pages[l],
                                                              c.kv_page_indices, c.kv_page_indptr,
                                                              c.kv_last_page_lens))
        # (the first passes over a fresh pool run a few percent slow: one untimed round first)
        median_us(lambda l: w.forward(wl.q[l], wl.pool.pages[l], causal=True))
        mixed_us = median_us(lambda l: w.forward(wl.q[l], wl.pool.pages[l], causal=True))
        w.end_forward()
        # the whole step as the engine runs it: plan + upload, then L x (append + attention)
        def step():
            cc = FlashPrefillCtx.init_and_plan(wl.tasks, wl.caches, w, Hq, Hkv, D, P)
            for l in range(L):
                append_paged_kv_cache(wl.k[l], wl.v[l], cc.indptr, wl.pool.pages[l], cc.kv_page_indices,
                                      cc.kv_page_indptr, cc.kv_last_page_lens)
                w.forward(wl.q[l], wl.pool.pages[l], causal=True)
            w.end_forward()
        for _ in range(2):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(10):
            step()
        torch.cuda.synchronize()
        step_ms = (time.perf_counter() - t0) / 10 * 1e3
        # the same batch with every request on the tile path (a one-row request = one live
        # row of a 64-row tile): what the step cost before the routing
        w2 = BatchPrefillWithPagedKVCacheWrapper(torch.empty(256 << 20, dtype=torch.uint8, device=dev))
        kw = dict(qo_indptr=c.indptr, paged_kv_indptr=c.kv_page_indptr, paged_kv_indices=c.kv_page_indices,
                  paged_kv_last_page_len=c.kv_last_page_lens, num_qo_heads=Hq, num_kv_heads=Hkv, head_dim=D,
                  page_size=P, qo_indptr_host=c.host["indptr"], paged_kv_indptr_host=c.host["kv_page_indptr"],
                  paged_kv_last_page_len_host=c.host["kv_last_page_lens"],
                  paged_kv_indices_host=c.host["kv_page_indices"])
        w2.begin_forward(route_one_row_requests=False, **kw)
        tiled_us = median_us(lambda l: w2.forward(wl.q[l], wl.pool.pages[l], causal=True))
        w2.end_forward()
        from deserve_amd import _lib
        w2.begin_forward(route_one_row_requests=_lib.ROUTE_TWO_LAUNCHES, **kw)
        two_us = median_us(lambda l: w2.forward(wl.q[l], wl.pool.pages[l], causal=True))
        w2.end_forward()
        w2.begin_forward(route_one_row_requests=_lib.ROUTE_SHARED_LAUNCH, **kw)
        shared_us = median_us(lambda l: w2.forward(wl.q[l], wl.pool.pages[l], causal=True))
        shared_shape = {"decode_workgroups": w2._info.n_decode_workgroups * -(-Hkv // 4),
                        "tile_workgroups": w2._n_tiles * Hkv, "chunk_parts_per_tile": w2._n_splits,
                        "waves_per_workgroup": 4}
        w2.end_forward()
        # the two halves alone: the decode rows as a batch of their own, the chunk as one
        h = {k_: v_.numpy() for k_, v_ in c.host.items()}
        i32 = lambda a_: torch.from_numpy(np.ascontiguousarray(a_, dtype=np.int32))
        def sub_batch(lo, hi):
            ip = h["kv_page_indptr"]
            host = dict(qo_indptr_host=i32(h["indptr"][lo: hi + 1] - h["indptr"][lo]),
                        paged_kv_indptr_host=i32(ip[lo: hi + 1] - ip[lo]),
                        paged_kv_last_page_len_host=i32(h["kv_last_page_lens"][lo:hi]),
                        paged_kv_indices_host=i32(h["kv_page_indices"][ip[lo]: ip[hi]]))
            devs = {k_[:-5]: v_.to(dev) for k_, v_ in host.items()}
            return dict(num_qo_heads=Hq, num_kv_heads=Hkv, head_dim=D, page_size=P, **devs, **host), \
                slice(int(h["indptr"][lo]), int(h["indptr"][hi]))
        halves = {}
        for name, (lo, hi) in (("decode_rows", (0, n_dec)), ("chunk", (n_dec, len(wl.tasks)))):
            kw_h, rows = sub_batch(lo, hi)
            w2.begin_forward(**kw_h)
            qh = wl.q[:, rows].contiguous()
            halves[name] = median_us(lambda l: w2.forward(qh[l], wl.pool.pages[l], causal=True))
            w2.end_forward()
        dec_bytes = wl.decode_kv_tokens() * tok_bytes + 2 * n_dec * Hq * D * 2 + \
            4 * int(h["kv_page_indptr"][n_dec])
        flops = wl.chunk_flops()
        out[tag] = {
            "layers": L, "n_qo_heads": Hq, "decode_rows": n_dec, "rows_routed_to_decode_kernel": routed_rows,
            "plan": "one launch, decode and tile workgroups share the compute units" if layout else
                    ("all rows as query tiles" if routed_rows == 0 else "decode pass, then tile pass"),
            "launch": launch_shape,
            "chunk_tokens": int(lens[0]), "chunk_prior": int(prior[0]), "chunk_parts_per_tile": parts,
            "decode_kv_tokens": wl.decode_kv_tokens(), "kv_pages": n_pages,
            "append_us_per_layer": round(append_us, 1),
            "attention_us_per_layer": round(mixed_us, 1),
            "attention_us_per_layer_all_rows_as_tiles": round(tiled_us, 1),
            "attention_us_per_layer_decode_pass_then_tile_pass": round(two_us, 1),
            "attention_us_per_layer_one_launch_shared_cus": round(shared_us, 1), "one_launch_shape": shared_shape,
            "decode_rows_alone_us_per_layer": round(halves["decode_rows"], 1),
            "decode_rows_GBps": round(dec_bytes / halves["decode_rows"] / 1e3, 1),
            "decode_rows_frac_of_hbm_peak": round(dec_bytes / halves["decode_rows"] / 1e3 / HBM_PEAK_GBPS, 4),
            "chunk_alone_us_per_layer": round(halves["chunk"], 1),
            "chunk_TFLOPs": round(flops / halves["chunk"] / 1e6, 1),
            "chunk_frac_of_mfma_bf16_peak": round(flops / halves["chunk"] / 1e6 / MFMA_PEAK_BF16_TFLOPS, 4),
            "step_ms": round(step_ms, 3), "step_tokens_per_s": round(nnz / step_ms * 1e3, 1),
            "whole_call_decode_bytes_GBps": round(dec_bytes / mixed_us / 1e3, 1),
            "whole_call_decode_bytes_frac_of_hbm_peak": round(dec_bytes / mixed_us / 1e3 / HBM_PEAK_GBPS, 4),
            "whole_call_chunk_TFLOPs": round(flops / mixed_us / 1e6, 1),
        }
        del wl, w2, c
        torch.cuda.empty_cache()
    return out


def fragmented_section(seed: int):
    """Baseline configuration 5 (Llama-3-70B stage, 10 layers, GQA 64q/8kv): 128 sequences with
    lognormal context lengths on a pool fragmented by evictions (40 % of the pages freed and
    handed out again, lowest id first); 25 % of the sequences are swapped out and back in
    (per-request offload / reload of scattered pages), then decode steps run."""
    import numpy as np
    import torch

    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.kvcache.manager import KVCacheManager
    from deserve_amd.kvcache.paged.chunk_pool import CpuChunkPool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.kvcache.virtual import VirtualPagedKVCache, VirtualPagePool
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.synthetic import config5_context_lengths, fill_normal
    from deserve_amd.task import SamplingParams, TaskData

    dev = torch.device("cuda")
    L, P, Hq, Hkv, D, B, steps = 10, 16, 64, 8, 128, 128, 6
    rng = np.random.default_rng(seed + 50)
    ctx_lens = config5_context_lengths(seed + 3)
    need = int((-(-(ctx_lens + steps + 8) // P)).sum())
    pool = VirtualPagePool(L, int(need / 0.4 * 1.05) + 128, 0, P, dev, torch.bfloat16)
    fill_normal(pool.pages, seed + 51)
    rows = PageTableAllocator(B + 40, 32768 + 64, P, dev)
    filler = pool.alloc(pool.num_avails)
    pool.free(torch.from_numpy(rng.permutation(filler.numpy())[: int(0.4 * len(filler))].copy()))
    made = {}
    for b in rng.permutation(B):                        # out-of-order arrival into the holes
        c = VirtualPagedKVCache.empty(rows, pool)
        c.extend(int(ctx_lens[b]))
        made[int(b)] = c
    tasks = [TaskData(f"f{b}", int(ctx_lens[b]), 1, 1, int(ctx_lens[b]), SamplingParams()) for b in range(B)]
    caches = [made[b] for b in range(B)]
    mgr = KVCacheManager(pool, CpuChunkPool(L, 15, P, torch.bfloat16), rows)
    swapped = sorted(rng.choice(B, size=B // 4, replace=False).tolist())
    page_bytes = 2 * P * Hkv * D * 2
    swap_bytes = sum(caches[b].page_table.occupied for b in swapped) * L * page_bytes

    def timed(fn):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        fn()
        mgr.synchronize()
        torch.cuda.synchronize()
        return time.perf_counter() - t0

    t_out = t_in = float("inf")
    for _ in range(2):                                   # the second round trip runs on warmed-up paths
        handles = []
        t_out = min(t_out, timed(lambda: handles.extend(
            mgr.copy_gpu_to_cpu(caches[b], tasks[b].task_id) for b in swapped)))
        for b in swapped:
            caches[b].free()
        back = []
        t_in = min(t_in, timed(lambda: back.extend(
            mgr.copy_cpu_to_gpu(h, tasks[b].task_id) for h, b in zip(handles, swapped))))
        for h in handles:
            h.free()
        for b, c in zip(swapped, back):
            caches[b] = c

    gen = torch.Generator(device="cuda").manual_seed(seed + 52)
    mk = lambda h: torch.randn((L, B, h, D), generator=gen, device=dev).to(torch.bfloat16)
    q, k, v = mk(Hq), mk(Hkv), mk(Hkv)
    w, _ = get_wrappers(dev)
    ev, attn_bytes = [], 0

    def decode_step(record: bool):
        nonlocal attn_bytes
        c = FlashDecodeCtx.init_and_plan(tasks, caches, w, Hq, Hkv, D, P)
        for layer in range(L):
            pages = pool.get_layered_pages(layer)
            new_kv = dict(k_append=k[layer], v_append=v[layer])   # written by the attention launch
            if record and layer % 2 == 0:
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                out = w.forward(q[layer], pages, phases=1, **new_kv)
                e.record()
                w.forward(q[layer], pages, phases=2, out=out)
                ev.append((s, e))
            else:
                w.forward(q[layer], pages, **new_kv)
        w.end_forward()
        if record:
            kv_lens = np.array([t.start_pos + 1 for t in tasks], dtype=np.int64)
            attn_bytes = attention_bytes_per_layer(kv_lens, int(c.host["kv_page_indptr"][-1]), B, Hq, D, 2,
                                                   2 * Hkv * D * 2)
        for t in tasks:
            t.step()

    for _ in range(2):
        decode_step(False)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps - 2):
        decode_step(True)
    torch.cuda.synchronize()
    ms_step = (time.perf_counter() - t0) / (steps - 2) * 1e3
    us = sorted(s.elapsed_time(e) for s, e in ev)
    attn_us = us[len(us) // 2] * 1e3
    return {"workload": "BASELINE.json configs[4]: 10 layers, bf16, GQA 64q/8kv, page 16, 128 sequences, "
                        "lognormal ctx (median 2048, [64,32768]), 40 % of the pool freed and reallocated out "
                        "of order; 32 sequences swapped out and back in (twice, best time) before the decode steps",
            "kv_tokens": int(sum(t.start_pos for t in tasks)),
            "swap_out_GBps": round(swap_bytes / t_out / 1e9, 2), "swap_in_GBps": round(swap_bytes / t_in / 1e9, 2),
            "swapped_bytes": swap_bytes, "decode_ms_per_step": round(ms_step, 3),
            "attention_us_per_layer": round(attn_us, 1),
            "attention_GBps": round(attn_bytes / attn_us / 1e3, 1),
            "attention_frac_of_hbm_peak": round(attn_bytes / attn_us / 1e3 / HBM_PEAK_GBPS, 4)}


def page8_in_child(seed: int):
    """Configuration 2 on pages of 8 tokens - the page size the reference deploys with
    (worker_api.py:170,187) - in a process of its own: the whole step and the attention pass."""
    import subprocess

    cmd = [sys.executable, os.path.abspath(__file__), "--page-size", "8", "--steps", "40", "--warmup", "6",
           "--seed", str(seed), "--no-cpu-baseline", "--no-swap", "--no-prefill", "--no-fragmented",
           "--no-graph", "--no-rope-step", "--no-mixed", "--no-page8"]
    res = subprocess.run(cmd, stdout=subprocess.PIPE, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"bench on 8-token pages failed with exit code {res.returncode}")
    d = json.loads(res.stdout.strip().splitlines()[-1])
    r = d.get("roofline", {})
    return {"workload": d["config"]["workload"], "ms_per_step": d["ms_per_step"], "value_GBps": d["value"],
            "pct_of_hbm_peak": d["pct_of_hbm_peak"], "attention_avg_launch_us": r.get("avg_launch_us"),
            "attention_frac_of_hbm_peak": r.get("frac"), "steps": d["steps"]}


def run_section_in_child(name: str, seed: int):
    """The host-link sections run in a process of their own, after this one has released the
    GPU memory it held: measured here, pinned-copy rates of a section depend on which streams
    and pinned buffers the process created before it (30 instead of 48 GB/s for the second
    section to run), which says nothing about the section."""
    import subprocess

    res = subprocess.run([sys.executable, os.path.abspath(__file__), "--section", name, "--seed", str(seed)],
                         stdout=subprocess.PIPE, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"bench section {name} failed with exit code {res.returncode}")
    return json.loads(res.stdout.strip().splitlines()[-1])


def main() -> int:
    a = parse_args()
    if a.section is not None:
        import torch
        torch.cuda.set_device(0)
        if a.section == "prefill":
            print(json.dumps(prefill_section(a.seed, extras=not a.prefill_config4_only,
                                             config4=not a.prefill_one_chunk_only)))
        elif a.section == "mfma-ceiling":
            print(json.dumps(mfma_ceiling_section(a.seed)))
        elif a.section == "power":
            print(json.dumps(power_section(a.seed)))
        elif a.section == "mixed":
            print(json.dumps(mixed_section(a.seed, shapes=tuple(a.mixed_shapes.split(",")))))
        else:
            print(json.dumps({"swap": swap_section, "fragmented": fragmented_section}[a.section](a.seed)))
        return 0
    if a.gpus != 1:
        print(f"bench.py measures one GPU: --gpus {a.gpus} is not supported in this build "
              "(the path has no cross-GPU exchange: it shards by layers, kv heads or sequences "
              "with one independent copy of this work per GPU)", file=sys.stderr)
        return 2
    import numpy as np
    import torch

    from deserve_amd import _lib
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.paged_ops import append_paged_kv_cache, rope_append_paged_kv_cache
    from deserve_amd.synthetic import config2_context_lengths, make_decode_workload

    if not os.path.exists(_lib.LIB_PATH):
        _lib.build()
    torch.cuda.set_device(0)
    L, Hq, Hkv, D, P = 16, 32, 8, 128, a.page_size
    graph_steps = 0 if a.no_graph else 24
    rope_steps = 0 if (a.rope or a.no_rope_step) else 24          # the step once more with rotation, as a model runs it
    total_steps = a.steps + a.warmup + graph_steps + rope_steps
    ctx = config2_context_lengths(a.seed)
    wl = make_decode_workload("cfg2", ctx, L, Hq, Hkv, D, P, torch.bfloat16,
                              headroom_tokens=total_steps + 8, seed=a.seed, use_rope=a.rope)
    decode_wrapper, _ = get_wrappers(wl.pool.main_device)
    settle_heap()
    e = wl.pool.pages.element_size()
    tok_bytes = wl.kv_bytes_per_token()
    torch.cuda.synchronize()

    if a.pmc_calibration:
        # move_pages_kernel<true> over 4096 consecutive 64 KiB pages of layer 0 -> scratch
        from deserve_amd.kvcache import _native
        ids = torch.arange(4096, dtype=torch.int32)
        one_layer = type("OneLayer", (), {"num_layers": 1, "pages": wl.pool.pages[:1],
                                          "layer_stride_bytes": wl.pool.layer_stride_bytes,
                                          "page_bytes": wl.pool.page_bytes})()
        _native.gather_pages(one_layer, ids)
        torch.cuda.synchronize()

    # (start, end) events around the split-KV attention pass, created before the timed region
    ev_pool = [] if a.no_kernel_events else [
        (torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
        for _ in range(a.steps * L // max(a.event_every, 1) + 1)]
    ev_pairs = []
    launch_no = [0]
    step_bytes = []
    attn_bytes_layer = []

    fused = not a.no_fused_append

    def one_step(timed: bool, rope: bool = a.rope):
        """prepare (metadata + plan in one upload) then L x (append + attention: one launch
        for both, or two with --no-fused-append)."""
        c = FlashDecodeCtx.init_and_plan(wl.tasks, wl.caches, decode_wrapper, Hq, Hkv, D, P,
                                         target_workgroups=a.workgroups)
        for layer in range(L):
            q, k, v = wl.q[layer], wl.k[layer], wl.v[layer]
            pages = wl.pool.get_layered_pages(layer)
            if fused:
                # the attention launch (rotates q and k and) writes the token
                new_kv = dict(k_append=k, v_append=v)
                if rope:
                    new_kv.update(rope_offsets=c.offsets, rope_theta=5e5)
            else:
                new_kv = {}
                if rope:
                    q = rope_append_paged_kv_cache(q, k, v, c.indptr, c.offsets, pages, c.kv_page_indices,
                                                   c.kv_page_indptr, c.kv_last_page_lens, rope_theta=5e5)
                else:
                    append_paged_kv_cache(k, v, c.indptr, pages, c.kv_page_indices, c.kv_page_indptr,
                                          c.kv_last_page_lens)
            launch_no[0] += 1
            if timed and not a.no_kernel_events and launch_no[0] % max(a.event_every, 1) == 0:
                s, t = ev_pool[len(ev_pairs)]
                s.record()
                out = decode_wrapper.forward(q, pages, phases=1, **new_kv)
                t.record()
                decode_wrapper.forward(q, pages, phases=2, out=out)
                ev_pairs.append((s, t))
            else:
                decode_wrapper.forward(q, pages, **new_kv)
        decode_wrapper.end_forward()
        if timed:
            kv_lens = np.array([t.start_pos + 1 for t in wl.tasks], dtype=np.int64)
            n_pages = int(c.host["kv_page_indptr"][-1])
            ab = attention_bytes_per_layer(kv_lens, n_pages, wl.batch, Hq, D, e, tok_bytes)
            attn_bytes_layer.append(ab)
            step_bytes.append(L * (ab + append_bytes_per_layer(wl.batch, wl.batch, n_pages, tok_bytes)))
        for t in wl.tasks:
            t.step()
        return c

    last_ctx = None
    for _ in range(a.warmup):
        last_ctx = one_step(False)
    torch.cuda.synchronize()
    in_flight = [torch.cuda.Event() for _ in range(max(a.steps_in_flight, 0))]

    def wait_turn(i: int):
        """Blocks until step i - len(in_flight) has run; returns the event to record after step i."""
        if not in_flight:
            return None
        ev = in_flight[i % len(in_flight)]
        if i >= len(in_flight):
            ev.synchronize()
        return ev

    t0 = time.perf_counter()
    marks = [t0]
    for i in range(a.steps):
        ev = wait_turn(i)
        last_ctx = one_step(True)
        if ev is not None:
            ev.record()
        marks.append(time.perf_counter())
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    loop_ms = np.diff(np.array(marks)) * 1e3       # host time per loop turn (enqueue + its wait)
    rope_ms = None
    if rope_steps:
        for _ in range(4):
            one_step(False, rope=True)
        torch.cuda.synchronize()
        r0 = time.perf_counter()
        for i in range(rope_steps - 4):
            ev = wait_turn(i)
            one_step(False, rope=True)
            if ev is not None:
                ev.record()
        torch.cuda.synchronize()
        rope_ms = (time.perf_counter() - r0) / (rope_steps - 4) * 1e3

    ms_per_step = elapsed / a.steps * 1e3
    value = sum(step_bytes) / elapsed / 1e9
    out = {
        "metric": "paged decode-attn HBM GB/s", "value": round(value, 1), "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": ("BASELINE.json configs[1]" if P == 16 else "BASELINE.json configs[1] with another page size")
                               + ": Llama-3-8B stage, 16 layers, bf16, GQA 32q/8kv, "
                               f"head_dim 128, page {P}, decode batch 64, ctx U[256,4096], scattered pages; "
                               "step = host plan + 16 x (append 1 token + paged decode attention)"
                               + (" + RoPE" if a.rope else ""),
                   "batch": wl.batch, "layers": L, "kv_tokens": int(sum(t.start_pos for t in wl.tasks)),
                   "work_items": decode_wrapper._n_items, "workgroups": decode_wrapper._n_workgroups, "seed": a.seed,
                   "append": "inside the attention launch" if fused else "own launch"},
        "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "stage_tokens_per_s": round(wl.batch / (elapsed / a.steps), 1),
        "with_rope_ms_per_step": None if rope_ms is None else round(rope_ms, 4),
        "host_loop_ms": {"median": round(float(np.median(loop_ms)), 3), "max": round(float(loop_ms.max()), 3),
                         "turns_over_3ms": int((loop_ms > 3.0).sum())},
    }
    if ev_pairs:
        all_ms = sorted(s.elapsed_time(t) for s, t in ev_pairs)
        # an interval in which the host fell behind the GPU holds host latency, not the
        # kernel: intervals beyond 1.5 x the median are left out of the average
        times_ms = [x for x in all_ms if x <= 1.5 * all_ms[len(all_ms) // 2]]
        avg_ms = sum(times_ms) / len(times_ms)
        achieved = (sum(attn_bytes_layer) / len(attn_bytes_layer)) / (avg_ms * 1e-3) / 1e9
        traffic = traffic_workload = traffic_alg = None
        tfile = os.path.join(ROOT, "profiles", "decode_attn_cfg2_traffic.json")
        if os.path.exists(tfile) and P == 16:                # measured on the 16-token pages of configuration 2
            tj = json.load(open(tfile))
            traffic = tj.get("hbm_bytes_per_launch")
            traffic_workload, traffic_alg = tj.get("workload"), tj.get("algorithmic_bytes_per_launch")
        # cross-checks of the bracketed figure: what a bracket costs with nothing inside it, and
        # the same pass over all layers back to back inside ONE bracket (no cache reuse between
        # layers); bracket - empty bracket, the back-to-back time and rocprofv3 agree
        empty = []
        for _ in range(21):
            s, t = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            wl.q[0].mul_(1.0)                                # the brackets follow work, as in a step
            s.record()
            t.record()
            empty.append((s, t))
        c = FlashDecodeCtx.init_paged_decode_ctx(wl.tasks, wl.caches, decode_wrapper)
        decode_wrapper.begin_forward(indptr=c.kv_page_indptr, indices=c.kv_page_indices,
                                     last_page_len=c.kv_last_page_lens, num_qo_heads=Hq,
                                     num_kv_heads=Hkv, head_dim=D, page_size=P,
                                     indptr_host=c.host["kv_page_indptr"],
                                     last_page_len_host=c.host["kv_last_page_lens"], indices_host=c.host["kv_page_indices"],
                                     target_workgroups=a.workgroups)
        scratch_out = torch.empty_like(wl.q[0])
        rounds = 3
        s, t = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for r in range(rounds + 1):
            if r == 1:
                s.record()
            for layer in range(L):
                decode_wrapper.forward(wl.q[layer], wl.pool.get_layered_pages(layer), phases=1, out=scratch_out)
        t.record()
        decode_wrapper.end_forward()
        torch.cuda.synchronize()
        empty_us = sorted(x.elapsed_time(y) for x, y in empty)[len(empty) // 2] * 1e3
        b2b_us = s.elapsed_time(t) * 1e3 / (rounds * L)
        out["roofline"] = {"bound": "hbm", "kernel": "decode_attn_mfma_kernel<bf16> (split-KV pass" + (", writes the step's token first)" if fused else ")"),
                           "empty_bracket_us": round(empty_us, 2), "back_to_back_us": round(b2b_us, 2),
                           "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                           "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                           "traffic_source": None if traffic is None else
                           "profiles/decode_attn_cfg2_traffic.json: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of an "
                           "earlier profiled run of this command (" + str(traffic_workload) + ", " +
                           str(traffic_alg) + " algorithmic bytes per launch there); replayed from that file, "
                           "not measured in this run",
                           "avg_launch_us": round(avg_ms * 1e3, 2), "launches": len(times_ms),
                           "intervals_left_out": len(all_ms) - len(times_ms),
                           "algorithmic_bytes_per_launch": int(sum(attn_bytes_layer) / len(attn_bytes_layer))}
    if graph_steps:
        # the same step (rope off: append + attention per layer through the stage) captured
        # once into a HIP graph and replayed; per step the host rebuilds metadata and plan only
        from deserve_amd.execution.graph import GraphedDecodeStep
        gstep = GraphedDecodeStep(wl.stage, decode_wrapper, max_batch=wl.batch,
                                  max_pages=int(last_ctx.host["kv_page_indptr"][-1]) + 4 * wl.batch,
                                  device=wl.pool.main_device, num_qo_heads=Hq, num_kv_heads=Hkv,
                                  head_dim=D, page_size=P, target_workgroups=a.workgroups)
        xs = (wl.q, wl.k, wl.v)

        def graphed():
            gstep.run(xs, wl.tasks, wl.caches)
            for t in wl.tasks:
                t.step()

        for _ in range(4):
            graphed()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(graph_steps - 4):
            ev = wait_turn(i)
            graphed()
            if ev is not None:
                ev.record()
        torch.cuda.synchronize()
        g_ms = (time.perf_counter() - t0) / (graph_steps - 4) * 1e3
        out["graph"] = {"ms_per_step": round(g_ms, 4),
                        "value_GBps": round(step_bytes[-1] / g_ms / 1e6, 1),
                        "pct_of_hbm_peak": round(100.0 * step_bytes[-1] / g_ms / 1e6 / HBM_PEAK_GBPS, 2),
                        "captures": gstep.captures,
                        "note": "same step replayed as one HIP graph (host: metadata + plan only)"}
    if not a.no_cpu_baseline:
        meta = {n: last_ctx.host[n].numpy() for n in ("kv_page_indices", "kv_page_indptr", "kv_last_page_lens")}
        scalar = cpu_baseline(wl, meta, sample_requests=16)
        out["cpu_baseline"] = cpu_reference_config1(a.seed)
        # second figure: the scalar C port on a sample of the benched configuration itself
        out["cpu_baseline"]["scalar_port_on_benched_config"] = scalar
    del wl, last_ctx
    torch.cuda.empty_cache()
    if not a.no_prefill:
        out["prefill"] = prefill_section(a.seed)
        torch.cuda.empty_cache()
    if not a.no_mixed:
        out["mixed"] = mixed_section(a.seed)
        torch.cuda.empty_cache()
    if not a.no_page8 and P == 16:
        out["page8"] = page8_in_child(a.seed)
    if not a.no_swap:
        # three processes in a row: whether a swap overlaps with compute used to depend on the
        # process (which hardware queue its streams were given); the figures of all three are kept
        procs = [run_section_in_child("swap", a.seed) for _ in range(3)]
        out["swap"] = procs[0]
        out["swap"]["three_processes"] = {
            "exchange_overlapped_GBps_each_way": [p["exchange_overlapped_GBps_each_way"] for p in procs],
            "frac_of_host_link_overlapped": [p["frac_of_host_link_overlapped"] for p in procs],
            "decode_slowdown": [p["decode_slowdown"] for p in procs]}
    if not a.no_fragmented:
        out["fragmented"] = run_section_in_child("fragmented", a.seed)
    print(json.dumps(out))
    return 0


if __name__ == "__main__":
    sys.exit(main())

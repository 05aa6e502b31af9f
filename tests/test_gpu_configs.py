"""The baseline configurations at their FULL sizes on one MI355X.  The CPU oracle
cannot redo gigabytes in seconds, so parity is shown through (a) the oracle on a
seeded sample of requests / query rows, (b) size-independent properties:
append -> read-back identity plus a checksum of everything that must not change,
swap round trips that must restore every bit, and invariance of attention under
relocation of the pages."""
import numpy as np
import pytest
import torch

from kvutil import max_rel_err_per_request
from oracle import c_oracle
from oracle import kv_oracle as orc


pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


def _announce(*what):
    print("[case]", *what, flush=True)


def _checksum(t: torch.Tensor) -> int:
    """Order-independent 64-bit sum of the raw 16-bit words."""
    return int(t.contiguous().view(torch.int16).to(torch.int64).sum().item())


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _decode_step(wl, wrapper, layers, fused=False, rope=False):
    """One engine-style decode step over the given layers; returns (ctx, {layer: out}).
    fused: the attention launch writes the step's token itself (the form the bench times);
    rope (with fused): it also rotates q and the new k at the tokens' positions."""
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.paged_ops import append_paged_kv_cache

    a = wl.args
    ctx = FlashDecodeCtx.init_paged_decode_ctx(wl.tasks, wl.caches, wrapper)
    wrapper.begin_forward(indptr=ctx.kv_page_indptr, indices=ctx.kv_page_indices,
                          last_page_len=ctx.kv_last_page_lens, num_qo_heads=a.n_heads,
                          num_kv_heads=a.n_kv_heads, head_dim=a.dim // a.n_heads, page_size=a.page_size,
                          indptr_host=ctx.host["kv_page_indptr"],
                          last_page_len_host=ctx.host["kv_last_page_lens"], indices_host=ctx.host["kv_page_indices"])
    outs = {}
    for layer in layers:
        pages = wl.pool.get_layered_pages(layer)
        if fused:
            extra = dict(rope_offsets=ctx.offsets, rope_theta=5e5) if rope else {}
            outs[layer] = wrapper.forward(wl.q[layer], pages, k_append=wl.k[layer], v_append=wl.v[layer],
                                          **extra)
        else:
            append_paged_kv_cache(wl.k[layer], wl.v[layer], ctx.indptr, pages, ctx.kv_page_indices,
                                  ctx.kv_page_indptr, ctx.kv_last_page_lens)
            outs[layer] = wrapper.forward(wl.q[layer], pages)
    plan_shape = (wrapper._n_items, wrapper._n_workgroups)
    wrapper.end_forward()
    torch.cuda.synchronize()
    return ctx, outs, plan_shape


def _oracle_rows(wl, ctx, layer, requests, q_bits=None):
    """fp32 oracle output (C port, fp32 accumulation) of the given requests, in their order:
    their pages are copied to the host as one compact array and attended in one call.
    q_bits: (B, Hq, D) bf16 bit patterns to use instead of the workload's q of the layer."""
    indptr, ids_all = ctx.host["kv_page_indptr"].numpy(), ctx.host["kv_page_indices"].numpy()
    last = ctx.host["kv_last_page_lens"].numpy()
    requests = np.asarray(list(requests), dtype=np.int64)
    ids = np.concatenate([ids_all[indptr[b]: indptr[b + 1]] for b in requests])
    local_indptr = np.concatenate([[0], np.cumsum(indptr[requests + 1] - indptr[requests])]).astype(np.int32)
    pages = _bits(wl.pool.pages[layer].index_select(0, torch.from_numpy(ids.astype(np.int64)).to(DEV)))
    if q_bits is None:
        q_bits = _bits(wl.q[layer])
    return c_oracle.decode_attn(np.ascontiguousarray(q_bits[requests]), pages,
                                np.arange(len(ids), dtype=np.int32), local_indptr,
                                np.ascontiguousarray(last[requests]), "bf16")


def _check_append(wl, ctx, layer, before_sum, old_rows):
    """The new rows read back through the block table equal k/v bit for bit, and the
    checksum of the whole layer moved by exactly (new rows - old rows)."""
    P = wl.args.page_size
    indptr, ids_all = ctx.host["kv_page_indptr"].numpy(), ctx.host["kv_page_indices"].numpy()
    last = ctx.host["kv_last_page_lens"].numpy()
    page = torch.from_numpy(ids_all[indptr[1:] - 1].astype(np.int64)).to(DEV)
    slot = torch.from_numpy((last - 1).astype(np.int64)).to(DEV)
    got = wl.pool.pages[layer][page, :, slot]                       # (B, 2, Hkv, D)
    assert torch.equal(got[:, 0].view(torch.int16), wl.k[layer].view(torch.int16))
    assert torch.equal(got[:, 1].view(torch.int16), wl.v[layer].view(torch.int16))
    delta = _checksum(wl.k[layer]) + _checksum(wl.v[layer]) - old_rows
    assert _checksum(wl.pool.pages[layer]) == before_sum + delta, "bytes outside the new rows changed"


def _old_rows_sum(wl, layer):
    """Checksum of the slots the next append will overwrite (position start_pos of every request)."""
    P = wl.args.page_size
    total = 0
    pages, slots = [], []
    for t, c in zip(wl.tasks, wl.caches):
        c.extend(t.start_pos + 1)                     # what prepare() will do
        pages.append(int(c.page_table.retrieve()[t.start_pos // P]))
        slots.append(t.start_pos % P)
    rows = wl.pool.pages[layer][torch.tensor(pages, device=DEV), :, torch.tensor(slots, device=DEV)]
    return _checksum(rows)


def _check_rope_append(wl, ctx, layer, before_sum, old_rows):
    """After the launch that rotates and appends: the new V rows equal v bit for bit, the new
    K rows are the oracle's rotation of k at the tokens' positions to within one bf16 ulp, and
    the checksum of the layer moved by exactly (new rows - old rows).  Returns the K rows as
    the device wrote them."""
    indptr, ids_all = ctx.host["kv_page_indptr"].numpy(), ctx.host["kv_page_indices"].numpy()
    last = ctx.host["kv_last_page_lens"].numpy()
    page = torch.from_numpy(ids_all[indptr[1:] - 1].astype(np.int64)).to(DEV)
    slot = torch.from_numpy((last - 1).astype(np.int64)).to(DEV)
    got = wl.pool.pages[layer][page, :, slot]                       # (B, 2, Hkv, D)
    assert torch.equal(got[:, 1].view(torch.int16), wl.v[layer].view(torch.int16))
    k_ref = orc.rope_interleaved(orc.f32_from_bf16_bits(_bits(wl.k[layer])), ctx.host["indptr"].numpy(),
                                 ctx.host["offsets"].numpy())
    k_dev = orc.f32_from_bf16_bits(_bits(got[:, 0]))
    assert np.abs(k_dev - k_ref).max() <= 2.0 ** -7 * max(float(np.abs(k_ref).max()), 1.0)
    delta = _checksum(got) - old_rows
    assert _checksum(wl.pool.pages[layer]) == before_sum + delta, "bytes outside the new rows changed"


def test_config2_llama8b_stage_decode_step_full_size():
    """The step the bench times: the attention launch of every layer writes the step's token
    itself, with the default plan (one persistent workgroup per CU, most requests cut).  Pages
    against the append's definition bit for bit; ALL 64 requests of three layers against the
    C oracle, each request against its own output scale.  Then the same with the rotation
    inside the launch on two more layers, and the append-then-attend pair on relocated pages."""
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.synthetic import config2_context_lengths, make_decode_workload

    _announce("config2 full size, fused append")
    wl = make_decode_workload("cfg2", config2_context_lengths(2), 16, 32, 8, 128, 16, torch.bfloat16,
                              headroom_tokens=32, seed=2)
    wrapper, _ = get_wrappers(DEV)
    B = wl.batch
    layers = [0, 7, 15]
    before = {l: _checksum(wl.pool.pages[l]) for l in layers}
    old = {l: _old_rows_sum(wl, l) for l in layers}
    ctx, outs, (n_items, n_wgs) = _decode_step(wl, wrapper, layers, fused=True)
    assert n_wgs == torch.cuda.get_device_properties(0).multi_processor_count
    assert n_items > B                                      # the plan of the bench: requests are cut
    for l in layers:
        _check_append(wl, ctx, l, before[l], old[l])
        want = _oracle_rows(wl, ctx, l, range(B))
        got = outs[l].float().cpu().numpy()
        assert np.isfinite(got).all()
        err = max_rel_err_per_request(got, want)
        _announce("config2 layer", l, "worst request error", err)
        assert err <= 2e-2, l
    # append-then-attend on the same pages gives the same bits (the token is there already),
    # also after relocating every page of the layer and renaming it in the block table
    perm = torch.randperm(wl.pool.num_pages, device=DEV)
    moved = torch.empty_like(wl.pool.pages[7])
    moved[perm] = wl.pool.pages[7]
    new_ids = perm[ctx.kv_page_indices.long()].to(torch.int32)
    for ids, pages in ((ctx.kv_page_indices, wl.pool.pages[7]), (new_ids, moved)):
        wrapper.begin_forward(indptr=ctx.kv_page_indptr, indices=ids, last_page_len=ctx.kv_last_page_lens,
                              num_qo_heads=32, num_kv_heads=8, head_dim=128, page_size=16,
                              indptr_host=ctx.host["kv_page_indptr"],
                              last_page_len_host=ctx.host["kv_last_page_lens"])    # ids are read back
        again = wrapper.forward(wl.q[7], pages)
        wrapper.end_forward()
        assert torch.equal(again.view(torch.int16), outs[7].view(torch.int16))
    del moved

    _announce("config2 full size, rotation + append inside the launch")
    for t in wl.tasks:
        t.step()
    layers = [3, 12]
    before = {l: _checksum(wl.pool.pages[l]) for l in layers}
    old = {l: _old_rows_sum(wl, l) for l in layers}
    ctx, outs, _ = _decode_step(wl, wrapper, layers, fused=True, rope=True)
    for l in layers:
        _check_rope_append(wl, ctx, l, before[l], old[l])
        q_rot = orc.rope_interleaved(orc.f32_from_bf16_bits(_bits(wl.q[l])), ctx.host["indptr"].numpy(),
                                     ctx.host["offsets"].numpy())
        want = _oracle_rows(wl, ctx, l, range(B), q_bits=orc.bf16_bits_from_f32(q_rot))
        got = outs[l].float().cpu().numpy()
        err = max_rel_err_per_request(got, want)
        _announce("config2 layer", l, "worst request error with rotation", err)
        assert np.isfinite(got).all() and err <= 2e-2, l


def test_config3_microbatch_exchange_round_trip_full_size():
    """4648+ scattered pages x 10 layers (~3 GB) out and back in: every bit restored,
    while the pages of the resident microbatch are never touched."""
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty
    from deserve_amd.synthetic import fill_normal, scatter_pool_order

    _announce("config3 full size")
    L, P = 10, 16
    rng = np.random.default_rng(3)
    n_mb = [int((-(-rng.integers(1024, 4097, size=32) // P)).sum()) for _ in range(2)]
    pool = GpuPagePool(L, sum(n_mb) + 100, P, DEV, torch.bfloat16)
    fill_normal(pool.pages, 3)
    scatter_pool_order(pool, 4)
    ids_a, ids_b = pool.alloc(n_mb[0]), pool.alloc(n_mb[1])
    sum_all = _checksum(pool.pages)
    image_a = pool.retrieve(ids_a)                                  # device copy (L, n, ...)
    sum_b = _checksum(pool.retrieve(ids_b))
    eng = _native.SwapEngine()
    shape = (L * n_mb[0],) + tuple(pool.pages.shape[2:])
    host_a, host_z = pinned_empty(shape, torch.bfloat16), pinned_empty(shape, torch.bfloat16)
    host_z.zero_()
    eng.exchange(host_a, host_z, pool, ids_a)                       # a goes out, zeros come in
    eng.wait()
    assert _checksum(pool.retrieve(ids_a)) == 0
    assert _checksum(pool.retrieve(ids_b)) == sum_b                 # resident microbatch untouched
    assert torch.equal(host_a.view(torch.int16).view(image_a.shape), image_a.cpu().view(torch.int16))
    eng.exchange(host_z, host_a, pool, ids_a)                       # and back
    eng.wait()
    assert torch.equal(pool.retrieve(ids_a).view(torch.int16), image_a.view(torch.int16))
    assert _checksum(pool.pages) == sum_all
    eng.close()


def test_config4_chunked_prefill_full_batch_all_layers():
    """16 sequences append a 512-token chunk behind a prior of U[0, 8192] tokens that ends
    mid-page (offset U[0, 15]), then attend causally over prior + chunk: all 16 layers of
    the stage; append read-back and checksum on every layer, sampled rows against the
    oracle on four of them."""
    from deserve_amd.kvcache.paged.kvcache import PagedKVCache
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.model.context.flash import FlashPrefillCtx
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper, append_paged_kv_cache
    from deserve_amd.synthetic import fill_normal, scatter_pool_order
    from deserve_amd.task import SamplingParams, TaskData

    _announce("config4")
    L, P, Hq, Hkv, D, B, n = 16, 16, 32, 8, 128, 16, 512
    rng = np.random.default_rng(4)
    prior = (rng.integers(0, 8193, size=B) // P) * P + rng.integers(0, 16, size=B)
    prior[0], prior[1] = 0, 8192 + 15                               # extremes: pure prompt, longest
    pool = GpuPagePool(L, int((-(-(prior + n) // P)).sum()) + 8, P, DEV, torch.bfloat16)
    fill_normal(pool.pages, 5)
    scatter_pool_order(pool, 6)
    rows = PageTableAllocator(B, 8192 + 1024, P, DEV)
    tasks = [TaskData(f"t{b}", int(prior[b]), 1, n, int(prior[b]) + n, SamplingParams()) for b in range(B)]
    caches = [PagedKVCache.empty(rows, pool) for _ in range(B)]
    g = torch.Generator(device=DEV)
    g.manual_seed(7)
    mk = lambda h: torch.randn((L, B * n, h, D), generator=g, device=DEV).to(torch.bfloat16)
    q, k, v = mk(Hq), mk(Hkv), mk(Hkv)
    w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(1 << 20, dtype=torch.uint8, device=DEV))
    ctx = FlashPrefillCtx.init_paged_prefill_ctx(tasks, caches, w)
    w.begin_forward(qo_indptr=ctx.indptr, paged_kv_indptr=ctx.kv_page_indptr,
                    paged_kv_indices=ctx.kv_page_indices, paged_kv_last_page_len=ctx.kv_last_page_lens,
                    num_qo_heads=Hq, num_kv_heads=Hkv, head_dim=D, page_size=P,
                    qo_indptr_host=ctx.host["indptr"],
                    paged_kv_indptr_host=ctx.host["kv_page_indptr"],
                    paged_kv_last_page_len_host=ctx.host["kv_last_page_lens"], paged_kv_indices_host=ctx.host["kv_page_indices"])
    before = [_checksum(pool.pages[l]) for l in range(L)]
    indptr, ids_all = ctx.host["kv_page_indptr"].numpy(), ctx.host["kv_page_indices"].numpy()
    # slots the chunk will overwrite: positions prior_b .. prior_b + n - 1
    pos = np.concatenate([np.arange(p, p + n) for p in prior])
    req = np.repeat(np.arange(B), n)
    page = torch.from_numpy(ids_all[indptr[req] + pos // P].astype(np.int64)).to(DEV)
    slot = torch.from_numpy((pos % P).astype(np.int64)).to(DEV)
    outs = []
    for l in range(L):
        old = _checksum(pool.pages[l][page, :, slot])
        append_paged_kv_cache(k[l], v[l], ctx.indptr, pool.pages[l], ctx.kv_page_indices,
                              ctx.kv_page_indptr, ctx.kv_last_page_lens)
        got = pool.pages[l][page, :, slot]
        assert torch.equal(got[:, 0].view(torch.int16), k[l].view(torch.int16))
        assert torch.equal(got[:, 1].view(torch.int16), v[l].view(torch.int16))
        assert _checksum(pool.pages[l]) == before[l] - old + _checksum(k[l]) + _checksum(v[l])
        outs.append(w.forward(q[l], pool.pages[l], causal=True))
    torch.cuda.synchronize()
    w.end_forward()
    # oracle on sampled query rows: row i of request b is decode attention over
    # prior_b + i + 1 tokens.  Per layer 16 rows: first and last row of the shortest and of
    # the longest prior (requests 0 and 1), a row that ends on a page boundary, and seeded ones
    # over all requests; every row against its own output scale.
    worst = 0.0
    for layer in (0, 5, 10, 15):
        assert np.isfinite(outs[layer].float().sum().item())
        picks = [(0, 0), (0, n - 1), (1, 0), (1, n - 1), (2, int((-prior[2] - 1) % P))]
        picks += [(int(rng.integers(0, B)), int(rng.integers(0, n))) for _ in range(11)]
        reqs = sorted({b for b, _ in picks})
        base, run = {}, 0
        for b in reqs:
            base[b] = run
            run += int(indptr[b + 1] - indptr[b])
        ids = np.concatenate([ids_all[indptr[b]: indptr[b + 1]] for b in reqs])
        pages = _bits(pool.pages[layer].index_select(0, torch.from_numpy(ids.astype(np.int64)).to(DEV)))
        tables, counts, lasts, rows_q = [], [], [], []
        for b, i in picks:
            limit = int(prior[b]) + i + 1
            npg = -(-limit // P)
            tables.append(base[b] + np.arange(npg, dtype=np.int32))
            counts.append(npg)
            lasts.append((limit - 1) % P + 1)
            rows_q.append(b * n + i)
        want = c_oracle.decode_attn(np.ascontiguousarray(_bits(q[layer])[rows_q]), pages,
                                    np.concatenate(tables), np.concatenate([[0], np.cumsum(counts)]),
                                    np.asarray(lasts), "bf16")
        got = outs[layer].float().cpu().numpy()
        assert np.isfinite(got).all()
        err = max_rel_err_per_request(got[rows_q], want)
        worst = max(worst, err)
        assert err <= 2e-2, (layer, picks)
    _announce("config4 worst sampled row error", worst)


def test_config5_fragmented_pool_swap_in_then_decode():
    """128 sequences with lognormal context lengths on a pool fragmented by evictions
    (40 % of the pages freed and re-allocated out of order); 25 % of the sequences are
    offloaded and reloaded into other pages before the decode step."""
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.kvcache.manager import KVCacheManager
    from deserve_amd.kvcache.paged.chunk_pool import CpuChunkPool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.kvcache.virtual import VirtualPagedKVCache, VirtualPagePool
    from deserve_amd.stage import KVStage, StageArgs
    from deserve_amd.synthetic import DecodeWorkload, config5_context_lengths, fill_normal
    from deserve_amd.task import SamplingParams, TaskData

    _announce("config5")
    L, P, Hq, Hkv, D, B = 10, 16, 64, 8, 128, 128
    rng = np.random.default_rng(5)
    ctx_lens = config5_context_lengths(5)
    ctx_lens[np.argmax(ctx_lens)], ctx_lens[np.argmin(ctx_lens)] = 32768, 64      # both clip bounds occur
    need = int((-(-(ctx_lens + 8) // P)).sum())
    pool = VirtualPagePool(L, int(need / 0.4 * 1.05) + 128, 0, P, DEV, torch.bfloat16)   # 40 % of it must hold everything
    fill_normal(pool.pages, 8)
    rows = PageTableAllocator(B + 40, 32768 + 64, P, DEV)
    # fragmentation: fill the pool with filler requests, free a seeded 40 % of all pages,
    # then allocate the real requests (they get the lowest free ids first = holes all over)
    filler = pool.alloc(pool.num_avails)
    freed = torch.from_numpy(rng.permutation(filler.numpy())[: int(0.4 * len(filler))].copy())
    pool.free(freed)
    tasks, caches = [], []
    order = rng.permutation(B)                         # out-of-order arrival
    made = {}
    for b in order:
        c = VirtualPagedKVCache.empty(rows, pool)
        c.extend(int(ctx_lens[b]))
        made[int(b)] = c
    for b in range(B):
        tasks.append(TaskData(f"t{b}", int(ctx_lens[b]), 1, 1, int(ctx_lens[b]), SamplingParams()))
        caches.append(made[b])
    ids0 = caches[0].page_table.retrieve().numpy()
    assert np.any(np.diff(ids0) != 1), "block table should be fragmented"
    mgr = KVCacheManager(pool, CpuChunkPool(L, 15, P, torch.bfloat16), rows)
    swapped = sorted(rng.choice(B, size=B // 4, replace=False).tolist())
    images = {b: pool.retrieve(caches[b].page_table.retrieve()) for b in swapped[:4]}
    handles = [mgr.copy_gpu_to_cpu(caches[b], tasks[b].task_id) for b in swapped]
    for b in swapped:
        caches[b].free()
    back = [mgr.copy_cpu_to_gpu(h, tasks[b].task_id) for h, b in zip(handles, swapped)]
    for h in handles:
        h.free()
    mgr.synchronize()
    for b, c in zip(swapped, back):
        caches[b] = c
    for b in swapped[:4]:
        assert torch.equal(pool.retrieve(caches[b].page_table.retrieve()).view(torch.int16),
                           images[b].view(torch.int16)), "swap-in changed the data"
    g = torch.Generator(device=DEV)
    g.manual_seed(9)
    mk = lambda h: torch.randn((L, B, h, D), generator=g, device=DEV).to(torch.bfloat16)
    args = StageArgs(n_heads=Hq, n_kv_heads=Hkv, dim=Hq * D, page_size=P, n_layers=L)
    wl = DecodeWorkload("cfg5", args, pool, rows, tasks, caches, KVStage(args, use_rope=False),
                        mk(Hq), mk(Hkv), mk(Hkv), ctx_lens)
    wrapper, _ = get_wrappers(DEV)
    # One layer with the append inside the attention launch (what the bench times): all 128
    # requests against the oracle.  A step later, one layer with the two calls: 16 requests -
    # the longest (32 k tokens, cut into dozens of parts), the shortest, four of the swapped
    # ones and seeded others
    sample = [int(np.argmax(ctx_lens)), int(np.argmin(ctx_lens))] + swapped[:2] + swapped[-2:]
    sample += [int(b) for b in rng.permutation(B) if int(b) not in sample][: 16 - len(sample)]
    assert ctx_lens.max() == 32768
    for layer, fused in ((4, True), (9, False)):
        before, old = _checksum(pool.pages[layer]), _old_rows_sum(wl, layer)
        ctx, outs, (n_items, _) = _decode_step(wl, wrapper, [layer], fused=fused)
        assert n_items > B
        _check_append(wl, ctx, layer, before, old)
        if fused:
            sample = list(range(B))       # the benched form: every request of the layer
        want = _oracle_rows(wl, ctx, layer, sample)
        got = outs[layer].float().cpu().numpy()
        assert np.isfinite(got).all()
        err = max_rel_err_per_request(got[sample], want)
        _announce("config5 layer", layer, "fused" if fused else "two calls", "worst request error", err)
        assert err <= 2e-2, (layer, fused)
        for t in tasks:
            t.step()


def test_mixed_step_full_size_through_batch_prefill():
    """The reference's usual step in its decode-first aggregated mode: 75 running requests
    (contexts U[256, 4096], one new token each) and one chunk that fills the 512-token budget
    over a prior of U[0, 4096] tokens, all through BatchPrefill (engine/microbatch/processor.py:
    116-145) at the Llama-3-8B stage shape (the chunk behind 4200 tokens, its tiles in parts)
    and at the 70B shape (behind 1500 tokens) - the planner runs both as one launch in which
    decode workgroups and query tiles share the compute units, as it does the 8B step in f16 on
    pages of 8 tokens - and a step of 8 running requests and a 504-token chunk, which it runs
    as tiles only.  EVERY row of the ragged output of
    two layers against the C oracle, each row against its own scale; the appended rows read
    back bit for bit; the layer's checksum moves by exactly the appended rows."""
    from deserve_amd.execution.exec import BatchPrefill, get_wrappers
    from deserve_amd.synthetic import make_mixed_workload, mixed_step_shape

    for tag, L, Hq in (("8B", 3, 32), ("70B", 2, 64), ("8B_few_rows", 2, 32), ("8B_page8_f16", 2, 32)):
        _announce("mixed step", tag)
        P, Hkv, D = (8 if tag == "8B_page8_f16" else 16), 8, 128          # 8 tokens: the page the reference deploys with
        dtype, dtype_name = (torch.float16, "f16") if tag == "8B_page8_f16" else (torch.bfloat16, "bf16")
        dctx, prior, lens = mixed_step_shape(11, decode_rows=8 if tag == "8B_few_rows" else 75)
        prior[0] = 4200 if tag == "8B" else 1500
        wl = make_mixed_workload("mixed" + tag, dctx, prior, lens, L, Hq, Hkv, D, P, dtype, seed=11)
        nnz, n_dec = wl.nnz, len(dctx)
        assert nnz == 512
        before = [_checksum(wl.pool.pages[l]) for l in range(L)]
        step = BatchPrefill((wl.q, wl.k, wl.v), wl.stage, wl.tasks, wl.caches)
        step.prepare()
        ctx = step.prefill_ctx
        _, w = get_wrappers(DEV)
        if tag == "8B_few_rows":     # a handful of decode rows: every row a tile of the usual launch
            assert w._info.layout == 0 and w._n_decode_rows == 0 and w._info.n_tile_rows == nnz
        else:                        # one launch, decode rows on the decode kernel's body, one merge pass
            assert w._info.layout == 1 and w._n_decode_rows == n_dec and w._info.n_tile_rows == nnz - n_dec
            assert w._n_splits > 1 or tag != "8B"
        indptr, ids_all = ctx.host["kv_page_indptr"].numpy(), ctx.host["kv_page_indices"].numpy()
        last, qo = ctx.host["kv_last_page_lens"].numpy(), ctx.host["indptr"].numpy()
        start = np.array([t.start_pos for t in wl.tasks])
        n_new = np.diff(qo)
        pos = np.concatenate([np.arange(s, s + n) for s, n in zip(start, n_new)])
        req = np.repeat(np.arange(len(wl.tasks)), n_new)
        page = torch.from_numpy(ids_all[indptr[req] + pos // P].astype(np.int64)).to(DEV)
        slot = torch.from_numpy((pos % P).astype(np.int64)).to(DEV)
        old = [_checksum(wl.pool.pages[l][page, :, slot]) for l in range(L)]
        result = step.step(ignore_eos=True).all_xs               # the stage's output (no sampling here)
        torch.cuda.synchronize()
        assert result.shape == (L, nnz, Hq * D)
        for l in range(L):
            got_rows = wl.pool.pages[l][page, :, slot]
            assert torch.equal(got_rows[:, 0].view(torch.int16), wl.k[l].view(torch.int16))
            assert torch.equal(got_rows[:, 1].view(torch.int16), wl.v[l].view(torch.int16))
            assert _checksum(wl.pool.pages[l]) == before[l] - old[l] + _checksum(wl.k[l]) + _checksum(wl.v[l])
        for l in (0, L - 1):
            pages = _bits(wl.pool.pages[l].index_select(0, torch.from_numpy(ids_all.astype(np.int64)).to(DEV)))
            want = c_oracle.prefill_attn(_bits(wl.q[l]), qo, pages, np.arange(len(ids_all), dtype=np.int32),
                                         indptr, last, dtype_name, causal=True)
            got = result[l].view(nnz, Hq, D).float().cpu().numpy()
            assert np.isfinite(got).all()
            err_dec = max_rel_err_per_request(got[:n_dec], want[:n_dec])
            err_chunk = max_rel_err_per_request(got[n_dec:], want[n_dec:])
            _announce("mixed", tag, "layer", l, "worst decode row", err_dec, "worst chunk row", err_chunk)
            assert err_dec <= 2e-2 and err_chunk <= 2e-2, (tag, l)
        del wl, result, step
        torch.cuda.empty_cache()

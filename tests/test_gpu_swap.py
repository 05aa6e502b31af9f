"""KV swap between HBM and pinned host memory on a real MI355X: bit-exact round
trips, host layouts as the reference defines them, and the manager / execution
layer driven the way the reference's engine drives them."""
import numpy as np
import pytest
import torch

from kvutil import max_rel_err_per_request
from oracle import kv_oracle as orc

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")


def _announce(*what):
    print("[case]", *what, flush=True)


def _same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and bool(np.array_equal(a.view(np.uint8), b.view(np.uint8)))


def _fill_random(t: torch.Tensor, seed: int) -> np.ndarray:
    """Random 16-bit patterns into a bf16/f16 tensor; returns the uint16 host image."""
    rng = np.random.default_rng(seed)
    bits = rng.integers(0, 2**16, size=tuple(t.shape), dtype=np.uint16)
    t.view(torch.int16).copy_(torch.from_numpy(bits.view(np.int16)))
    return bits


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def test_swap_slice_bulk_exchange_matches_oracle_layout():
    from deserve_amd.kvcache.virtual import CopiedPinnedMemory, VirtualPagePool

    _announce("swap2 bulk")
    L, main, swap, P = 4, 6, 5, 16
    pool = VirtualPagePool(L, main, swap, P, DEV, torch.bfloat16)
    image = _fill_random(pool.pages, 1)
    mems = [CopiedPinnedMemory(pool.calc_swap_size(), swap, DEV, torch.bfloat16) for _ in range(3)]
    host = [_fill_random(m.memory, 10 + i) for i, m in enumerate(mems)]
    # step 1: slice 1 (inactive) goes to mems[0], comes from mems[1]
    want = image.copy()
    h0, h1 = host[0].copy(), host[1].copy()
    orc.swap_slice(want, pool.slices[1], h0, h1)
    pool.swap2(mems[1], mems[0])
    pool.stream.synchronize(), pool.stream2.synchronize()
    assert _same_bits(_bits(pool.pages), want)
    assert _same_bits(_bits(mems[0].memory), h0)                  # (L, S, 2, P, 8, 128) image
    assert _same_bits(_bits(mems[0].memory).reshape(L, swap, -1), image[:, main + swap:].reshape(L, swap, -1))
    # step 2 (num_rounds == 2): dump to and refill from the SAME buffer leaves the slice unchanged
    pool.switch()
    before = _bits(pool.pages).copy()
    pool.swap2(mems[2], mems[2])
    pool.stream.synchronize(), pool.stream2.synchronize()
    assert _same_bits(_bits(pool.pages), before)
    assert _same_bits(_bits(mems[2].memory).reshape(L, swap, -1), before[:, main: main + swap].reshape(L, swap, -1))
    # single-stream form
    pool.swap(mems[0], mems[1])
    pool.stream.synchronize()
    assert _same_bits(_bits(pool.pages)[:, main: main + swap].reshape(L, swap, -1), h0.reshape(L, swap, -1))
    with pytest.raises(RuntimeError):
        bad = CopiedPinnedMemory(16, swap, DEV, torch.bfloat16)
        pool.swap2(bad, mems[0])


@pytest.mark.parametrize("staging_mib,n", [(1, 37), (64, 300)])
def test_swap_engine_scattered_pages_round_trip(staging_mib, n):
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty

    _announce("swap engine", staging_mib, n)
    L, P, num_pages = 3, 16, 400
    pool = GpuPagePool(L, num_pages, P, DEV, torch.bfloat16)
    image = _fill_random(pool.pages, 2)
    rng = np.random.default_rng(3)
    ids = rng.permutation(num_pages)[:n].astype(np.int32)
    eng = _native.SwapEngine(staging_mib << 20)
    host = pinned_empty((L * n,) + tuple(pool.pages.shape[2:]), torch.bfloat16)
    eng.swap_out(host, pool, torch.from_numpy(ids))
    eng.wait()
    assert _same_bits(_bits(host), orc.gather_pages(image, ids))          # layer major, table order
    # wipe the pages, swap them back in to other page ids
    pool.pages.zero_()
    ids2 = rng.permutation(num_pages)[:n].astype(np.int32)
    eng.swap_in(pool, host, torch.from_numpy(ids2))
    eng.fence()
    torch.cuda.synchronize()
    want = np.zeros_like(image)
    orc.scatter_pages(want, ids2, orc.gather_pages(image, ids))
    assert _same_bits(_bits(pool.pages), want)
    # exchange: pages go out to host_a and are refilled from host_b in one call
    host_a = pinned_empty(tuple(host.shape), torch.bfloat16)
    host_b = pinned_empty(tuple(host.shape), torch.bfloat16)
    b_bits = _fill_random(host_b, 4)
    now = _bits(pool.pages).copy()
    eng.exchange(host_a, host_b, pool, torch.from_numpy(ids2))
    eng.wait()
    assert _same_bits(_bits(host_a), orc.gather_pages(now, ids2))
    want = now.copy()
    orc.scatter_pages(want, ids2, b_bits)
    assert _same_bits(_bits(pool.pages), want)
    # same buffer both ways: pages unchanged, buffer holds their image
    eng.exchange(host_a, host_a, pool, torch.from_numpy(ids2))
    eng.wait()
    assert _same_bits(_bits(pool.pages), want) and _same_bits(_bits(host_a), orc.gather_pages(want, ids2))
    eng.close()


def test_swap_engine_refuses_page_ids_outside_the_pool():
    """The gather and scatter kernels index the pool by page id; a bad id is refused on the
    host, before anything is launched, and the engine keeps working."""
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty

    _announce("swap engine refusals")
    L, P, num_pages = 2, 16, 8
    pool = GpuPagePool(L, num_pages, P, DEV, torch.bfloat16)
    before = _fill_random(pool.pages, 7)
    eng = _native.SwapEngine(1 << 20)
    host = pinned_empty((L * 2,) + tuple(pool.pages.shape[2:]), torch.bfloat16)
    with pytest.raises(ValueError, match="page id"):
        eng.swap_out(host, pool, torch.tensor([1, num_pages], dtype=torch.int32))
    with pytest.raises(ValueError, match="page id"):
        eng.swap_in(pool, host, torch.tensor([-1, 2], dtype=torch.int32))
    with pytest.raises(ValueError, match="page id"):
        eng.exchange(host, host.clone().pin_memory(), pool, torch.tensor([0, 1 << 30], dtype=torch.int32))
    eng.wait()
    assert _same_bits(_bits(pool.pages), before)
    ids = torch.tensor([1, 5], dtype=torch.int32)
    eng.swap_out(host, pool, ids)
    eng.wait()
    assert _same_bits(_bits(host), orc.gather_pages(before, ids.numpy()))
    eng.close()


def test_manager_offload_reload_keeps_bits_and_reference_call_order():
    from deserve_amd.kvcache.manager import KVCacheManager
    from deserve_amd.kvcache.paged.chunk_pool import CpuChunkPool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.kvcache.virtual import VirtualPagedKVCache, VirtualPagePool

    _announce("manager offload/reload")
    L, P = 3, 16
    pool = VirtualPagePool(L, 80, 20, P, DEV, torch.float16)
    image = _fill_random(pool.pages, 5)
    rows = PageTableAllocator(8, 4096, P, DEV)
    chunks = CpuChunkPool(L, 8, P, torch.float16)
    mgr = KVCacheManager(pool, chunks, rows, staging_bytes=2 << 20)
    caches = {}
    for name, tokens in (("a", 333), ("b", 16), ("c", 1000)):
        c = VirtualPagedKVCache.empty(rows, pool)
        c.extend(tokens)
        caches[name] = c
    ids = {k: c.page_table.retrieve().clone() for k, c in caches.items()}
    # the microbatch engine's order: copy all, then free all (engine/microbatch/processor.py:62-75)
    handles = {k: mgr.copy_gpu_to_cpu(caches[k], k) for k in ("a", "c")}
    for k in ("a", "c"):
        caches[k].free()
    mgr.synchronize()
    for k in ("a", "c"):
        n = len(ids[k])
        assert handles[k].initial_size == n
        assert _same_bits(_bits(handles[k].retrieve()[: L * n]), orc.gather_pages(image, ids[k].numpy()))
    # overwrite the freed pages, as another request would
    pool.pages[:, torch.cat([ids["a"], ids["c"]]).long()] = 0
    back = {k: mgr.copy_cpu_to_gpu(handles[k], k) for k in ("c", "a")}
    for k in ("c", "a"):
        handles[k].free()
    mgr.synchronize()
    for k in ("a", "c"):
        new_ids = back[k].page_table.retrieve()
        assert back[k].page_table.occupied == len(ids[k])
        got = _bits(pool.retrieve(new_ids))
        assert _same_bits(got.reshape(L * len(new_ids), -1), orc.gather_pages(image, ids[k].numpy()).reshape(L * len(new_ids), -1))
        assert torch.equal(back[k].isswap[: len(new_ids)], new_ids >= pool.num_pages_main)
    assert chunks.available_ids == [[] for _ in range(7)] + [[0]]           # every chunk returned
    assert _same_bits(_bits(pool.retrieve(ids["b"])), orc.gather_pages(image, ids["b"].numpy()).reshape(L, -1, 2, P, 8, 128))


def test_execution_layer_decode_and_chunked_prefill_steps_match_oracle():
    """BatchPrefill (first chunk, then second chunk) followed by BatchDecode steps over a
    2-layer stage, with RoPE; the pool contents and outputs follow the oracle."""
    from deserve_amd.execution.exec import BatchDecode, BatchPrefill
    from deserve_amd.kvcache.paged.kvcache import PagedKVCache
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.stage import KVStage, StageArgs
    from deserve_amd.task import SamplingParams, TaskData

    _announce("exec layer")
    L, P, Hq, Hkv, D = 2, 16, 32, 8, 128
    rng = np.random.default_rng(7)
    pool = GpuPagePool(L, 64, P, DEV, torch.bfloat16)
    pool.pages.zero_()
    rows = PageTableAllocator(4, 1024, P, DEV)
    stage = KVStage(StageArgs(n_heads=Hq, n_kv_heads=Hkv, dim=Hq * D, page_size=P, n_layers=L))
    prompts = [45, 20]
    tasks = [TaskData.empty(f"t{i}", n, SamplingParams()) for i, n in enumerate(prompts)]
    caches = [PagedKVCache.empty(rows, pool) for _ in prompts]
    ref_pages = np.zeros(tuple(pool.pages.shape), np.uint16)
    as_t = lambda a: torch.from_numpy(a.view(np.int16)).view(torch.bfloat16).to(DEV)
    bf = lambda a: orc.bf16_bits_from_f32(a)
    chunk_plan = [[30, 20], [15, 0], [1, 1], [1, 1]]          # per step: tokens per task (0 = idle)
    for step, lens in enumerate(chunk_plan):
        active = [i for i, n in enumerate(lens) if n > 0]
        for i in active:
            tasks[i].init(lens[i])
        nnz = sum(lens[i] for i in active)
        q = bf(rng.standard_normal((L, nnz, Hq, D)).astype(np.float32))
        k = bf(rng.standard_normal((L, nnz, Hkv, D)).astype(np.float32))
        v = bf(rng.standard_normal((L, nnz, Hkv, D)).astype(np.float32))
        decode = all(lens[i] == 1 for i in active)
        cls = BatchDecode if decode else BatchPrefill
        ex = cls((as_t(q), as_t(k), as_t(v)), stage, [tasks[i] for i in active], [caches[i] for i in active])
        ex.prepare()
        ctx = ex.decode_ctx if decode else ex.prefill_ctx
        res = ex.step(ignore_eos=True)
        torch.cuda.synchronize()
        assert res.all_task_ids == [tasks[i].task_id for i in active]
        got = res.all_xs.float().cpu().numpy().reshape(L, nnz, Hq, D)
        m = {n: ctx.host[n].numpy() for n in ctx.host}
        for layer in range(L):
            qr = bf(orc.rope_interleaved(orc.f32_from_bf16_bits(q[layer]), m["indptr"], m["offsets"]))
            kr = bf(orc.rope_interleaved(orc.f32_from_bf16_bits(k[layer]), m["indptr"], m["offsets"]))
            # the device's rope may round an element to the neighbouring bf16: append what the device wrote
            dev_pages = _bits(pool.pages[layer])
            orc.append_paged_kv(ref_pages[layer], kr, v[layer], m["indptr"], m["kv_page_indices"],
                                m["kv_page_indptr"], m["kv_last_page_lens"])
            # V rows are pure copies: bit-exact; K rows went through rope: within one bf16 ulp
            assert _same_bits(dev_pages[:, 1], ref_pages[layer][:, 1])
            kd = orc.f32_from_bf16_bits(dev_pages[:, 0])
            kw = orc.f32_from_bf16_bits(ref_pages[layer][:, 0])
            assert np.abs(kd - kw).max() <= 2.0 ** -7 * max(np.abs(kw).max(), 1.0)
            ref_pages[layer][:, 0] = dev_pages[:, 0]
            want = orc.prefill_attention(qr, m["indptr"], ref_pages[layer], m["kv_page_indices"],
                                         m["kv_page_indptr"], m["kv_last_page_lens"], "bf16")
            assert max_rel_err_per_request(got[layer], want) <= 2e-2, (step, layer)
        for i in active:
            tasks[i].step()
    assert [t.start_pos for t in tasks] == [47, 22]
    assert [c.page_table.occupied for c in caches] == [3, 2]


def test_graft_smoke_entry():
    import __graft_entry__ as g

    _announce("smoke")
    g.smoke()


def test_config3_exchange_overlapped_with_decode_is_bit_exact():
    """Baseline configuration 3 at full size: while the resident microbatch (32 sequences, 10
    layers, GQA 64q/8kv) runs decode steps whose attention launches append the step's token,
    one exchange carries the ~5000 scattered pages of the previous microbatch out to pinned
    memory and the next microbatch's in - twice in a row, so that four microbatch images are
    involved (resident, the one first in the slots, and two that arrive from the host).
    Ordering as the reference's engine fixes it: prepare, start the swap, step; join at the end
    (engine/microbatch/processor.py:124-131, engine/pipeline/processor.py:226-229).
    Checked: (i) what went out is the pages' content in layer-major, block-table order, (ii)
    the slots hold the incoming image, (iii) every decode output equals, bit for bit, that of
    the same steps run with no swap in flight, (iv) the resident layers changed only in the
    appended rows."""
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.synthetic import make_decode_workload

    _announce("config3 exchange under decode")
    L, Hq, Hkv, D, P, STEPS = 10, 64, 8, 128, 16, 12
    rng = np.random.default_rng(33)
    ctx_lens = [rng.integers(1024, 4097, size=32) for _ in range(4)]      # 4 microbatches
    n_swap = int(max((-(-c // P)).sum() for c in ctx_lens[1:]))           # slots of the exchanged ones
    wl = make_decode_workload("cfg3", ctx_lens[0], L, Hq, Hkv, D, P, torch.bfloat16,
                              headroom_tokens=2 * STEPS + 8, seed=33, spare_pages=n_swap + 64)
    pool = wl.pool
    ids = pool.alloc(n_swap)                                # scattered over the pool
    ids_dev = ids.to(DEV).long()
    shape = (L * n_swap,) + tuple(pool.pages.shape[2:])

    def host_image(seed):
        """Pinned image of a microbatch filled with seeded random bit patterns."""
        h = pinned_empty(shape, torch.bfloat16)
        g = torch.Generator(device=DEV).manual_seed(seed)
        for l in range(L):                                  # one layer at a time bounds device memory
            part = torch.randint(-32768, 32768, (n_swap,) + shape[1:], generator=g, device=DEV,
                                 dtype=torch.int16)
            h.view(torch.int16)[l * n_swap: (l + 1) * n_swap].copy_(part)
        return h

    images_in = [host_image(101), host_image(102)]
    images_out = [pinned_empty(shape, torch.bfloat16), pinned_empty(shape, torch.bfloat16)]
    w, _ = get_wrappers(DEV)
    eng = _native.SwapEngine(staging_bytes=images_in[0].numel() * 2)     # one chunk per direction
    # whether the runtime gave the engine queues of its own decides how much overlaps, not what
    # the bytes are: reported, not asserted
    _announce("engine streams run beside the compute stream:", eng.independent)

    def decode_step(outs):
        c = FlashDecodeCtx.init_paged_decode_ctx(wl.tasks, wl.caches, w)
        w.begin_forward(indptr=c.kv_page_indptr, indices=c.kv_page_indices,
                        last_page_len=c.kv_last_page_lens, num_qo_heads=Hq, num_kv_heads=Hkv,
                        head_dim=D, page_size=P, indptr_host=c.host["kv_page_indptr"],
                        last_page_len_host=c.host["kv_last_page_lens"], indices_host=c.host["kv_page_indices"])
        for layer in range(L):
            outs.append(w.forward(wl.q[layer], pool.get_layered_pages(layer), k_append=wl.k[layer],
                                  v_append=wl.v[layer]))
        w.end_forward()
        for t in wl.tasks:
            t.step()
        return c

    def rows_of_steps(first_pos, n_steps):
        """(page, slot) of the rows that n_steps steps append, for every request."""
        pages, slots = [], []
        for t, c, p0 in zip(wl.tasks, wl.caches, first_pos):
            c.extend(p0 + n_steps)
            row = c.page_table.retrieve().numpy()
            for pos in range(p0, p0 + n_steps):
                pages.append(int(row[pos // P]))
                slots.append(pos % P)
        return torch.tensor(pages, device=DEV), torch.tensor(slots, device=DEV)

    def checksum(t):
        return int(t.contiguous().view(torch.int16).to(torch.int64).sum().item())

    start = [t.start_pos for t in wl.tasks]
    # resident pages = everything the exchange must not touch
    resident = torch.ones(pool.num_pages, dtype=torch.bool, device=DEV)
    resident[ids_dev] = False
    res_ids = torch.nonzero(resident).flatten()
    page_r, slot_r = rows_of_steps(start, 2 * STEPS)
    sums_before = [checksum(pool.pages[l][res_ids]) for l in range(L)]
    old_rows = [checksum(pool.pages[l][page_r, :, slot_r]) for l in range(L)]
    first_image = pool.pages[:, ids_dev].contiguous()       # torch's own gather: (L, n, ...)

    overlapped, in_flight_after_decode = [], []
    for r in range(2):
        torch.cuda.synchronize()
        eng.exchange(images_out[r], images_in[r], pool, ids)          # enqueue-only
        for _ in range(STEPS):
            decode_step(overlapped)
        decode_done = torch.cuda.Event(enable_timing=True)
        decode_done.record()
        eng.fence()                                                   # the join
        swap_done = torch.cuda.Event(enable_timing=True)
        swap_done.record()
        torch.cuda.synchronize()
        in_flight_after_decode.append(decode_done.elapsed_time(swap_done))
    _announce("swap outlasted the decode steps by (ms; positive = they ran under it)", in_flight_after_decode)

    # (i) + (ii)
    as_i16 = lambda t: t.view(torch.int16)
    assert torch.equal(as_i16(images_out[0]).view(first_image.shape), as_i16(first_image).cpu())
    del first_image
    assert torch.equal(as_i16(images_out[1]), as_i16(images_in[0]))   # went in, came out again
    now = pool.pages[:, ids_dev].contiguous()
    assert torch.equal(as_i16(now).cpu().view(shape), as_i16(images_in[1]))
    del now
    # (iv) resident layers: only the appended rows moved, and they hold k / v
    for l in range(L):
        got = pool.pages[l][page_r, :, slot_r].view(len(wl.tasks), 2 * STEPS, 2, Hkv, D)
        assert torch.equal(as_i16(got[:, :, 0]), as_i16(wl.k[l])[:, None].expand(-1, 2 * STEPS, -1, -1))
        assert torch.equal(as_i16(got[:, :, 1]), as_i16(wl.v[l])[:, None].expand(-1, 2 * STEPS, -1, -1))
        assert checksum(pool.pages[l][res_ids]) == sums_before[l] - old_rows[l] + checksum(got), l
    # (iii) the same steps with nothing else on the GPU
    for t, p0 in zip(wl.tasks, start):
        t.start_pos = p0
    alone = []
    for _ in range(2 * STEPS):
        decode_step(alone)
    torch.cuda.synchronize()
    assert len(alone) == len(overlapped) == 2 * STEPS * L
    for i, (a, b) in enumerate(zip(alone, overlapped)):
        assert torch.equal(as_i16(a), as_i16(b)), ("step", i // L, "layer", i % L)
    # and they are right: last step, one layer, every request against the oracle
    from oracle import c_oracle
    for t in wl.tasks:                                       # rebuild the metadata of the last step
        t.start_pos -= 1
    c = FlashDecodeCtx.init_paged_decode_ctx(wl.tasks, wl.caches, w)
    indptr, ids_all = c.host["kv_page_indptr"].numpy(), c.host["kv_page_indices"].numpy()
    layer = L - 1
    pages = _bits(pool.pages[layer].index_select(0, torch.from_numpy(ids_all.astype(np.int64)).to(DEV)))
    want = c_oracle.decode_attn(_bits(wl.q[layer]), pages, np.arange(len(ids_all), dtype=np.int32),
                                indptr, c.host["kv_last_page_lens"].numpy(), "bf16")
    got = overlapped[-1].float().cpu().numpy()
    assert max_rel_err_per_request(got, want) <= 2e-2
    eng.close()


def test_swap_calls_never_block_on_a_full_id_ring():
    """The engine keeps the page ids of calls in flight in a ring of 2^20 entries.  With the
    engine held up behind a (bounded) sleeping kernel, the call that no longer fits is
    refused with an error instead of waiting inside an enqueue-only call; once the earlier
    calls have run, the same call goes through, and every byte arrives."""
    from deserve_amd.kvcache import _native
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.pinned.pinned_memory import pinned_empty

    _announce("swap id ring")
    n = 300_000                                                     # ids per call; 3 calls fit the ring
    pool = GpuPagePool(1, 64, 1, DEV, torch.float16, n_kv_heads=1, head_dim=4)      # 16-byte pages
    bits = _fill_random(pool.pages, 77)
    ids = torch.from_numpy(np.random.default_rng(78).integers(0, 64, size=n).astype(np.int32))
    hosts = [pinned_empty((n, 2, 1, 1, 4), torch.float16) for _ in range(4)]
    eng = _native.SwapEngine(8 << 20)
    torch.cuda.synchronize()
    torch.cuda._sleep(50_000_000)              # 25 ms at the shader clock, 0.5 s at a 100 MHz counter
    for h in hosts[:3]:
        eng.swap_out(h, pool, ids)                                  # wait (on the device) for the sleep
    # The fourth call finds the ring held by the three before it - as long as they are still
    # behind the sleeping kernel, which depends on clocks and host speed, not on the code under
    # test.  A refusal proves by itself that the call did not wait for room.
    try:
        eng.swap_out(hosts[3], pool, ids)
        refused = False
    except RuntimeError as err:
        assert "ring" in str(err)
        refused = True
    eng.wait()
    assert eng.done()
    if refused:
        eng.swap_out(hosts[3], pool, ids)                           # the same call, now that there is room
        eng.wait()
    want = bits[0][ids.numpy()]
    for h in hosts:
        assert _same_bits(_bits(h), want)
    eng.close()
    if not refused:
        pytest.skip("the engine drained before the ring filled: the refusal was not exercised on this box")

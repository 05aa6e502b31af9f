"""The stage driver in the reference's call order (synchronize/switch -> adjust ->
cancel/offload/reload -> join -> prepare -> swap2 -> forward) over rotating
microbatches: every microbatch must see exactly its own KV, whichever swap slice
it currently lives in.  Expected outputs come from a shadow copy of each
request's K/V rows kept in numpy, independent of any page layout."""
import numpy as np
import pytest
import torch

from kvutil import max_rel_err_per_request
from oracle import kv_oracle as orc

pytestmark = pytest.mark.gpu
DEV = torch.device("cuda")
L, P, HQ, HKV, D = 2, 16, 32, 8, 128


def _bf(x):
    return orc.bf16_bits_from_f32(x)


def _to_dev(bits):
    return torch.from_numpy(bits.view(np.int16)).view(torch.bfloat16).to(DEV)


class Shadow:
    """Per request and layer: all K/V rows appended so far (bf16 bit patterns)."""

    def __init__(self):
        self.k = {}
        self.v = {}

    def expect(self, tid, layer, q_bits, k_bits, v_bits):
        key = (tid, layer)
        self.k[key] = np.concatenate([self.k.get(key, np.zeros((0, HKV, D), np.uint16)), k_bits])
        self.v[key] = np.concatenate([self.v.get(key, np.zeros((0, HKV, D), np.uint16)), v_bits])
        T, n = self.k[key].shape[0], q_bits.shape[0]
        npg = -(-T // P)
        kk = np.zeros((npg * P, HKV, D), np.uint16)
        vv = np.zeros((npg * P, HKV, D), np.uint16)
        kk[:T], vv[:T] = self.k[key], self.v[key]
        pages = np.stack([kk.reshape(npg, P, HKV, D), vv.reshape(npg, P, HKV, D)], axis=1)
        return orc.prefill_attention(q_bits, np.array([0, n], np.int32), pages,
                                     np.arange(npg, dtype=np.int32), np.array([0, npg], np.int32),
                                     np.array([(T - 1) % P + 1], np.int32), "bf16", causal=True)


@pytest.mark.parametrize("rounds", [2, 3, 4])
def test_rotating_microbatches_keep_their_kv(rounds):
    from deserve_amd.engine.pipeline.processor import PipelineProcessor, StepRequest
    from deserve_amd.stage import KVStage, StageArgs
    from deserve_amd.task import SamplingParams

    print("[case] engine rounds", rounds, flush=True)
    rng = np.random.default_rng(100 + rounds)
    stage = KVStage(StageArgs(n_heads=HQ, n_kv_heads=HKV, dim=HQ * D, page_size=P, n_layers=L),
                    use_rope=False)
    # a tiny main region forces every microbatch into the swap slices
    proc = PipelineProcessor(num_rounds=rounds, num_pages_main=3, num_pages_swap=24, page_size=P,
                             batch_size=2, layer_storage=stage, num_layers=L, buddy_height=6,
                             main_dtype=torch.bfloat16, max_context_len=512)
    proc.virtual_page_pool.pages.view(torch.int16).fill_(0x7FC0)      # NaN everywhere: stale reads show
    shadow = Shadow()
    prompts = {m: {f"m{m}r{r}": int(rng.integers(20, 90)) for r in range(2)} for m in range(rounds)}
    used_swap_pages = False
    for step in range(rounds * 6):
        m = step % rounds
        first = step < rounds
        ids = list(prompts[m].keys())
        seqlens = [prompts[m][t] if first else 1 for t in ids]
        nnz = sum(seqlens)
        q = _bf(rng.standard_normal((L, nnz, HQ, D)).astype(np.float32))
        k = _bf(rng.standard_normal((L, nnz, HKV, D)).astype(np.float32))
        v = _bf(rng.standard_normal((L, nnz, HKV, D)).astype(np.float32))
        req = StepRequest(microbatch_id=m, xs=(_to_dev(q), _to_dev(k), _to_dev(v)), exec_task_ids=ids,
                          exec_seqlens=seqlens,
                          init_tasks={t: (prompts[m][t], SamplingParams()) for t in ids} if first else {})
        proc.run_step(req)
        torch.cuda.synchronize()
        got = proc.last_result.all_xs.float().cpu().numpy().reshape(L, nnz, HQ, D)
        assert np.isfinite(got).all(), (step, "a stale or foreign page was read")
        pos = 0
        for t, n in zip(ids, seqlens):
            for layer in range(L):
                want = shadow.expect(t, layer, q[layer, pos: pos + n], k[layer, pos: pos + n],
                                     v[layer, pos: pos + n])
                assert max_rel_err_per_request(got[layer, pos: pos + n], want) <= 2e-2, (step, t, layer)
            pos += n
        for c in proc.microbatches[m].ongoing_paged_kvcaches.values():
            used_swap_pages |= bool(c.isswap[: c.page_table.occupied].any())
    assert used_swap_pages, "the scenario was meant to exercise the swap slices"
    proc.synchronize()


def test_offload_reload_and_cancel_through_the_stage_driver():
    from deserve_amd.engine.pipeline.processor import PipelineProcessor, StepRequest
    from deserve_amd.stage import KVStage, StageArgs
    from deserve_amd.task import SamplingParams

    print("[case] engine offload/reload", flush=True)
    rng = np.random.default_rng(7)
    stage = KVStage(StageArgs(n_heads=HQ, n_kv_heads=HKV, dim=HQ * D, page_size=P, n_layers=L),
                    use_rope=False)
    proc = PipelineProcessor(num_rounds=2, num_pages_main=40, num_pages_swap=8, page_size=P,
                             batch_size=4, layer_storage=stage, num_layers=L, buddy_height=6,
                             main_dtype=torch.bfloat16, max_context_len=512)
    shadow = Shadow()
    lens = {"a": 50, "b": 33, "c": 70}

    def run(m, ids, seqlens, init=False, **kw):
        nnz = sum(seqlens)
        q = _bf(rng.standard_normal((L, nnz, HQ, D)).astype(np.float32))
        k = _bf(rng.standard_normal((L, nnz, HKV, D)).astype(np.float32))
        v = _bf(rng.standard_normal((L, nnz, HKV, D)).astype(np.float32))
        req = StepRequest(m, (_to_dev(q), _to_dev(k), _to_dev(v)), ids, seqlens,
                          init_tasks={t: (lens[t], SamplingParams()) for t in ids} if init else {}, **kw)
        proc.run_step(req)
        torch.cuda.synchronize()
        got = proc.last_result.all_xs.float().cpu().numpy().reshape(L, nnz, HQ, D)
        pos = 0
        for t, n in zip(ids, seqlens):
            for layer in range(L):
                want = shadow.expect(t, layer, q[layer, pos: pos + n], k[layer, pos: pos + n],
                                     v[layer, pos: pos + n])
                assert max_rel_err_per_request(got[layer, pos: pos + n], want) <= 2e-2, (t, layer)
            pos += n

    idle = lambda m, **kw: proc.run_step(StepRequest(m, None, **kw))
    run(0, ["a", "b", "c"], [50, 33, 70], init=True)
    idle(1)
    avail = proc.virtual_page_pool.num_avails
    run(0, ["a", "c"], [1, 1], offload_task_ids=["b"])              # b leaves for pinned memory
    assert "b" in proc.offloaded_kvcaches and proc.virtual_page_pool.num_avails >= avail + 3 - 2
    idle(1)
    run(0, ["a", "c"], [1, 1])
    idle(1)
    run(0, ["a", "b", "c"], [1, 1, 1], reload_task_ids=["b"])       # b comes back into other pages
    assert not proc.offloaded_kvcaches
    idle(1)
    run(0, ["a", "b"], [1, 1], cancel_task_ids=["c"])
    assert "c" not in proc.microbatches[0].ongoing_paged_kvcaches
    assert proc.cpu_chunk_pool.available_ids[-1] == [0]              # the chunk was returned


@pytest.mark.parametrize("policy", ["decode_first", "prefill_first", "vanilla"])
def test_scheduler_policies_under_page_pressure(policy):
    """Prompts arrive faster than the pool can hold them: the join stage batches, the
    swap stage evicts to pinned memory and reloads when cancelled tasks free pages.
    Whatever the policy decides, every executed token must attend to exactly its own
    request's history."""
    from deserve_amd.engine.pipeline.processor import StepRequest
    from deserve_amd.engine.pipeline.scheduler import PipelineScheduler
    from deserve_amd.stage import PackedKVStage, StageArgs
    from deserve_amd.task import SamplingParams

    print("[case] scheduler", policy, flush=True)
    rng = np.random.default_rng({"decode_first": 1, "prefill_first": 2, "vanilla": 3}[policy])
    stage = PackedKVStage(StageArgs(n_heads=HQ, n_kv_heads=HKV, dim=HQ * D, page_size=P, n_layers=L),
                          use_rope=False)
    sched = PipelineScheduler(num_rounds=2, num_pages_main=10, num_pages_swap=6, page_size=P,
                              batch_size=8, layer_storage=stage, num_layers=L, buddy_height=7,
                              main_dtype=torch.bfloat16, max_context_len=512,
                              decode_first_aggregate=policy == "decode_first",
                              prefill_first_aggregate=policy == "prefill_first",
                              max_aggregated_tokens=48)
    sched.virtual_page_pool.pages.view(torch.int16).fill_(0x7FC0)
    shadow = Shadow()
    width = HQ + 2 * HKV

    def rows(n):
        bits = _bf(rng.standard_normal((n, L, width, D)).astype(np.float32))
        return _to_dev(bits)

    def bits_of(x):
        return x.view(torch.int16).cpu().numpy().view(np.uint16)

    # prompts end just short of a page boundary and decode across one or two: the running
    # batch outgrows the 16 pages it was admitted into
    prompt_len = {f"t{i}": n for i, n in enumerate([30, 46, 62, 31, 47, 29, 45])}
    arrivals = {0: ["t0", "t1"], 1: ["t2"], 2: ["t3", "t4"], 5: ["t5"], 9: ["t6"]}
    decode_budget = {t: int(n) for t, n in zip(prompt_len, rng.integers(18, 30, size=7))}
    decoded = {t: 0 for t in prompt_len}
    finished, offloads, reloads = set(), 0, 0
    requests = [StepRequest.empty(m, torch.bfloat16, DEV) for m in range(2)]
    for step in range(400):
        for t in arrivals.get(step, []):
            sched.process_init(t, rows(prompt_len[t]), SamplingParams())
        m = step % 2
        req = requests[m]
        sched.synchronize()
        req = sched.process_step(req)
        torch.cuda.synchronize()
        offloads += len(req.offload_task_ids)
        reloads += len(req.reload_task_ids)
        ids, seqlens, xs = sched.last_exec
        if ids:
            got = sched.last_result.all_xs.float().cpu().numpy().reshape(L, sum(seqlens), HQ, D)
            assert np.isfinite(got).all(), (step, "a stale or foreign page was read")
            xb = bits_of(xs)
            pos = 0
            for t, n in zip(ids, seqlens):
                chunk = xb[pos: pos + n]
                for layer in range(L):
                    want = shadow.expect(t, layer, chunk[:, layer, :HQ], chunk[:, layer, HQ:HQ + HKV],
                                         chunk[:, layer, HQ + HKV:])
                    assert max_rel_err_per_request(got[layer, pos: pos + n], want) <= 2e-2, (step, t, layer)
                pos += n
        # a task that has produced its budget of tokens is cancelled on its next round;
        # one that is still prefilling has no next input yet and drops out of the batch
        keep, keep_rows, cancel = [], [], []
        for i, t in enumerate(req.exec_task_ids):
            d = sched.task_manager.get(t)
            if d.seqlen == 0:
                continue
            decoded[t] += 1
            if decoded[t] >= decode_budget[t]:
                cancel.append(t)
                finished.add(t)
            else:
                keep.append(t)
        req.exec_task_ids = keep
        req.xs = rows(len(keep)) if keep else torch.empty((0,), dtype=torch.bfloat16, device=DEV)
        req.cancel_task_ids = cancel
        requests[m] = req
        if len(finished) == len(prompt_len):
            break
    sched.synchronize()
    assert finished == set(prompt_len), (finished, decoded)
    assert offloads > 0 and reloads > 0, (offloads, reloads)


def test_graphed_decode_step_matches_eager_steps():
    """The decode step replayed as a HIP graph gives, step after step, the bits of the eager
    step: contexts grow across page boundaries between replays (new block-table entries, a
    new work list), eager launches run between replays, and a different batch re-captures."""
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.execution.graph import GraphedDecodeStep
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.stage import KVStage, StageArgs
    from deserve_amd.synthetic import make_decode_workload

    print("[case] graphed decode step", flush=True)
    Lg, B = 3, 6
    lens = np.array([13, 16, 300, 47, 1000, 31])
    args = dict(n_heads=HQ, n_kv_heads=HKV, dim=HQ * D, page_size=P, n_layers=Lg)

    def fresh(batch_lens, seed):
        return make_decode_workload("g", batch_lens, Lg, HQ, HKV, D, P, torch.bfloat16,
                                    headroom_tokens=96, seed=seed, fill=True)

    wl_e, wl_g = fresh(lens, 11), fresh(lens, 11)          # identical twins: eager and graphed
    assert torch.equal(wl_e.pool.pages.view(torch.int16), wl_g.pool.pages.view(torch.int16))
    stage = KVStage(StageArgs(**args), use_rope=True)
    wrapper, _ = get_wrappers(DEV)
    gwrapper = type(wrapper)(torch.empty(32 << 20, dtype=torch.uint8, device=DEV))
    step = GraphedDecodeStep(stage, gwrapper, max_batch=8, max_pages=4096, device=DEV,
                             num_qo_heads=HQ, num_kv_heads=HKV, head_dim=D, page_size=P,
                             target_workgroups=16)     # fixed: with fewer tiles than CUs the count would follow the tiles

    def eager(wl, xs):
        ctx = FlashDecodeCtx.init_paged_decode_ctx(wl.tasks, wl.caches, wrapper)
        wrapper.begin_forward(indptr=ctx.kv_page_indptr, indices=ctx.kv_page_indices,
                              last_page_len=ctx.kv_last_page_lens, num_qo_heads=HQ, num_kv_heads=HKV,
                              head_dim=D, page_size=P, indptr_host=ctx.host["kv_page_indptr"],
                              last_page_len_host=ctx.host["kv_last_page_lens"], target_workgroups=16)
        out = stage.forward(xs, ctx)
        wrapper.end_forward()
        return out

    gen = torch.Generator(device="cuda").manual_seed(5)
    for it in range(8):                                    # 8 tokens: requests 1, 3 and 5 open new pages
        n = len(wl_e.tasks)
        xs = tuple(torch.randn((Lg, n, h, D), device=DEV, generator=gen).to(torch.bfloat16)
                   for h in (HQ, HKV, HKV))
        want = eager(wl_e, xs).clone()
        got = step.run(xs, wl_g.tasks, wl_g.caches).clone()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), it
        assert torch.equal(wl_e.pool.pages.view(torch.int16), wl_g.pool.pages.view(torch.int16)), it
        for wl in (wl_e, wl_g):
            for t in wl.tasks:
                t.step()
        if it == 4:                                        # a request leaves: smaller batch, new capture
            for wl in (wl_e, wl_g):
                wl.caches.pop(2).free()
                wl.tasks.pop(2)
    assert step.captures == 2
    # the host running ahead of the GPU: steps enqueued back to back, no synchronisation
    # between them (the staging of a step must not be refilled under a pending copy)
    for it in range(20):
        n = len(wl_e.tasks)
        xs = tuple(torch.randn((Lg, n, h, D), device=DEV, generator=gen).to(torch.bfloat16)
                   for h in (HQ, HKV, HKV))
        want = eager(wl_e, xs)
        got = step.run(xs, wl_g.tasks, wl_g.caches)
        for wl in (wl_e, wl_g):
            for t in wl.tasks:
                t.step()
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    assert torch.equal(wl_e.pool.pages.view(torch.int16), wl_g.pool.pages.view(torch.int16))
    assert step.captures == 2 and len(step._graphs) == 2       # both batch shapes are held for replay


def test_joined_prepare_equals_context_then_begin_forward():
    """FlashDecodeCtx.init_and_plan (metadata and work list in one pinned block, one upload
    kernel) against init_paged_decode_ctx + begin_forward (one upload each): the same six
    arrays on the device, the same work list, the same launch shape, the same output bits."""
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.synthetic import make_decode_workload

    print("[case] joined prepare", flush=True)
    lens = np.array([13, 16, 300, 47, 1000, 31, 1, 4095])
    fresh = lambda: make_decode_workload("j", lens, 2, HQ, HKV, D, P, torch.bfloat16, headroom_tokens=64,
                                         seed=31, fill=True)
    wl_a, wl_b = fresh(), fresh()
    w_a, _ = get_wrappers(DEV)
    w_b = type(w_a)(torch.empty(32 << 20, dtype=torch.uint8, device=DEV))
    shape = dict(num_qo_heads=HQ, num_kv_heads=HKV, head_dim=D, page_size=P)
    for step in range(3):                                   # lengths 16 and 4095 cross a page boundary
        a = FlashDecodeCtx.init_paged_decode_ctx(wl_a.tasks, wl_a.caches, w_a)
        w_a.begin_forward(indptr=a.kv_page_indptr, indices=a.kv_page_indices, last_page_len=a.kv_last_page_lens,
                          indptr_host=a.host["kv_page_indptr"], last_page_len_host=a.host["kv_last_page_lens"],
                          indices_host=a.host["kv_page_indices"], target_workgroups=24, **shape)
        b = FlashDecodeCtx.init_and_plan(wl_b.tasks, wl_b.caches, w_b, target_workgroups=24, **shape)
        for f in ("indptr", "kv_page_indices", "kv_page_indptr", "kv_last_page_lens", "offsets", "seqlens"):
            assert torch.equal(getattr(a, f), getattr(b, f)), f
            assert torch.equal(getattr(b, f).cpu(), b.host[f]), f
        assert (w_a._n_items, w_a._n_workgroups, w_a._batch) == (w_b._n_items, w_b._n_workgroups, w_b._batch)
        assert torch.equal(w_a._plan[: w_b._plan.numel()], w_b._plan[: w_a._plan.numel()])
        assert torch.equal(w_b._indices, b.kv_page_indices) and torch.equal(w_b._indptr, b.kv_page_indptr)
        for layer in range(2):
            out_a = w_a.forward(wl_a.q[layer], wl_a.pool.pages[layer], k_append=wl_a.k[layer], v_append=wl_a.v[layer])
            out_b = w_b.forward(wl_b.q[layer], wl_b.pool.pages[layer], k_append=wl_b.k[layer], v_append=wl_b.v[layer])
            assert torch.equal(out_a.view(torch.int16), out_b.view(torch.int16)), (step, layer)
        w_a.end_forward()
        w_b.end_forward()
        for wl in (wl_a, wl_b):
            for t in wl.tasks:
                t.step()
    assert torch.equal(wl_a.pool.pages.view(torch.int16), wl_b.pool.pages.view(torch.int16))


def test_joined_prefill_prepare_equals_context_then_begin_forward():
    """FlashPrefillCtx.init_and_plan (metadata and plan in one pinned block, one upload kernel)
    against init_paged_prefill_ctx + begin_forward: the same six arrays on the device, the same
    plan (in parts per tile here: two chunks are few tiles), the same output bits."""
    from deserve_amd.kvcache.paged.kvcache import PagedKVCache
    from deserve_amd.kvcache.paged.page_pool import GpuPagePool
    from deserve_amd.kvcache.paged.page_table import PageTableAllocator
    from deserve_amd.model.context.flash import FlashPrefillCtx
    from deserve_amd.paged_ops import BatchPrefillWithPagedKVCacheWrapper
    from deserve_amd.synthetic import fill_normal
    from deserve_amd.task import SamplingParams, TaskData

    print("[case] joined prefill prepare", flush=True)
    prior, chunk = [1500, 37], [130, 64]
    shape = dict(num_qo_heads=HQ, num_kv_heads=HKV, head_dim=D, page_size=P)
    outs, ctxs, wrappers = [], [], []
    gen = torch.Generator(device="cuda").manual_seed(5)
    q = torch.randn((sum(chunk), HQ, D), device=DEV, generator=gen).to(torch.bfloat16)
    for joined in (False, True):
        pool = GpuPagePool(1, 200, P, DEV, torch.bfloat16)
        fill_normal(pool.pages, 77)
        rows = PageTableAllocator(2, 4096, P, DEV)
        tasks = [TaskData(f"j{b}", prior[b], 1, chunk[b], prior[b] + chunk[b], SamplingParams()) for b in range(2)]
        caches = [PagedKVCache.empty(rows, pool) for _ in range(2)]
        w = BatchPrefillWithPagedKVCacheWrapper(torch.empty(32 << 20, dtype=torch.uint8, device=DEV))
        if joined:
            c = FlashPrefillCtx.init_and_plan(tasks, caches, w, **shape)
        else:
            c = FlashPrefillCtx.init_paged_prefill_ctx(tasks, caches, w)
            w.begin_forward(qo_indptr=c.indptr, paged_kv_indptr=c.kv_page_indptr, paged_kv_indices=c.kv_page_indices,
                            paged_kv_last_page_len=c.kv_last_page_lens, qo_indptr_host=c.host["indptr"],
                            paged_kv_indptr_host=c.host["kv_page_indptr"],
                            paged_kv_last_page_len_host=c.host["kv_last_page_lens"],
                            paged_kv_indices_host=c.host["kv_page_indices"], **shape)
        outs.append(w.forward(q, pool.pages[0], causal=True))
        ctxs.append(c)
        wrappers.append(w)
    a, b = ctxs
    for f in ("indptr", "kv_page_indices", "kv_page_indptr", "kv_last_page_lens", "offsets", "seqlens"):
        assert torch.equal(getattr(a, f), getattr(b, f)), f
        assert torch.equal(getattr(b, f).cpu(), b.host[f]), f
    wa, wb = wrappers
    assert (wa._n_tiles, wa._n_splits, wa._batch, wa._nnz) == (wb._n_tiles, wb._n_splits, wb._batch, wb._nnz)
    assert wa._n_splits > 1
    n = min(wa._tiles.numel(), wb._tiles.numel())
    assert torch.equal(wa._tiles[:n], wb._tiles[:n])
    for x, y in ((wb._qo_indptr, b.indptr), (wb._indptr, b.kv_page_indptr), (wb._indices, b.kv_page_indices),
                 (wb._last, b.kv_last_page_lens)):
        assert torch.equal(x, y)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))


def test_graphed_decode_step_on_the_generic_kernel_follows_the_item_count():
    """head_dim 64 takes the generic attention kernel, which is launched with one workgroup
    per work item: a captured launch is only valid for its item count.  Contexts grow by a
    token per step so that the planner's item count changes between steps (5, then 7, ...);
    every replay must equal the eager step."""
    from deserve_amd.execution.exec import get_wrappers
    from deserve_amd.execution.graph import GraphedDecodeStep
    from deserve_amd.model.context.flash import FlashDecodeCtx
    from deserve_amd.stage import KVStage, StageArgs
    from deserve_amd.synthetic import make_decode_workload

    print("[case] graphed decode step, generic kernel", flush=True)
    Lg, hq, hkv, d = 2, 8, 2, 64
    lens = np.array([100, 37, 63, 15])
    fresh = lambda: make_decode_workload("gg", lens, Lg, hq, hkv, d, P, torch.bfloat16, headroom_tokens=64,
                                         seed=21, fill=True)
    wl_e, wl_g = fresh(), fresh()
    stage = KVStage(StageArgs(n_heads=hq, n_kv_heads=hkv, dim=hq * d, page_size=P, n_layers=Lg), use_rope=False)
    wrapper, _ = get_wrappers(DEV)
    gwrapper = type(wrapper)(torch.empty(8 << 20, dtype=torch.uint8, device=DEV))
    shape = dict(num_qo_heads=hq, num_kv_heads=hkv, head_dim=d, page_size=P)
    step = GraphedDecodeStep(stage, gwrapper, max_batch=4, max_pages=256, device=DEV, target_workgroups=4, **shape)
    gen = torch.Generator(device="cuda").manual_seed(6)
    counts = []
    for it in range(12):
        xs = tuple(torch.randn((Lg, 4, h, d), device=DEV, generator=gen).to(torch.bfloat16) for h in (hq, hkv, hkv))
        ctx = FlashDecodeCtx.init_paged_decode_ctx(wl_e.tasks, wl_e.caches, wrapper)
        wrapper.begin_forward(indptr=ctx.kv_page_indptr, indices=ctx.kv_page_indices,
                              last_page_len=ctx.kv_last_page_lens, indptr_host=ctx.host["kv_page_indptr"],
                              last_page_len_host=ctx.host["kv_last_page_lens"],
                              indices_host=ctx.host["kv_page_indices"], target_workgroups=4, **shape)
        assert not wrapper.fused_append_supported(torch.bfloat16)
        counts.append(wrapper._n_items)
        want = stage.forward(xs, ctx).clone()
        wrapper.end_forward()
        got = step.run(xs, wl_g.tasks, wl_g.caches).clone()
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (it, counts)
        assert torch.equal(wl_e.pool.pages.view(torch.int16), wl_g.pool.pages.view(torch.int16)), it
        for wl in (wl_e, wl_g):
            for t in wl.tasks:
                t.step()
    assert len(set(counts)) > 1, counts                     # the scenario did change the item count
    assert step.captures == len(set(counts))                # one capture per item count, replays otherwise


@pytest.mark.gpu
def test_staged_uploads_are_exact_and_blocks_wait_for_their_readers():
    """dskv_upload_words through the staging pool: every length (quads + tail words), and a
    host that refills blocks while earlier uploads are still queued behind a long kernel."""
    from deserve_amd import staging

    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    for words in (1, 3, 4, 5, 255, 1023, 1024, 1025, 100_001):
        src = rng.integers(-2**31, 2**31 - 1, size=words, dtype=np.int64).astype(np.int32)
        blk = staging.take(words)
        blk.tensor.numpy()[:words] = src
        dst = torch.full((words + 8,), 77, dtype=torch.int32, device=dev)
        staging.upload(blk, dst, words)
        got = dst.cpu().numpy()
        assert np.array_equal(got[:words], src) and np.all(got[words:] == 77), words
    # queue a long kernel, then 32 uploads whose blocks the host fills back to back
    busy = torch.empty((1 << 28,), dtype=torch.int32, device=dev)
    busy.zero_()
    outs, refs = [], []
    for i in range(32):
        src = rng.integers(0, 1 << 30, size=5000, dtype=np.int64).astype(np.int32)
        blk = staging.take(5000)
        blk.tensor.numpy()[:5000] = src
        outs.append(staging.to_device(blk, 5000, dev))
        refs.append(src)
        if i % 8 == 0:
            busy.add_(1)
    torch.cuda.synchronize()
    for o, r in zip(outs, refs):
        assert np.array_equal(o.cpu().numpy(), r)
    with pytest.raises(ValueError):
        staging.upload(staging.take(4), torch.zeros(2, dtype=torch.int32, device=dev), 4)


def test_step_request_with_device_tensors_crosses_the_stage_hop_bit_for_bit():
    """The stage hop (deserve_worker/request.py:199-210, engine/pipeline/processor.py:224): a
    StepRequest whose activations live on the GPU goes through into_safetensors -> dumps ->
    loads -> from_safetensors back onto the device.  The tensor that arrives has the bits of
    the one that left, the metadata is equal, and a decode step driven by what arrived gives
    the outputs and the pages of the same step driven by the original."""
    from deserve_amd import serde
    from deserve_amd.engine.pipeline.processor import StepRequest
    from deserve_amd.execution.exec import BatchDecode
    from deserve_amd.stage import PackedKVStage
    from deserve_amd.synthetic import make_decode_workload
    from deserve_amd.task import SamplingParams

    ctx_lens = [700, 33, 16, 1, 2049, 255, 4000, 90]
    sides = [make_decode_workload("hop", ctx_lens, L, HQ, HKV, D, P, torch.bfloat16, headroom_tokens=8, seed=21)
             for _ in range(2)]
    a, b = sides
    assert torch.equal(a.pool.pages.view(torch.int16), b.pool.pages.view(torch.int16))
    # one tensor per token, as the scheduler's queues carry it: (B, L, Hq + 2 Hkv, D)
    xs = torch.cat([a.q, a.k, a.v], dim=2).permute(1, 0, 2, 3).contiguous()
    ids = [t.task_id for t in a.tasks]
    req = StepRequest(3, xs, exec_task_ids=list(ids), exec_seqlens=[1] * len(ids), cancel_task_ids=["gone"],
                      offload_task_ids=[ids[1]], reload_task_ids=[],
                      init_tasks={ids[0]: (700, SamplingParams(temperature=0.5, max_new_tokens=7))})
    assert req.xs.is_cuda
    wire = serde.dumps(*req.into_safetensors())
    assert isinstance(wire, bytes) and len(wire) > req.get_tensors_size()
    back = StepRequest.from_safetensors(*serde.loads(wire), device=DEV)
    assert back.xs.is_cuda and back.xs.dtype == xs.dtype and back.xs.shape == xs.shape
    assert torch.equal(back.xs.view(torch.int16), xs.view(torch.int16))
    for name in ("microbatch_id", "exec_task_ids", "exec_seqlens", "cancel_task_ids", "offload_task_ids",
                 "reload_task_ids"):
        assert getattr(back, name) == getattr(req, name), name
    assert back.init_tasks[ids[0]][0] == 700 and back.init_tasks[ids[0]][1].model_dump() == \
        req.init_tasks[ids[0]][1].model_dump()
    outs = []
    for side, x in ((a, req.xs), (b, back.xs)):
        step = BatchDecode(x, PackedKVStage(side.args, use_rope=True), side.tasks, side.caches)
        step.prepare()
        outs.append(step.step(ignore_eos=True).all_xs)
    torch.cuda.synchronize()
    assert outs[0].shape == (L, len(ids), HQ * D)
    assert torch.equal(outs[0].view(torch.int16), outs[1].view(torch.int16))
    assert torch.equal(a.pool.pages.view(torch.int16), b.pool.pages.view(torch.int16))
    # an empty request keeps the reference's quirk on the way (a one-element stand-in) and comes back empty
    empty = StepRequest.from_safetensors(*serde.loads(serde.dumps(*StepRequest.empty(0, torch.bfloat16, DEV).into_safetensors())),
                                         device=DEV)
    assert empty.is_empty() and empty.xs.is_cuda and empty.xs.dtype == torch.bfloat16

"""Execution-layer objects (deserve_worker/execution/exec.py:20-22,58-243).

``prepare()`` builds the forward context (extending the caches) and plans the
attention; ``step()`` runs ``layer_storage.forward(xs, ctx)`` and closes the
plan.  ``layer_storage`` is whatever owns the layers of this stage: it must
offer ``forward(xs, ctx)``, ``model_args`` (n_heads, n_kv_heads, dim,
page_size) and ``need_sample`` (+ ``sample`` when true); the dense model itself
is outside this package.  The reference's module-level workspace and wrapper
pair become lazily created per-device singletons.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch

from deserve_amd.execution.result import BatchResult
from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.model.context.flash import FlashDecodeCtx, FlashPrefillCtx
from deserve_amd.paged_ops import (BatchDecodeWithPagedKVCacheWrapper,
                                   BatchPrefillWithPagedKVCacheWrapper)
from deserve_amd.task import TaskData

WORKSPACE_BYTES = 128 * 1024 * 1024
_wrappers: Dict[torch.device, Tuple[BatchDecodeWithPagedKVCacheWrapper,
                                    BatchPrefillWithPagedKVCacheWrapper]] = {}


def get_wrappers(device: torch.device):
    """(decode_wrapper, prefill_wrapper) sharing one 128 MiB workspace per device."""
    device = torch.device(device)
    if device not in _wrappers:
        ws = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=device)
        _wrappers[device] = (BatchDecodeWithPagedKVCacheWrapper(ws),
                             BatchPrefillWithPagedKVCacheWrapper(ws))
    return _wrappers[device]


@dataclass
class BatchExec:
    xs: torch.Tensor                 # ragged: one row per token of the batch
    layer_storage: object
    task_datas: List[TaskData]
    kvcaches: List[PagedKVCache]

    def bsz(self) -> int:
        return len(self.task_datas)

    def seqlens(self) -> List[int]:
        return [t.seqlen for t in self.task_datas]

    def total_seqlen(self) -> int:
        return sum(self.seqlens())

    @classmethod
    def merge(cls, execs: Sequence["BatchExec"]):
        return cls(torch.cat([e.xs for e in execs]), execs[0].layer_storage,
                   [t for e in execs for t in e.task_datas],
                   [c for e in execs for c in e.kvcaches])

    def split(self):
        out, pos = [], 0
        for task, cache in zip(self.task_datas, self.kvcaches):
            out.append(type(self)(self.xs[pos: pos + task.seqlen], self.layer_storage, [task],
                                  [cache]))
            pos += task.seqlen
        return out

    def pop(self):
        task, cache = self.task_datas.pop(), self.kvcaches.pop()
        tail = type(self)(self.xs[-task.seqlen:], self.layer_storage, [task], [cache])
        self.xs = self.xs[: -task.seqlen]
        return tail

    def post_process(self, result: torch.Tensor, ignore_eos: bool) -> BatchResult:
        ids = [t.task_id for t in self.task_datas]
        if not getattr(self.layer_storage, "need_sample", False):
            return BatchResult(result, ids, result, list(ids), [], {})
        ongoing_tok, ongoing, all_tok, all_datas, done, probs = self.layer_storage.sample(
            result, self.task_datas, ignore_eos)
        empty = torch.empty(0, dtype=torch.int, device=result.device)
        return BatchResult(torch.cat(ongoing_tok) if ongoing_tok else empty,
                           [t.task_id for t in ongoing],
                           torch.cat(all_tok) if all_tok else empty,
                           [t.task_id for t in all_datas], [t.task_id for t in done],
                           {t.task_id: p for t, p in probs})

    def _shape_kwargs(self) -> dict:
        a = self.layer_storage.model_args
        n_kv = a.n_heads if a.n_kv_heads is None else a.n_kv_heads
        return dict(num_qo_heads=a.n_heads, num_kv_heads=n_kv, head_dim=a.dim // a.n_heads,
                    page_size=a.page_size)


@dataclass
class BatchDecode(BatchExec):
    decode_ctx: Optional[FlashDecodeCtx] = None

    def prepare(self) -> None:
        with torch.inference_mode():
            wrapper, _ = get_wrappers(self.kvcaches[0].pool.main_device)
            # the context's index arrays and the attention work list go up in one kernel
            ctx = FlashDecodeCtx.init_and_plan(self.task_datas, self.kvcaches, wrapper,
                                               **self._shape_kwargs())
            self.decode_ctx = ctx

    def step(self, ignore_eos: bool) -> BatchResult:
        with torch.inference_mode():
            assert self.decode_ctx is not None
            result = self.layer_storage.forward(self.xs, self.decode_ctx)
            self.decode_ctx.decode_wrapper.end_forward()
            return self.post_process(result, ignore_eos)


@dataclass
class BatchPrefill(BatchExec):
    prefill_ctx: Optional[FlashPrefillCtx] = None

    def prepare(self) -> None:
        with torch.inference_mode():
            _, wrapper = get_wrappers(self.kvcaches[0].pool.main_device)
            # metadata and plan in one pinned block, one upload kernel
            self.prefill_ctx = FlashPrefillCtx.init_and_plan(self.task_datas, self.kvcaches, wrapper,
                                                             **self._shape_kwargs())

    def step(self, ignore_eos: bool) -> BatchResult:
        with torch.inference_mode():
            assert self.prefill_ctx is not None
            result = self.layer_storage.forward(self.xs, self.prefill_ctx)
            self.prefill_ctx.prefill_wrapper.end_forward()
            return self.post_process(result, ignore_eos)

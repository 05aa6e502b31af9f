"""Batch-forming policies (deserve_worker/engine/pipeline/stage/join.py:11-221).

All three work on the same three queues: prefills nobody has started
(`global_pending_prefills`: task id -> (tokens, SamplingParams)), prefills whose
remaining tokens wait on this worker (`local_suspended_prefills`) and decodes
waiting on this worker (`local_suspended_decodes`).  A prefill is admitted if its
whole prompt fits the page budget; only as many of its tokens run this step as
the batch has room for, the rest keeps waiting.  A decode is admitted if the
page its next token may need fits."""
from __future__ import annotations

from typing import Dict, Tuple

from deserve_amd.engine.pipeline.processor import StepRequest
from deserve_amd.task import TaskManager

from . import Stage, by_length


def _fill_with_prefills(stage, request: StepRequest, rest_pages: int, current_bs: int) -> Tuple[int, int]:
    """Chunked-prefill admission shared by the two aggregating policies: waiting
    remainders first (their pages are already accounted for), then new prompts,
    shortest first, until the batch holds max_batch_size tokens."""
    room = stage.max_batch_size
    if current_bs >= room:      # (the reference would append an empty chunk here and assert)
        return rest_pages, current_bs
    for task_id, x in by_length(stage.local_suspended_prefills):
        take = min(x.shape[0], room - current_bs)
        if take == x.shape[0]:
            del stage.local_suspended_prefills[task_id]
        else:
            stage.local_suspended_prefills[task_id] = x[take:]
        request.append_exec(task_id, x[:take], None)
        current_bs += take
        if current_bs == room:
            return rest_pages, current_bs
    pending = sorted(stage.global_pending_prefills.items(), key=lambda kv: kv[1][0].shape[0])
    for task_id, (x, sampling) in pending:
        need = stage.manager.calc_initial_space([task_id])
        if rest_pages < need:
            continue
        rest_pages -= need
        del stage.global_pending_prefills[task_id]
        take = min(x.shape[0], room - current_bs)
        if take < x.shape[0]:
            stage.local_suspended_prefills[task_id] = x[take:]
        request.append_exec(task_id, x[:take], (x.shape[0], sampling))
        current_bs += take
        if current_bs == room:
            break
    return rest_pages, current_bs


def _fill_with_decodes(stage, request: StepRequest, rest_pages: int, current_bs: int, room) -> Tuple[int, int]:
    """Waiting decodes in arrival order, each if the page its token may need fits."""
    for task_id, x in list(stage.local_suspended_decodes.items()):
        need = stage.manager.calc_extended_space([task_id])
        if rest_pages < need:
            continue
        assert x.shape[0] == 1
        rest_pages -= need
        current_bs += 1
        del stage.local_suspended_decodes[task_id]
        request.append_exec(task_id, x, None)
        if room is not None and current_bs == room:
            break
    return rest_pages, current_bs


def _park_decodes(stage, request: StepRequest) -> None:
    """The executing decodes step aside for a prefill batch."""
    for i, task_id in enumerate(request.exec_task_ids):
        stage.local_suspended_decodes[task_id] = request.xs[i:i + 1]


class DecodeFirstAgggregatedJoinStage(Stage):
    """Keeps the running decodes, tops the batch up with prefill chunks, then with
    waiting decodes (join.py:11-88)."""

    def __init__(self, manager: TaskManager, global_pending_prefills: Dict[str, tuple],
                 local_suspended_prefills: Dict[str, object], local_suspended_decodes: Dict[str, object],
                 max_batch_size: int) -> None:
        super().__init__(manager)
        self.global_pending_prefills = global_pending_prefills
        self.local_suspended_prefills = local_suspended_prefills
        self.local_suspended_decodes = local_suspended_decodes
        self.max_batch_size = max_batch_size
        self.max_extra_batch_size = max_batch_size

    def process(self, rest_pages: int, request: StepRequest) -> Tuple[int, StepRequest]:
        rest_pages -= self.manager.calc_extended_space(request.exec_task_ids)
        current_bs = request.get_bsz()
        if (self.global_pending_prefills or self.local_suspended_prefills) and rest_pages > 0:
            rest_pages, current_bs = _fill_with_prefills(self, request, rest_pages, current_bs)
        if current_bs < self.max_batch_size:
            rest_pages, current_bs = _fill_with_decodes(self, request, rest_pages, current_bs,
                                                        self.max_batch_size)
        return rest_pages, request


class PrefillFirstAgggregatedJoinStage(Stage):
    """If any prefill can run, the step is a prefill batch and the running decodes
    wait; otherwise the decodes go on.  Waiting decodes fill what room is left
    (join.py:91-175)."""

    def __init__(self, manager: TaskManager, global_pending_prefills: Dict[str, tuple],
                 local_suspended_prefills: Dict[str, object], local_suspended_decodes: Dict[str, object],
                 max_batch_size: int) -> None:
        super().__init__(manager)
        self.global_pending_prefills = global_pending_prefills
        self.local_suspended_prefills = local_suspended_prefills
        self.local_suspended_decodes = local_suspended_decodes
        self.max_batch_size = max_batch_size

    def process(self, rest_pages: int, request: StepRequest) -> Tuple[int, StepRequest]:
        current_bs = 0
        switched = False
        if self.global_pending_prefills or self.local_suspended_prefills:
            fresh = StepRequest.empty(request.microbatch_id, request.xs.dtype, request.xs.device)
            rest_pages, current_bs = _fill_with_prefills(self, fresh, rest_pages, 0)
            if fresh.exec_task_ids:
                _park_decodes(self, request)
                fresh.cancel_task_ids.extend(request.cancel_task_ids)
                request, switched = fresh, True
        if not switched:
            rest_pages -= self.manager.calc_extended_space(request.exec_task_ids)
        if current_bs < self.max_batch_size:
            rest_pages, current_bs = _fill_with_decodes(self, request, rest_pages, current_bs,
                                                        self.max_batch_size)
        return rest_pages, request


class VanillaJoinStage(Stage):
    """One whole prompt per step if one fits (the decodes wait meanwhile), else
    every decode that fits (join.py:178-221)."""

    def __init__(self, manager: TaskManager, global_pending_prefills: Dict[str, tuple],
                 local_suspended_decodes: Dict[str, object]) -> None:
        super().__init__(manager)
        self.global_pending_prefills = global_pending_prefills
        self.local_suspended_decodes = local_suspended_decodes

    def process(self, rest_pages: int, request: StepRequest) -> Tuple[int, StepRequest]:
        pending = sorted(self.global_pending_prefills.items(), key=lambda kv: kv[1][0].shape[0])
        for task_id, (x, sampling) in pending:
            need = self.manager.calc_initial_space([task_id])
            if rest_pages < need:
                continue
            rest_pages -= need
            del self.global_pending_prefills[task_id]
            fresh = StepRequest.empty(request.microbatch_id, request.xs.dtype, request.xs.device)
            fresh.append_exec(task_id, x, (x.shape[0], sampling))
            _park_decodes(self, request)
            fresh.cancel_task_ids.extend(request.cancel_task_ids)
            return rest_pages, fresh
        rest_pages -= self.manager.calc_extended_space(request.exec_task_ids)
        rest_pages, _ = _fill_with_decodes(self, request, rest_pages, 0, None)
        return rest_pages, request


# the reference's class names carry a typo; both spellings work
DecodeFirstAggregatedJoinStage = DecodeFirstAgggregatedJoinStage
PrefillFirstAggregatedJoinStage = PrefillFirstAgggregatedJoinStage

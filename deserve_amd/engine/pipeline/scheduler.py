"""First-stage driver: the step processor plus the policy stages that turn a
returning step request into the next batch
(deserve_worker/engine/pipeline/scheduler.py:20-168), without the request queue,
the HTTP relay and the trace path.

    process_init(task_id, x, sampling)   a new prompt joins the pending queue
    process_step(request)                refresh -> join stage -> swap stage -> PipelineProcessor.process_step
"""
from __future__ import annotations

from typing import Dict, List, Tuple

import torch

from deserve_amd.engine.pipeline.processor import PipelineProcessor, StepRequest
from deserve_amd.engine.pipeline.stage import Stage
from deserve_amd.engine.pipeline.stage.join import (DecodeFirstAgggregatedJoinStage,
                                                    PrefillFirstAgggregatedJoinStage,
                                                    VanillaJoinStage)
from deserve_amd.engine.pipeline.stage.swap import SwapStage
from deserve_amd.task import SamplingParams, TaskData


class PipelineScheduler(PipelineProcessor):
    def __init__(self, *args, prefill_first_aggregate: bool = False, decode_first_aggregate: bool = False,
                 max_aggregated_tokens: int = 512, **kwargs) -> None:
        super().__init__(*args, **kwargs)
        self.pending_prefills: Dict[str, Tuple[torch.Tensor, SamplingParams]] = {}
        self.offloaded_decodes: Dict[str, torch.Tensor] = {}
        self.offloaded_prefills: Dict[str, torch.Tensor] = {}
        tm = self.task_manager
        self.join_stages: List[Stage] = []
        for mb in self.microbatches:
            if decode_first_aggregate:
                stage: Stage = DecodeFirstAgggregatedJoinStage(
                    tm, self.pending_prefills, mb.suspended_prefills, mb.suspended_decodes,
                    max_aggregated_tokens)
            elif prefill_first_aggregate:
                stage = PrefillFirstAgggregatedJoinStage(
                    tm, self.pending_prefills, mb.suspended_prefills, mb.suspended_decodes,
                    max_aggregated_tokens)
            else:
                stage = VanillaJoinStage(tm, self.pending_prefills, mb.suspended_decodes)
            self.join_stages.append(stage)
        self.swap_stages: List[SwapStage] = [
            SwapStage(tm, mb.suspended_prefills, mb.suspended_decodes, self.offloaded_prefills,
                      self.offloaded_decodes) for mb in self.microbatches]

    def process_init(self, task_id: str, x: torch.Tensor, sampling_params: SamplingParams) -> None:
        self.task_manager.add(TaskData.empty(task_id, x.shape[0], sampling_params))
        self.pending_prefills[task_id] = (x, sampling_params)

    def convert_step_request(self, request: StepRequest) -> StepRequest:
        """Page budget of the step = free pages + what the cancelled tasks give back; the
        join stage spends it, the swap stage covers a deficit or uses a surplus."""
        rest_pages = (self.virtual_page_pool.num_avails
                      + self.task_manager.calc_occupied_space(request.cancel_task_ids))
        request.refresh()
        rest_pages, request = self.join_stages[request.microbatch_id].process(rest_pages, request)
        rest_pages, request = self.swap_stages[request.microbatch_id].process(rest_pages, request)
        return request

    def process_step(self, request: StepRequest) -> StepRequest:
        request = self.convert_step_request(request)
        for tid, (initial_seqlen, sampling) in request.init_tasks.items():
            if tid not in self.task_manager.task_datas:
                self.task_manager.add(TaskData.empty(tid, initial_seqlen, sampling))
        return super().process_step(request)

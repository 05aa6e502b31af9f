"""The per-step driver of one stage's KV path
(deserve_worker/engine/pipeline/processor.py:41-111, 226-301), without the parts
that are not on the path: no HTTP server, no weight download, no sampling
relay.  It builds the KV objects from the same sizes the reference's command
line gives, and `process_step` performs a step request in the reference's order:

    synchronize()   join the side streams of the previous step's bulk swap, switch slices
    adjust          (odd number of rounds only)
    init seqlens -> cancel -> offload -> reload -> kvcache_manager.synchronize()
    join new tasks -> microbatch.step(prepare -> swap2 -> forward) -> task.step()
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Tuple

import torch

from deserve_amd.engine.microbatch.processor import MicroBatchScheduler
from deserve_amd.execution.result import BatchResult
from deserve_amd.kvcache.manager import KVCacheManager
from deserve_amd.kvcache.paged.chunk_pool import ChunkHandle, CpuChunkPool
from deserve_amd.kvcache.paged.page_table import PageTableAllocator
from deserve_amd.kvcache.virtual import VirtualPagePool
from deserve_amd.task import SamplingParams, TaskData, TaskManager


@dataclass
class StepRequest:
    """Data of deserve_worker/request.py:137-146; into_safetensors / from_safetensors are the
    pair that deserve_amd.serde.dumps / loads put on the wire (request.py:199-210)."""
    microbatch_id: int
    xs: object
    exec_task_ids: List[str] = field(default_factory=list)
    exec_seqlens: List[int] = field(default_factory=list)
    cancel_task_ids: List[str] = field(default_factory=list)
    offload_task_ids: List[str] = field(default_factory=list)
    reload_task_ids: List[str] = field(default_factory=list)
    init_tasks: Dict[str, Tuple[int, SamplingParams]] = field(default_factory=dict)

    @staticmethod
    def empty(group_id: int, dtype: torch.dtype, device=None) -> "StepRequest":
        from deserve_amd.task import main_device
        return StepRequest(group_id, torch.empty((0,), dtype=dtype, device=device or main_device))

    def is_empty(self) -> bool:
        return (self.xs.numel() == 0 and not self.exec_task_ids and not self.exec_seqlens
                and not self.cancel_task_ids and not self.offload_task_ids
                and not self.reload_task_ids and not self.init_tasks)

    def append_exec(self, task_id: str, x: torch.Tensor, init_info=None) -> None:
        """Adds a task's tokens to the batch (request.py:172-188); init_info =
        (initial_seqlen, SamplingParams) for a task seen for the first time."""
        assert x.numel() > 0
        self.exec_task_ids.append(task_id)
        self.exec_seqlens.append(x.shape[0])
        self.xs = x if self.xs.numel() == 0 else torch.cat([self.xs, x], dim=0)
        if init_info is not None:
            self.init_tasks[task_id] = init_info

    def get_bsz(self) -> int:
        return len(self.exec_task_ids)

    def into_safetensors(self):
        return {"xs": self.xs}, {
            "group_id": self.microbatch_id,
            "exec_task_ids": self.exec_task_ids,
            "exec_seqlens": self.exec_seqlens,
            "cancel_task_ids": self.cancel_task_ids,
            "offload_task_ids": self.offload_task_ids,
            "reload_task_ids": self.reload_task_ids,
            "init_tasks": self.init_tasks,
        }

    @staticmethod
    def from_safetensors(tensors, metadata, device=None) -> "StepRequest":
        """Inverse of into_safetensors; xs is moved to `device` if one is given."""
        xs = tensors["xs"] if device is None else tensors["xs"].to(device)
        return StepRequest(metadata["group_id"], xs, list(metadata["exec_task_ids"]),
                           list(metadata["exec_seqlens"]), list(metadata["cancel_task_ids"]),
                           list(metadata["offload_task_ids"]), list(metadata["reload_task_ids"]),
                           dict(metadata["init_tasks"]))

    def get_tensors_size(self) -> int:
        return self.xs.numel() * self.xs.element_size()

    def refresh(self) -> None:
        """A request that comes round again carries only decodes (request.py:193-197)."""
        self.offload_task_ids = []
        self.reload_task_ids = []
        self.exec_seqlens = [1] * len(self.exec_task_ids)
        self.init_tasks = {}


class PipelineProcessor:
    def __init__(self, num_rounds: int, num_pages_main: int, num_pages_swap: int, page_size: int,
                 batch_size: int, layer_storage, num_layers: int, buddy_height: int,
                 ignore_eos: bool = True, main_device: torch.device = torch.device("cuda"),
                 main_dtype: torch.dtype = torch.float16, max_context_len: int = 4096,
                 n_kv_heads: int = 8, head_dim: int = 128) -> None:
        self.num_rounds, self.num_layers, self.max_batch_size = num_rounds, num_layers, batch_size
        self.cpu_chunk_pool = CpuChunkPool(num_layers, buddy_height, page_size, main_dtype,
                                           n_kv_heads, head_dim)
        self.virtual_page_pool = VirtualPagePool(num_layers, num_pages_main, num_pages_swap, page_size,
                                                 main_device, main_dtype, n_kv_heads, head_dim)
        self.page_table_allocator = PageTableAllocator(batch_size * num_rounds * 8, max_context_len,
                                                       page_size, main_device)
        self.kvcache_manager = KVCacheManager(self.virtual_page_pool, self.cpu_chunk_pool,
                                              self.page_table_allocator)
        self.task_manager = TaskManager(num_pages_main + num_pages_swap, page_size)
        self.offloaded_kvcaches: Dict[str, ChunkHandle] = {}
        self.layer_storage = layer_storage
        self.microbatches = [MicroBatchScheduler(self.kvcache_manager, self.task_manager, layer_storage,
                                                 self.page_table_allocator, ignore_eos)
                             for _ in range(num_rounds)]
        self.current_microbatch_id = 0
        self.ignore_eos = ignore_eos
        self.last_result: BatchResult = None   # type: ignore[assignment]
        self.last_exec = ([], [], None)        # what the last step ran: task ids, seqlens, inputs

    def synchronize(self) -> None:
        pool = self.virtual_page_pool
        pool.stream.synchronize()
        pool.stream2.synchronize()
        pool.switch()

    def run_step(self, request: StepRequest) -> StepRequest:
        """What the reference's run loop does for one StepRequest."""
        self.synchronize()
        for tid, (initial_seqlen, sampling) in request.init_tasks.items():
            self.task_manager.add(TaskData.empty(tid, initial_seqlen, sampling))
        return self.process_step(request)

    def process_step(self, request: StepRequest) -> StepRequest:
        mb = self.microbatches[request.microbatch_id]
        assert request.microbatch_id == self.current_microbatch_id
        self.current_microbatch_id = (self.current_microbatch_id + 1) % self.num_rounds
        if self.num_rounds % 2 == 1:
            mb.adjust()
        prev_mb = self.microbatches[(request.microbatch_id - 1) % self.num_rounds]
        next_mb = self.microbatches[(request.microbatch_id + 1) % self.num_rounds]

        for tid, seqlen in zip(request.exec_task_ids, request.exec_seqlens):
            self.task_manager.get(tid).init(seqlen)
        mb.cancel(request.cancel_task_ids)
        for tid, handle in zip(request.offload_task_ids, mb.offload(request.offload_task_ids)):
            self.offloaded_kvcaches[tid] = handle
        mb.reload(request.reload_task_ids,
                  [self.offloaded_kvcaches.pop(tid) for tid in request.reload_task_ids])
        mb.kvcache_manager.synchronize()

        self.last_exec = (list(request.exec_task_ids), list(request.exec_seqlens), request.xs)
        if request.exec_task_ids:
            mb.join(list(request.init_tasks.keys()))
            result = mb.step(request.exec_task_ids, request.xs, prev_mb, next_mb)
            for tid in request.exec_task_ids:
                self.task_manager.get(tid).step()
            self.last_result = result
            if getattr(self.layer_storage, "need_sample", False):
                request.cancel_task_ids = result.done_task_ids
            request.xs = result.ongoing_xs
            request.exec_task_ids = result.ongoing_task_ids
        else:
            # nothing to run for this round: the bulk swap still has to rotate
            self.virtual_page_pool.swap2(next_mb.pinned_memory, prev_mb.pinned_memory)
            if getattr(self.layer_storage, "need_sample", False):
                request.cancel_task_ids = []
        return request

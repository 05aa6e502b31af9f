"""A decode step of a stage as a replayed HIP graph.

The reference launches every kernel of every layer from Python each step; at
decode sizes the step is a few dozen short launches.  ``GraphedDecodeStep``
captures what ``layer_storage.forward(xs, ctx)`` launches for one batch shape
into a graph and replays it: per step the host only rebuilds the CSR metadata
and the split-KV work list in pinned buffers that never move, copies both to
device buffers that never move, and replays.  A new batch size (or workgroup
count) triggers a new capture; the last few captures are kept, so a scheduler that
alternates between batch sizes replays instead of capturing again.

Nothing that is captured clears memory with a memset node, and the library
calls allocate nothing; the outputs of the captured forward live in the graph's
own memory pool and are overwritten by every replay.
"""
from __future__ import annotations

from collections import OrderedDict
from typing import List, Sequence

import torch

from deserve_amd import _lib
from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.model.context.flash import FlashDecodeCtx, MetadataBuffers, StagedUpload
from deserve_amd.paged_ops import BatchDecodeWithPagedKVCacheWrapper
from deserve_amd.task import TaskData


class GraphedDecodeStep:
    def __init__(self, layer_storage, wrapper: BatchDecodeWithPagedKVCacheWrapper, max_batch: int,
                 max_pages: int, device: torch.device, num_qo_heads: int, num_kv_heads: int,
                 head_dim: int, page_size: int, target_workgroups: int = 0, max_graphs: int = 8) -> None:
        self.layer_storage, self.wrapper = layer_storage, wrapper
        self.shape = dict(num_qo_heads=num_qo_heads, num_kv_heads=num_kv_heads, head_dim=head_dim,
                          page_size=page_size)
        self.target_workgroups = target_workgroups
        self.meta = MetadataBuffers(max_batch, max_pages, device)
        words = int(_lib.lib().dskv_decode_plan_bound(max_batch, max_pages * page_size))
        self.plan = StagedUpload(words, device)
        self.max_graphs = max_graphs
        self._graphs: "OrderedDict[tuple, tuple]" = OrderedDict()   # key -> (graph, inputs, output)
        self._graph = None                     # the one replayed last
        self._inputs: List[torch.Tensor] = []
        self._output = None
        self.captures = 0

    def _prepare(self, task_datas: Sequence[TaskData], kvcaches: Sequence[PagedKVCache]) -> FlashDecodeCtx:
        ctx = FlashDecodeCtx.init_paged_decode_ctx(list(task_datas), list(kvcaches), self.wrapper, self.meta)
        self.wrapper.begin_forward(indptr=ctx.kv_page_indptr, indices=ctx.kv_page_indices,
                                   last_page_len=ctx.kv_last_page_lens,
                                   indptr_host=ctx.host["kv_page_indptr"],
                                   last_page_len_host=ctx.host["kv_last_page_lens"],
                                   indices_host=ctx.host["kv_page_indices"],
                                   target_workgroups=self.target_workgroups, plan_buffers=self.plan,
                                   **self.shape)
        return ctx

    @staticmethod
    def graph_key(batch: int, n_workgroups: int, n_items: int, tensors: Sequence[torch.Tensor],
                  persistent_kernel: bool) -> tuple:
        """What decides which launches a captured step holds.  Always: batch, workgroup
        count, whether anything is merged and with which of the two merge kernels (the
        launcher takes the wide one from 32 parts per request on), input shapes.  The
        attention kernel of the 16-bit head_dim-128 path is launched with one workgroup per
        planned workgroup and reads its items from the plan, so the item count is not part
        of its launch; the generic kernel (fp32 pools, other head dims, groups over 16) is
        launched with one workgroup per item, so there the item count is part of the key -
        a replay with another count would skip items or run on stale plan words."""
        key = (batch, n_workgroups, n_items > batch, n_items > 32 * batch,
               tuple((tuple(t.shape), t.dtype) for t in tensors))
        return key if persistent_kernel else key + (n_items,)

    def run(self, xs, task_datas: Sequence[TaskData], kvcaches: Sequence[PagedKVCache]) -> torch.Tensor:
        """xs: a tensor or a tuple of tensors, as the stage's forward takes them.  Returns the
        stage's output (valid until the next run)."""
        tensors = list(xs) if isinstance(xs, (tuple, list)) else [xs]
        ctx = self._prepare(task_datas, kvcaches)
        w = self.wrapper
        key = self.graph_key(len(task_datas), w._n_workgroups, w._n_items, tensors,
                             w.fused_append_supported(tensors[0].dtype))
        held = self._graphs.get(key)
        if held is None:
            inputs = [t.clone() for t in tensors]
            static = tuple(inputs) if isinstance(xs, (tuple, list)) else inputs[0]
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                output = self.layer_storage.forward(static, ctx)
            self._graphs[key] = held = (graph, inputs, output)
            self.captures += 1
            while len(self._graphs) > self.max_graphs:
                self._graphs.popitem(last=False)        # least recently used
        else:
            self._graphs.move_to_end(key)
            # one copy kernel on the launch stream for all inputs: device-to-device memcpy
            # calls may go through a DMA engine, whose hand-over to and from the compute
            # queue costs more than the copies themselves
            torch._foreach_copy_(held[1], tensors)
        self._graph, self._inputs, self._output = held
        self._graph.replay()
        w.end_forward()
        return self._output

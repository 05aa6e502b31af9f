"""Per-step CSR metadata for the paged kernels
(deserve_worker/model/context/flash.py:17-120).

For every request: current_len = start_pos + seqlen tokens are visible, the
cache is extended to max(current_len, initial_seqlen) (a chunked prefill
reserves the whole prompt up front), ceil(current_len / P) block-table entries
are exposed and the last page holds (current_len - 1) % P + 1 tokens.

The reference builds six small device tensors with a cat of B device slices and
five host-to-device constructions per step.  Here all six arrays are laid out in
ONE pinned staging block and reach the device through ONE upload kernel; the
device tensors of the context are views of that upload, and the host arrays are
kept (``host`` dict) so the attention planner never reads back from the device.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Sequence

import numpy as np
import torch

from deserve_amd import staging
from deserve_amd.kvcache.paged.kvcache import PagedKVCache
from deserve_amd.kvcache.paged.page_pool import GpuPagePool
from deserve_amd.model.context.forward import PagedForwardCtx
from deserve_amd.paged_ops import (BatchDecodeWithPagedKVCacheWrapper,
                                   BatchPrefillWithPagedKVCacheWrapper)
from deserve_amd.task import TaskData

_FIELDS = ("indptr", "kv_page_indptr", "kv_last_page_lens", "offsets", "seqlens",
           "kv_page_indices")


def build_host_metadata(task_datas: Sequence[TaskData],
                        kvcaches: Sequence[PagedKVCache]) -> Dict[str, np.ndarray]:
    """The six int32 arrays on the host; extends the caches as a side effect (in request
    order, as the reference's loop does: the order decides which page ids a request gets)."""
    B = len(task_datas)
    start = np.fromiter((t.start_pos for t in task_datas), np.int64, B)
    seq = np.fromiter((t.seqlen for t in task_datas), np.int64, B)
    want = np.fromiter((t.initial_seqlen for t in task_datas), np.int64, B)
    current = start + seq
    np.maximum(want, current, out=want)
    indptr = np.zeros(B + 1, np.int32)
    np.cumsum(seq, out=indptr[1:])
    one_pool = B > 0 and all(c.pool is kvcaches[0].pool for c in kvcaches)
    one_table = one_pool and all(c.page_table.allocator is kvcaches[0].page_table.allocator
                                 for c in kvcaches)
    if not one_table:
        # caches over several pools or tables: request by request
        exposed = np.zeros(B, np.int64)
        last = np.zeros(B, np.int32)
        rows: List[np.ndarray] = []
        for i, cache in enumerate(kvcaches):
            page_size = cache.pool.page_size
            cache.extend(int(want[i]))
            exposed[i] = -(-int(current[i]) // page_size)
            rows.append(cache.page_table.retrieve()[: int(exposed[i])].numpy())
            last[i] = (int(current[i]) - 1) % page_size + 1
        indices = np.concatenate(rows).astype(np.int32) if rows else np.zeros(0, np.int32)
    else:
        # the usual case, without a Python-level pass per request: only the caches that
        # cross a page boundary are touched, and the block-table rows are gathered at once
        page_size = kvcaches[0].pool.page_size
        have = np.fromiter((c.page_table.occupied for c in kvcaches), np.int64, B) * page_size
        for i in np.flatnonzero(want > have):
            kvcaches[i].extend(int(want[i]))
        exposed = -(-current // page_size)
        last = ((current - 1) % page_size + 1).astype(np.int32)
        table = kvcaches[0].page_table.allocator.tables.numpy()
        slots = np.fromiter((c.page_table.offset for c in kvcaches), np.int64, B)
        width = int(exposed.max())
        picked = table[slots, :width]
        indices = picked[np.arange(width)[None, :] < exposed[:, None]].astype(np.int32, copy=False)
    kv_indptr = np.zeros(B + 1, np.int32)
    np.cumsum(exposed, out=kv_indptr[1:])
    return dict(indptr=indptr, kv_page_indptr=kv_indptr, kv_last_page_lens=last,
                offsets=start.astype(np.int32), seqlens=seq.astype(np.int32), kv_page_indices=indices)


class StagedUpload:
    """An int32 device buffer that stays where it is from step to step, fed from pinned
    staging blocks: for callers that replay captured launches (the kernels then find their
    inputs at the same addresses every step)."""

    def __init__(self, words: int, device: torch.device) -> None:
        self.dev = torch.empty((words,), dtype=torch.int32, device=device)
        self._block = None

    def staging(self) -> torch.Tensor:
        """A pinned buffer to fill for the next upload."""
        self._block = staging.take(self.dev.numel())
        return self._block.tensor

    def upload(self, words: int) -> None:
        """Enqueues the copy of the first `words` words of the staging buffer handed out last."""
        block, self._block = self._block, None
        staging.upload(block, self.dev, words)


class MetadataBuffers(StagedUpload):
    """StagedUpload sized for the six CSR arrays of a step.  The batch-sized arrays come
    first, the block-table entries last, so only the batch decides where an array starts."""

    def __init__(self, max_batch: int, max_pages: int, device: torch.device) -> None:
        super().__init__(5 * ((max_batch + 1 + 3) // 4 * 4) + (max_pages + 3) // 4 * 4, device)


def metadata_layout(meta: Dict[str, np.ndarray]):
    """(start word of every array, total words): each array starts on a 16-byte boundary."""
    starts, total = {}, 0
    for f in _FIELDS:
        starts[f] = total
        total += (meta[f].shape[0] + 3) // 4 * 4
    return starts, total


def upload_metadata(meta: Dict[str, np.ndarray], device: torch.device,
                    buffers: "MetadataBuffers | None" = None):
    """One pinned staging block, one upload kernel; returns (device views, host views).
    The host views are the arrays of `meta` themselves, not the staging block."""
    sizes = [meta[f].shape[0] for f in _FIELDS]
    # each array starts on a 16-byte boundary
    starts, total = [], 0
    for n in sizes:
        starts.append(total)
        total += (n + 3) // 4 * 4
    host_views = {f: torch.from_numpy(meta[f]) for f in _FIELDS}
    if torch.device(device).type != "cuda":
        dev = torch.zeros((max(total, 4),), dtype=torch.int32)
        for f, s, n in zip(_FIELDS, starts, sizes):
            dev[s: s + n] = host_views[f]
    else:
        if buffers is not None and total > buffers.dev.numel():
            raise ValueError(f"step metadata needs {total} words, the buffers hold {buffers.dev.numel()}")
        block = None if buffers is not None else staging.take(total)
        host_np = (buffers.staging() if buffers is not None else block.tensor).numpy()
        for f, s, n in zip(_FIELDS, starts, sizes):
            host_np[s: s + n] = meta[f]
        if buffers is not None:
            dev = buffers.dev
            buffers.upload(total)
        else:
            dev = staging.to_device(block, total, device)
    dev_views = {f: dev[s: s + n] for f, s, n in zip(_FIELDS, starts, sizes)}
    return dev_views, host_views


@dataclass
class FlashForwardCtx(PagedForwardCtx):
    indptr: torch.Tensor
    kv_page_indices: torch.Tensor
    kv_page_indptr: torch.Tensor
    kv_last_page_lens: torch.Tensor
    host: Dict[str, torch.Tensor] = field(default_factory=dict, repr=False)

    @classmethod
    def init_paged_forward_ctx(cls, task_datas: List[TaskData],
                               kvcaches: List[PagedKVCache[GpuPagePool]],
                               buffers: "MetadataBuffers | None" = None, **extra):
        pool = kvcaches[0].pool
        dev, host = upload_metadata(build_host_metadata(task_datas, kvcaches), pool.main_device, buffers)
        return cls(bsz=len(task_datas), seqlens=dev["seqlens"], layer_id=0, page_pool=pool,
                   offsets=dev["offsets"], indptr=dev["indptr"],
                   kv_page_indices=dev["kv_page_indices"], kv_page_indptr=dev["kv_page_indptr"],
                   kv_last_page_lens=dev["kv_last_page_lens"], host=host, **extra)


@dataclass
class FlashDecodeCtx(FlashForwardCtx):
    decode_wrapper: BatchDecodeWithPagedKVCacheWrapper = None   # type: ignore[assignment]

    @classmethod
    def init_paged_decode_ctx(cls, task_datas: List[TaskData],
                              kvcaches: List[PagedKVCache[GpuPagePool]],
                              wrapper: BatchDecodeWithPagedKVCacheWrapper,
                              buffers: "MetadataBuffers | None" = None) -> "FlashDecodeCtx":
        return cls.init_paged_forward_ctx(task_datas, kvcaches, buffers, decode_wrapper=wrapper)

    @classmethod
    def init_and_plan(cls, task_datas: List[TaskData], kvcaches: List[PagedKVCache[GpuPagePool]],
                      wrapper: BatchDecodeWithPagedKVCacheWrapper, num_qo_heads: int, num_kv_heads: int,
                      head_dim: int, page_size: int, target_workgroups: int = 0) -> "FlashDecodeCtx":
        """init_paged_decode_ctx + wrapper.begin_forward as ONE upload: the six index arrays
        and the attention work list share a pinned block and reach the device through one
        kernel (what BatchDecode.prepare does; the reference makes five host-to-device
        tensor constructions and FlashInfer its own plan upload, flash.py:46-64,
        exec.py:184-192)."""
        pool = kvcaches[0].pool
        meta = build_host_metadata(task_datas, kvcaches)
        starts, total = metadata_layout(meta)
        host = {f: torch.from_numpy(meta[f]) for f in _FIELDS}

        def fill(view: torch.Tensor) -> None:
            arr = view.numpy()
            for f in _FIELDS:
                arr[starts[f]: starts[f] + meta[f].shape[0]] = meta[f]

        dev = wrapper.begin_forward_with_metadata(
            total, fill, starts["kv_page_indptr"], starts["kv_page_indices"], host["kv_page_indptr"],
            host["kv_last_page_lens"], host["kv_page_indices"], num_qo_heads, num_kv_heads, head_dim,
            page_size, pool.main_device, target_workgroups)
        v = {f: dev[starts[f]: starts[f] + meta[f].shape[0]] for f in _FIELDS}
        return cls(bsz=len(task_datas), seqlens=v["seqlens"], layer_id=0, page_pool=pool,
                   offsets=v["offsets"], indptr=v["indptr"], kv_page_indices=v["kv_page_indices"],
                   kv_page_indptr=v["kv_page_indptr"], kv_last_page_lens=v["kv_last_page_lens"],
                   host=host, decode_wrapper=wrapper)


@dataclass
class FlashPrefillCtx(FlashForwardCtx):
    prefill_wrapper: BatchPrefillWithPagedKVCacheWrapper = None   # type: ignore[assignment]

    @classmethod
    def init_paged_prefill_ctx(cls, task_datas: List[TaskData],
                               kvcaches: List[PagedKVCache[GpuPagePool]],
                               wrapper: BatchPrefillWithPagedKVCacheWrapper) -> "FlashPrefillCtx":
        return cls.init_paged_forward_ctx(task_datas, kvcaches, prefill_wrapper=wrapper)

    @classmethod
    def init_and_plan(cls, task_datas: List[TaskData], kvcaches: List[PagedKVCache[GpuPagePool]],
                      wrapper: BatchPrefillWithPagedKVCacheWrapper, num_qo_heads: int, num_kv_heads: int,
                      head_dim: int, page_size: int, target_workgroups: int = 0) -> "FlashPrefillCtx":
        """init_paged_prefill_ctx + wrapper.begin_forward as ONE upload, as
        FlashDecodeCtx.init_and_plan does for decode (what BatchPrefill.prepare does; the
        reference: flash.py:46-64, exec.py:227-236)."""
        pool = kvcaches[0].pool
        meta = build_host_metadata(task_datas, kvcaches)
        starts, total = metadata_layout(meta)
        host = {f: torch.from_numpy(meta[f]) for f in _FIELDS}

        def fill(view: torch.Tensor) -> None:
            arr = view.numpy()
            for f in _FIELDS:
                arr[starts[f]: starts[f] + meta[f].shape[0]] = meta[f]

        dev = wrapper.begin_forward_with_metadata(
            total, fill, starts, host["indptr"], host["kv_page_indptr"], host["kv_last_page_lens"],
            host["kv_page_indices"], num_qo_heads, num_kv_heads, head_dim, page_size, pool.main_device,
            target_workgroups)
        v = {f: dev[starts[f]: starts[f] + meta[f].shape[0]] for f in _FIELDS}
        return cls(bsz=len(task_datas), seqlens=v["seqlens"], layer_id=0, page_pool=pool,
                   offsets=v["offsets"], indptr=v["indptr"], kv_page_indices=v["kv_page_indices"],
                   kv_page_indptr=v["kv_page_indptr"], kv_last_page_lens=v["kv_last_page_lens"],
                   host=host, prefill_wrapper=wrapper)

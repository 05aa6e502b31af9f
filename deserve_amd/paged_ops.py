"""Operators that replace the reference's FlashInfer call sites
(deserve_worker/model/layer/attention.py:166-192 and
deserve_worker/execution/exec.py:20-22,184-192,227-236), with the same names,
argument order and begin_forward/forward/end_forward protocol, implemented by the
gfx950 kernels behind the C ABI.

All tensors are torch tensors on the GPU; work is enqueued on the current torch
stream.  ``pages`` is one layer of the pool: (num_pages, 2, page_size, Hkv, D).
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional, Tuple

import torch

from deserve_amd import _lib, staging


def _i32(t: torch.Tensor) -> torch.Tensor:
    if t.dtype != torch.int32:
        raise ValueError(f"index tensors must be int32, got {t.dtype}")
    return t.contiguous()


def append_paged_kv_cache(append_key: torch.Tensor, append_value: torch.Tensor,
                          append_indptr: torch.Tensor, paged_kv_data: torch.Tensor,
                          kv_indices: torch.Tensor, kv_indptr: torch.Tensor,
                          kv_last_page_len: torch.Tensor) -> None:
    """In place on ``paged_kv_data``: the n_b new tokens of request b become the
    last n_b positions of its kv_len_b = (npages_b - 1) * P + last_b tokens."""
    if paged_kv_data.dim() != 5 or paged_kv_data.shape[1] != 2 or not paged_kv_data.is_contiguous():
        raise ValueError("paged_kv_data must be a contiguous (num_pages, 2, P, Hkv, D) tensor")
    _, _, P, Hkv, D = paged_kv_data.shape
    k, v = append_key.contiguous(), append_value.contiguous()
    if k.shape != v.shape or tuple(k.shape[1:]) != (Hkv, D) or k.dtype != paged_kv_data.dtype \
            or v.dtype != paged_kv_data.dtype:
        raise ValueError("append_key/append_value must be (nnz, Hkv, D) of the pool's dtype")
    rc = _lib.lib().dskv_append_paged_kv(
        paged_kv_data.data_ptr(), paged_kv_data.shape[0], k.data_ptr(), v.data_ptr(), _i32(append_indptr).data_ptr(),
        _i32(kv_indices).data_ptr(), _i32(kv_indptr).data_ptr(), _i32(kv_last_page_len).data_ptr(),
        append_indptr.shape[0] - 1, k.shape[0], P, Hkv, D, k.element_size(), _lib.current_stream())
    _lib.check(rc, "append_paged_kv_cache")


def apply_rope(q: torch.Tensor, k: torch.Tensor, indptr: torch.Tensor, offsets: torch.Tensor,
               interleave: bool = False, rope_scale: float = 1.0,
               rope_theta: float = 1e4) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rotary embedding of ragged q (nnz, Hq, D) / k (nnz, Hkv, D); returns new
    tensors.  Only the adjacent-pair convention (interleave=True) that the
    reference uses is implemented."""
    if not interleave or rope_scale != 1.0:
        raise ValueError("apply_rope: only interleave=True, rope_scale=1 is implemented")
    q, k = q.contiguous(), k.contiguous()
    q_out, k_out = torch.empty_like(q), torch.empty_like(k)
    rc = _lib.lib().dskv_apply_rope(
        q_out.data_ptr(), k_out.data_ptr(), q.data_ptr(), k.data_ptr(), _i32(indptr).data_ptr(),
        _i32(offsets).data_ptr(), indptr.shape[0] - 1, q.shape[0], q.shape[1], k.shape[1],
        q.shape[2], float(rope_theta), _lib.dtype_code(q.dtype), _lib.current_stream())
    _lib.check(rc, "apply_rope")
    return q_out, k_out


def rope_append_paged_kv_cache(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor,
                               indptr: torch.Tensor, offsets: torch.Tensor,
                               paged_kv_data: torch.Tensor, kv_indices: torch.Tensor,
                               kv_indptr: torch.Tensor, kv_last_page_len: torch.Tensor,
                               rope_theta: float = 1e4) -> torch.Tensor:
    """apply_rope(interleave=True) + append_paged_kv_cache in one kernel: returns the
    rotated q; the rotated k and v land in their page slots.  Same bits as the two
    separate calls."""
    if paged_kv_data.dim() != 5 or paged_kv_data.shape[1] != 2 or not paged_kv_data.is_contiguous():
        raise ValueError("paged_kv_data must be a contiguous (num_pages, 2, P, Hkv, D) tensor")
    _, _, P, Hkv, D = paged_kv_data.shape
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    if k.shape != v.shape or tuple(k.shape[1:]) != (Hkv, D) or q.shape[2] != D or \
            not (q.dtype == k.dtype == v.dtype == paged_kv_data.dtype):
        raise ValueError("q/k/v must be (nnz, H, D) of the pool's dtype")
    q_out = torch.empty_like(q)
    rc = _lib.lib().dskv_rope_append_paged_kv(
        q_out.data_ptr(), paged_kv_data.data_ptr(), paged_kv_data.shape[0], q.data_ptr(), k.data_ptr(), v.data_ptr(),
        _i32(indptr).data_ptr(), _i32(offsets).data_ptr(), _i32(kv_indices).data_ptr(),
        _i32(kv_indptr).data_ptr(), _i32(kv_last_page_len).data_ptr(), indptr.shape[0] - 1,
        q.shape[0], P, q.shape[1], Hkv, D, float(rope_theta), _lib.dtype_code(q.dtype),
        _lib.current_stream())
    _lib.check(rc, "rope_append_paged_kv_cache")
    return q_out


class _PagedWrapper:
    def __init__(self, workspace_buffer: torch.Tensor, kv_layout: str = "NHD") -> None:
        if kv_layout != "NHD":
            raise ValueError("only the NHD page layout is implemented")
        self._workspace = workspace_buffer
        self._planned = False
        self._rope_table, self._rope_key = None, None
        self._max_page_id = -1
        self._empty_requests = []

    def _shape_args(self, num_qo_heads: int, num_kv_heads: int, head_dim: int, page_size: int) -> None:
        self._hq, self._hkv, self._d, self._p = num_qo_heads, num_kv_heads, head_dim, page_size

    @staticmethod
    def _host(t: torch.Tensor, host: Optional[torch.Tensor]) -> torch.Tensor:
        """Host copy of a small index tensor (synchronises only if none was given)."""
        src = host if host is not None else t.cpu()
        return src.to(torch.int32).contiguous()

    def _check_block_tables(self, h_indptr: torch.Tensor, indices: torch.Tensor,
                            indices_host: Optional[torch.Tensor], h_last: torch.Tensor) -> None:
        """The kernels index the pool by block-table entries: refuse, on the host, tables that
        are shorter than indptr says or hold a negative id, last-page lengths that are missing
        or outside [1, page_size], and remember the largest id so that forward() can refuse a
        pool that does not have that page."""
        batch = h_indptr.shape[0] - 1
        used = int(h_indptr[-1]) if batch > 0 else 0
        if batch > 0 and (int(h_indptr[0]) != 0 or bool((h_indptr[1:] < h_indptr[:-1]).any())):
            raise ValueError("kv page indptr must start at 0 and not decrease")
        if h_last.numel() < max(batch, 0):
            raise ValueError(f"kv last-page lengths hold {h_last.numel()} entries for {batch} requests")
        if batch > 0:
            last = h_last[:batch]
            bad = (h_indptr[1:] > h_indptr[:-1]) & ((last < 1) | (last > self._p))
            if bool(bad.any()):
                b = int(bad.nonzero()[0])
                raise ValueError(f"kv_last_page_len[{b}] = {int(last[b])} outside [1, {self._p}]")
        if indices.numel() < used:
            raise ValueError(f"kv page indices hold {indices.numel()} entries, indptr[-1] is {used}")
        ids = self._host(indices, indices_host)[:used]
        if indices_host is not None and indices_host.numel() < used:
            raise ValueError(f"indices_host holds {indices_host.numel()} entries, indptr[-1] is {used}")
        self._max_page_id = -1
        if used > 0:
            lo, hi = int(ids.min()), int(ids.max())
            if lo < 0:
                raise ValueError(f"negative page id {lo} in the block tables")
            self._max_page_id = hi

    def _check_pool(self, paged_kv_data: torch.Tensor, dtype: torch.dtype) -> None:
        want = (2, self._p, self._hkv, self._d)
        if paged_kv_data.dim() != 5 or tuple(paged_kv_data.shape[1:]) != want:
            raise ValueError(f"paged_kv_data must be (num_pages, {', '.join(map(str, want))}) as given to "
                             f"begin_forward, got {tuple(paged_kv_data.shape)}")
        if not paged_kv_data.is_contiguous() or paged_kv_data.dtype != dtype:
            raise ValueError("paged_kv_data must be contiguous and of q's dtype")
        if self._max_page_id >= paged_kv_data.shape[0]:
            raise ValueError(f"the block tables name page {self._max_page_id}, the pool has "
                             f"{paged_kv_data.shape[0]} pages")

    def end_forward(self) -> None:
        self._planned = False


class BatchDecodeWithPagedKVCacheWrapper(_PagedWrapper):
    """begin_forward plans the split-KV work list on the host and uploads it once;
    forward (once per layer) launches the attention and merge kernels."""

    def begin_forward(self, indptr: torch.Tensor, indices: torch.Tensor,
                      last_page_len: torch.Tensor, num_qo_heads: int, num_kv_heads: int,
                      head_dim: int, page_size: int, *, indptr_host: Optional[torch.Tensor] = None,
                      last_page_len_host: Optional[torch.Tensor] = None,
                      indices_host: Optional[torch.Tensor] = None,
                      target_workgroups: int = 0, plan_buffers=None, **_ignored) -> None:
        """The *_host arguments are host copies of the index tensors: the planner and the
        checks of the block tables run on the host; without them the device tensors are read
        back, which synchronises.
        plan_buffers: optional staged upload (an object with staging() / upload(words) /
        dev, see model.context.flash.StagedUpload) that receives the work list instead of
        fresh tensors, for callers that replay captured launches."""
        self._shape_args(num_qo_heads, num_kv_heads, head_dim, page_size)
        self._indptr, self._indices = _i32(indptr), _i32(indices)
        h_indptr = self._host(indptr, indptr_host)
        h_last = self._host(last_page_len, last_page_len_host)
        self._check_block_tables(h_indptr, indices, indices_host, h_last)
        batch = h_indptr.shape[0] - 1
        cap = self._plan_bound(batch, h_indptr, page_size)
        if plan_buffers is not None:
            if plan_buffers.dev.numel() < cap:
                raise ValueError(f"plan buffer holds {plan_buffers.dev.numel()} words, {cap} may be needed")
            plan = plan_buffers.staging()
        else:
            block = staging.take(max(cap, 1))
            plan = block.tensor
        words = self._plan_into(plan, cap, h_indptr, h_last, target_workgroups)
        if plan_buffers is not None:
            self._plan = plan_buffers.dev
            plan_buffers.upload(max(words, 1))
        else:
            self._plan = staging.to_device(block, max(words, 1), indices.device)
        self._planned = True

    @staticmethod
    def _plan_bound(batch: int, h_indptr: torch.Tensor, page_size: int) -> int:
        total_tokens = int(h_indptr[-1]) * page_size if batch > 0 else 0
        return int(_lib.lib().dskv_decode_plan_bound(batch, total_tokens))

    def _plan_into(self, plan: torch.Tensor, cap: int, h_indptr: torch.Tensor, h_last: torch.Tensor,
                   target_workgroups: int) -> int:
        """Runs the host planner into `plan` (pinned int32, at least cap words); returns the
        words written.  Sets the launch shape of the following forward() calls."""
        batch = h_indptr.shape[0] - 1
        n_items, n_wgs = ctypes.c_int32(), ctypes.c_int32()
        words, ws = ctypes.c_int64(), ctypes.c_int64()
        rc = _lib.lib().dskv_decode_plan(h_indptr.data_ptr(), h_last.data_ptr(), batch, self._p,
                                         self._hq, self._hkv, self._d, target_workgroups,
                                         plan.data_ptr(), cap, ctypes.byref(n_items), ctypes.byref(n_wgs),
                                         ctypes.byref(words), ctypes.byref(ws))
        _lib.check(rc, "decode begin_forward")
        if ws.value > self._workspace.numel() * self._workspace.element_size():
            raise RuntimeError(f"decode workspace too small: need {ws.value} bytes")
        self._batch, self._n_items, self._n_workgroups = batch, n_items.value, n_wgs.value
        self._rope_table, self._rope_key = None, None     # positions change with the step
        # requests without a page: the fused append has no slot to write their token to
        n_pages = h_indptr[1:] - h_indptr[:-1]
        self._empty_requests = [int(b) for b in (n_pages <= 0).nonzero().flatten()[:4]] if batch > 0 else []
        return int(words.value)

    def begin_forward_with_metadata(self, meta_words: int, fill_metadata, indptr_at: int, indices_at: int,
                                    indptr_host: torch.Tensor, last_page_len_host: torch.Tensor,
                                    indices_host: torch.Tensor, num_qo_heads: int, num_kv_heads: int,
                                    head_dim: int, page_size: int, device: torch.device,
                                    target_workgroups: int = 0) -> torch.Tensor:
        """begin_forward for callers that also have the step's other index arrays to upload
        (the forward context): metadata and work list travel in ONE pinned block and ONE
        upload kernel instead of one each.  fill_metadata(view) writes the caller's
        meta_words int32 words (a multiple of 4) into the front of the block; indptr_at /
        indices_at are the word offsets of kv_page_indptr and kv_page_indices in it.  Returns
        the device tensor that holds the metadata words (the caller slices its views)."""
        if meta_words % 4:
            raise ValueError("meta_words must be a multiple of 4 (16-byte alignment of the work list)")
        self._shape_args(num_qo_heads, num_kv_heads, head_dim, page_size)
        h_indptr = indptr_host.to(torch.int32).contiguous()
        h_last = last_page_len_host.to(torch.int32).contiguous()
        self._check_block_tables(h_indptr, indices_host, indices_host, h_last)
        batch = h_indptr.shape[0] - 1
        cap = self._plan_bound(batch, h_indptr, page_size)
        block = staging.take(meta_words + max(cap, 4))
        fill_metadata(block.tensor[:meta_words])
        words = self._plan_into(block.tensor[meta_words:], cap, h_indptr, h_last, target_workgroups)
        dev = staging.to_device(block, meta_words + max(words, 1), device)
        self._plan = dev[meta_words:]
        self._indptr = dev[indptr_at: indptr_at + batch + 1]
        used = int(h_indptr[-1]) if batch > 0 else 0
        self._indices = dev[indices_at: indices_at + used]
        self._planned = True
        return dev[:meta_words]

    def fused_append_supported(self, dtype: torch.dtype) -> bool:
        """Whether forward(..., k_append=, v_append=) can write the step's token itself for
        the shape given to begin_forward."""
        if dtype not in (torch.bfloat16, torch.float16):
            return False
        return bool(_lib.lib().dskv_decode_append_attn_supported(self._hq, self._hkv, self._d, self._p,
                                                                 _lib.dtype_code(dtype)))

    def forward(self, q: torch.Tensor, paged_kv_data: torch.Tensor,
                sm_scale: Optional[float] = None, *, phases: int = 3,
                out: Optional[torch.Tensor] = None, k_append: Optional[torch.Tensor] = None,
                v_append: Optional[torch.Tensor] = None, rope_offsets: Optional[torch.Tensor] = None,
                rope_theta: float = 500000.0, **_ignored) -> torch.Tensor:
        """phases: 1 = split-KV pass only, 2 = merge pass only, 3 = both (default).
        k_append, v_append (batch, Hkv, D): the step's token of every request, not yet in the
        pages - the attention launch writes them into their slots itself (one launch less than
        append_paged_kv_cache + forward; see fused_append_supported).
        rope_offsets (batch, int32, with k_append / v_append): the positions of those tokens;
        q and k_append are then taken unrotated and rotated inside the launch (in place of
        apply_rope before it).  The cos / sin table of the step is built at the first such call
        after begin_forward and shared by the following layers."""
        if not self._planned:
            raise RuntimeError("decode forward called before begin_forward")
        q = q.contiguous()
        if tuple(q.shape) != (self._batch, self._hq, self._d):
            raise ValueError(f"q must be ({self._batch}, {self._hq}, {self._d}), got {tuple(q.shape)}")
        self._check_pool(paged_kv_data, q.dtype)
        if out is None:
            out = torch.empty_like(q)
        scale = 1.0 / math.sqrt(self._d) if sm_scale is None else sm_scale
        ws_bytes = self._workspace.numel() * self._workspace.element_size()
        if k_append is not None or v_append is not None:
            if k_append is None or v_append is None or phases not in (1, 3):
                raise ValueError("the fused form takes both k_append and v_append, with the attention pass")
            if self._empty_requests:
                # the appended token is the request's last one (model/layer/attention.py:175-185):
                # every request of the plan owns at least the page that holds it
                raise ValueError(f"k_append / v_append: request(s) {self._empty_requests} have no page "
                                 "(kv length 0 after the append); extend the caches before begin_forward")
            k_append, v_append = k_append.contiguous(), v_append.contiguous()
            want = (self._batch, self._hkv, self._d)
            if tuple(k_append.shape) != want or tuple(v_append.shape) != want or \
                    k_append.dtype != q.dtype or v_append.dtype != q.dtype:
                raise ValueError(f"k_append / v_append must be {want} of q's dtype")
            if rope_offsets is not None:
                key = (rope_offsets.data_ptr(), float(rope_theta))
                if self._rope_key != key:
                    if rope_offsets.dtype != torch.int32 or rope_offsets.numel() != self._batch:
                        raise ValueError(f"rope_offsets must be {self._batch} int32 positions")
                    table = torch.empty((self._batch, self._d), dtype=torch.float32, device=q.device)
                    _lib.check(_lib.lib().dskv_rope_table(table.data_ptr(), rope_offsets.data_ptr(),
                                                          self._batch, self._d, rope_theta,
                                                          _lib.current_stream()), "rope table")
                    self._rope_table, self._rope_key = table, key
                rc = _lib.lib().dskv_decode_rope_append_attn(
                    out.data_ptr(), q.data_ptr(), k_append.data_ptr(), v_append.data_ptr(),
                    paged_kv_data.data_ptr(), self._indices.data_ptr(), self._plan.data_ptr(),
                    self._n_items, self._n_workgroups, self._workspace.data_ptr(), ws_bytes,
                    self._batch, self._hq, self._hkv, self._d, self._p, scale,
                    _lib.dtype_code(q.dtype), self._rope_table.data_ptr(), phases,
                    _lib.current_stream())
                _lib.check(rc, "decode rope + append + forward")
                return out
            rc = _lib.lib().dskv_decode_append_attn(
                out.data_ptr(), q.data_ptr(), k_append.data_ptr(), v_append.data_ptr(),
                paged_kv_data.data_ptr(), self._indices.data_ptr(), self._plan.data_ptr(),
                self._n_items, self._n_workgroups, self._workspace.data_ptr(), ws_bytes, self._batch,
                self._hq, self._hkv, self._d, self._p, scale, _lib.dtype_code(q.dtype), phases,
                _lib.current_stream())
            _lib.check(rc, "decode append + forward")
            return out
        rc = _lib.lib().dskv_decode_attn_phases(
            out.data_ptr(), q.data_ptr(), paged_kv_data.data_ptr(), self._indices.data_ptr(),
            self._plan.data_ptr(), self._n_items, self._n_workgroups, self._workspace.data_ptr(),
            ws_bytes, self._batch, self._hq, self._hkv, self._d, self._p, scale,
            _lib.dtype_code(q.dtype), phases, _lib.current_stream())
        _lib.check(rc, "decode forward")
        return out


class BatchPrefillWithPagedKVCacheWrapper(_PagedWrapper):
    """begin_forward plans on the host: requests with one query row (the decode rows of a
    mixed step, which the reference sends through this wrapper together with the chunk:
    engine/microbatch/processor.py:116-145) become split-KV decode work, the others query
    tiles; forward (once per layer) launches the decode pass for the former and the tile
    pass for the latter, both writing their rows of the same ragged output."""

    def begin_forward(self, qo_indptr: torch.Tensor, paged_kv_indptr: torch.Tensor,
                      paged_kv_indices: torch.Tensor, paged_kv_last_page_len: torch.Tensor,
                      num_qo_heads: int, num_kv_heads: int, head_dim: int, page_size: int, *,
                      qo_indptr_host: Optional[torch.Tensor] = None,
                      paged_kv_indptr_host: Optional[torch.Tensor] = None,
                      paged_kv_last_page_len_host: Optional[torch.Tensor] = None,
                      paged_kv_indices_host: Optional[torch.Tensor] = None,
                      target_workgroups: int = 0, route_one_row_requests: bool = True,
                      **_ignored) -> None:
        """The *_host arguments are host copies of the index tensors (the planner and the
        checks of the block tables run on the host; without them the device tensors are read
        back, which synchronises).
        target_workgroups: a batch of few query tiles (a chunk of a few hundred tokens) is
        planned in several parts per tile, merged by a second pass, so that the launch has
        about this many workgroups (0: one per compute unit; negative: never split); the parts'
        partials go to the workspace buffer.
        route_one_row_requests: True lets the planner choose how one-row requests run (alone:
        the decode kernel; beside chunks: one launch in which decode workgroups and query
        tiles share the compute units, if the decode rows hold enough kv tokens); False keeps
        them on the tile path (one live row of a 64-row tile each), as a plan of
        dskv_prefill_plan does; _lib.ROUTE_TWO_LAUNCHES / _lib.ROUTE_SHARED_LAUNCH force a form."""
        self._shape_args(num_qo_heads, num_kv_heads, head_dim, page_size)
        self._qo_indptr, self._indptr = _i32(qo_indptr), _i32(paged_kv_indptr)
        self._indices, self._last = _i32(paged_kv_indices), _i32(paged_kv_last_page_len)
        h_qo = self._host(qo_indptr, qo_indptr_host)
        h_kv = self._host(paged_kv_indptr, paged_kv_indptr_host)
        h_last = self._host(paged_kv_last_page_len, paged_kv_last_page_len_host)
        cap = self._check_and_bound(h_qo, h_kv, h_last, paged_kv_indices, paged_kv_indices_host)
        block = staging.take(max(cap, 4))
        words = self._plan_into(block.tensor, cap, h_qo, h_kv, h_last, target_workgroups, route_one_row_requests)
        self._tiles = staging.to_device(block, max(words, 4), paged_kv_indices.device)
        self._planned = True

    def _check_and_bound(self, h_qo: torch.Tensor, h_kv: torch.Tensor, h_last: torch.Tensor,
                         indices: torch.Tensor, indices_host: Optional[torch.Tensor]):
        """Host-side checks of the index arrays; returns the words the plan may need."""
        batch = h_qo.shape[0] - 1
        if batch > 0 and (int(h_qo[0]) != 0 or bool((h_qo[1:] < h_qo[:-1]).any())):
            raise ValueError("qo_indptr must start at 0 and not decrease")
        if h_kv.shape[0] != h_qo.shape[0]:
            raise ValueError("qo_indptr and paged_kv_indptr disagree about the batch")
        self._check_block_tables(h_kv, indices, indices_host, h_last)
        nnz = int(h_qo[-1]) if batch > 0 else 0
        total_tokens = int(h_kv[-1]) * self._p if batch > 0 else 0
        return int(_lib.lib().dskv_mixed_plan_bound(batch, nnz, total_tokens))

    def _plan_into(self, plan: torch.Tensor, cap: int, h_qo: torch.Tensor, h_kv: torch.Tensor,
                   h_last: torch.Tensor, target_workgroups: int, route: bool = True) -> int:
        """Runs the host planner into `plan` (pinned int32, at least cap words); returns the words
        written.  The kv lengths order the tiles longest first and allow parts per tile; when
        the workspace cannot hold the parts' partials, whole tiles (which need none) are planned,
        and if it cannot even hold the partials of cut decode rows, nothing is routed."""
        batch = h_qo.shape[0] - 1
        info = _lib.MixedPlanInfo()
        ws_bytes = self._workspace.numel() * self._workspace.element_size()
        route = int(route)          # True = _lib.ROUTE_AUTO
        for target, routed in ((target_workgroups, route), (-1, route), (-1, _lib.ROUTE_OFF)):
            rc = _lib.lib().dskv_mixed_plan(h_qo.data_ptr(), h_kv.data_ptr(), h_last.data_ptr(), batch,
                                            self._p, self._hq, self._hkv, self._d, target, int(routed),
                                            plan.data_ptr(), cap, ctypes.byref(info))
            _lib.check(rc, "prefill begin_forward")
            if info.tile_workspace_bytes + info.decode_workspace_bytes <= ws_bytes:
                break
        self._batch, self._nnz = batch, (int(h_qo[-1]) if batch > 0 else 0)
        self._info = info
        self._n_tiles, self._n_splits = info.n_tiles, info.n_splits
        self._n_decode_rows = info.n_decode_rows
        return int(info.plan_words)

    def begin_forward_with_metadata(self, meta_words: int, fill_metadata, starts: dict,
                                    qo_indptr_host: torch.Tensor, paged_kv_indptr_host: torch.Tensor,
                                    paged_kv_last_page_len_host: torch.Tensor,
                                    paged_kv_indices_host: torch.Tensor, num_qo_heads: int,
                                    num_kv_heads: int, head_dim: int, page_size: int, device: torch.device,
                                    target_workgroups: int = 0, route_one_row_requests: bool = True) -> torch.Tensor:
        """begin_forward for callers that also have the step's other index arrays to upload
        (the forward context): metadata and plan travel in ONE pinned block and ONE upload
        kernel.  fill_metadata(view) writes the caller's meta_words int32 words (a multiple of
        4) into the front of the block; starts maps "indptr", "kv_page_indptr",
        "kv_page_indices" and "kv_last_page_lens" to their word offsets in it.  Returns the
        device tensor that holds the metadata words (the caller slices its views)."""
        if meta_words % 4:
            raise ValueError("meta_words must be a multiple of 4 (16-byte alignment of the plan)")
        self._shape_args(num_qo_heads, num_kv_heads, head_dim, page_size)
        h_qo = qo_indptr_host.to(torch.int32).contiguous()
        h_kv = paged_kv_indptr_host.to(torch.int32).contiguous()
        h_last = paged_kv_last_page_len_host.to(torch.int32).contiguous()
        cap = self._check_and_bound(h_qo, h_kv, h_last, paged_kv_indices_host, paged_kv_indices_host)
        block = staging.take(meta_words + max(cap, 4))
        fill_metadata(block.tensor[:meta_words])
        words = self._plan_into(block.tensor[meta_words:], cap, h_qo, h_kv, h_last, target_workgroups,
                                route_one_row_requests)
        dev = staging.to_device(block, meta_words + max(words, 4), device)
        batch = h_qo.shape[0] - 1
        used = int(h_kv[-1]) if batch > 0 else 0
        self._tiles = dev[meta_words:]
        self._qo_indptr = dev[starts["indptr"]: starts["indptr"] + batch + 1]
        self._indptr = dev[starts["kv_page_indptr"]: starts["kv_page_indptr"] + batch + 1]
        self._indices = dev[starts["kv_page_indices"]: starts["kv_page_indices"] + used]
        self._last = dev[starts["kv_last_page_lens"]: starts["kv_last_page_lens"] + batch]
        self._planned = True
        return dev[:meta_words]

    def forward(self, q: torch.Tensor, paged_kv_data: torch.Tensor, causal: bool = True,
                sm_scale: Optional[float] = None, *, out: Optional[torch.Tensor] = None,
                **_ignored) -> torch.Tensor:
        """out: optional result tensor (contiguous, q's shape and dtype); every row is written."""
        if not self._planned:
            raise RuntimeError("prefill forward called before begin_forward")
        q = q.contiguous()
        if tuple(q.shape) != (self._nnz, self._hq, self._d):
            raise ValueError(f"q must be ({self._nnz}, {self._hq}, {self._d}), got {tuple(q.shape)}")
        self._check_pool(paged_kv_data, q.dtype)
        if out is None:
            out = torch.empty_like(q)
        elif out.shape != q.shape or out.dtype != q.dtype or not out.is_contiguous():
            raise ValueError("out must be contiguous and of q's shape and dtype")
        scale = 1.0 / math.sqrt(self._d) if sm_scale is None else sm_scale
        rc = _lib.lib().dskv_mixed_attn(
            out.data_ptr(), q.data_ptr(), self._qo_indptr.data_ptr(), paged_kv_data.data_ptr(),
            self._indices.data_ptr(), self._indptr.data_ptr(), self._last.data_ptr(),
            self._tiles.data_ptr(), ctypes.byref(self._info), self._workspace.data_ptr(),
            self._workspace.numel() * self._workspace.element_size(), self._batch, self._nnz, self._hq,
            self._hkv, self._d, self._p, scale, int(causal), _lib.dtype_code(q.dtype),
            _lib.current_stream())
        _lib.check(rc, "prefill forward")
        return out

"""The KV part of one attention layer: RoPE -> KV append -> paged attention
(deserve_worker/model/layer/attention.py:160-193).  The q/k/v/o projections
around it are dense GEMMs of the model proper and are not part of this package;
``paged_forward`` takes the projected q, k, v and returns the attention output
in ragged (nnz, Hq * D) form, as the reference's method does before ``wo``."""
from __future__ import annotations

import torch

from deserve_amd.model.context.flash import FlashDecodeCtx, FlashForwardCtx, FlashPrefillCtx
from deserve_amd.paged_ops import (append_paged_kv_cache, apply_rope,
                                   rope_append_paged_kv_cache)


class PagedAttentionCore:
    def __init__(self, n_heads: int, n_kv_heads: int, head_dim: int, rope_theta: float = 500000.0,
                 use_rope: bool = True, fuse_rope_append: bool = True,
                 fuse_decode_append: bool = True) -> None:
        self.n_local_heads, self.n_local_kv_heads = n_heads, n_kv_heads
        self.head_dim, self.dim = head_dim, n_heads * head_dim
        self.rope_theta, self.use_rope = rope_theta, use_rope
        self.fuse_rope_append = fuse_rope_append
        self.fuse_decode_append = fuse_decode_append

    @torch.inference_mode()
    def paged_forward(self, xq: torch.Tensor, xk: torch.Tensor, xv: torch.Tensor,
                      ctx: FlashForwardCtx) -> torch.Tensor:
        xq = xq.view(-1, self.n_local_heads, self.head_dim)
        xk = xk.view(-1, self.n_local_kv_heads, self.head_dim)
        xv = xv.view(-1, self.n_local_kv_heads, self.head_dim)
        pages = ctx.page_pool.get_layered_pages(ctx.layer_id)
        if (isinstance(ctx, FlashDecodeCtx) and self.fuse_decode_append and xk.shape[0] == ctx.bsz
                and ctx.decode_wrapper.fused_append_supported(xq.dtype)):
            # a decode step: the attention launch rotates q and the new k and writes the new
            # token into its page slot itself
            rope = dict(rope_offsets=ctx.offsets, rope_theta=self.rope_theta) if self.use_rope else {}
            out = ctx.decode_wrapper.forward(xq, pages, k_append=xk, v_append=xv, **rope)
            return out.view(-1, self.dim)
        if self.use_rope and self.fuse_rope_append:
            # one kernel: rotated q comes back, rotated k and v go straight into their slots
            xq = rope_append_paged_kv_cache(xq, xk, xv, ctx.indptr, ctx.offsets, pages,
                                            ctx.kv_page_indices, ctx.kv_page_indptr,
                                            ctx.kv_last_page_lens, rope_theta=self.rope_theta)
        else:
            if self.use_rope:
                xq, xk = apply_rope(xq, xk, ctx.indptr, ctx.offsets, interleave=True,
                                    rope_theta=self.rope_theta)
            append_paged_kv_cache(xk, xv, ctx.indptr, pages, ctx.kv_page_indices,
                                  ctx.kv_page_indptr, ctx.kv_last_page_lens)
        if isinstance(ctx, FlashDecodeCtx):
            out = ctx.decode_wrapper.forward(xq, pages)
        elif isinstance(ctx, FlashPrefillCtx):
            out = ctx.prefill_wrapper.forward(xq, pages, causal=True)
        else:
            raise TypeError(f"unsupported forward context {type(ctx).__name__}")
        return out.view(-1, self.dim)

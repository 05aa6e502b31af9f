"""A stage's KV path without the dense model around it.

``KVStage`` plays the role of the reference's ``LayerStorage`` for the execution
layer (deserve_worker/layer_storage.py:182-197 walks the layers and bumps
``ctx.layer_id``): per layer it runs RoPE -> KV append -> paged attention on
already projected q/k/v.  It lets the hot path be driven, tested and timed at
its real shape on one GPU; the projections and MLPs between the attention calls
belong to the model and are not reproduced.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from deserve_amd.model.context.flash import FlashForwardCtx
from deserve_amd.model.layer.attention import PagedAttentionCore


@dataclass
class StageArgs:
    n_heads: int = 32
    n_kv_heads: Optional[int] = 8
    dim: int = 4096
    page_size: int = 16
    n_layers: int = 16
    rope_theta: float = 500000.0


class KVStage:
    need_sample = False

    def __init__(self, model_args: StageArgs, use_rope: bool = True) -> None:
        self.model_args = model_args
        n_kv = model_args.n_heads if model_args.n_kv_heads is None else model_args.n_kv_heads
        self.core = PagedAttentionCore(model_args.n_heads, n_kv, model_args.dim // model_args.n_heads,
                                       model_args.rope_theta, use_rope)

    def forward(self, xs: Tuple[torch.Tensor, torch.Tensor, torch.Tensor],
                ctx: FlashForwardCtx) -> torch.Tensor:
        """xs = (q, k, v) stacked per layer: (L, nnz, Hq, D), (L, nnz, Hkv, D) x2.
        Returns the attention outputs of all layers, (L, nnz, Hq * D)."""
        q, k, v = xs
        outs = []
        for layer in range(q.shape[0]):
            outs.append(self.core.paged_forward(q[layer], k[layer], v[layer], ctx))
            ctx.layer_id += 1
        return torch.stack(outs)


class PackedKVStage(KVStage):
    """KVStage for callers that carry one tensor per token, as the scheduler's
    queues do: xs is (nnz, L, Hq + 2*Hkv, D) with each token's q, k and v heads of
    every layer side by side."""

    def forward(self, xs: torch.Tensor, ctx: FlashForwardCtx) -> torch.Tensor:   # type: ignore[override]
        hq = self.model_args.n_heads
        hkv = hq if self.model_args.n_kv_heads is None else self.model_args.n_kv_heads
        by_layer = xs.permute(1, 0, 2, 3)
        q = by_layer[:, :, :hq].contiguous()
        k = by_layer[:, :, hq:hq + hkv].contiguous()
        v = by_layer[:, :, hq + hkv:].contiguous()
        return super().forward((q, k, v), ctx)

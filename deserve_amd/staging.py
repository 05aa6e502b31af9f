"""Pinned staging for the small per-step uploads (CSR metadata, attention work lists).

The reference creates its per-step index tensors with ``torch.tensor(...,
device=main_device)`` (deserve_worker/model/context/flash.py:46-64): pageable
host memory, one blocking copy each.  Here the host fills a pinned block and a
kernel of the C-ABI library (``dskv_upload_words``) pulls it to the device on
the caller's stream, so a step holds kernels only and the host never waits.

A block is handed out again once the kernel that read it has run (an event per
block tells); with a host that runs ahead of the GPU the pool simply grows by
one block per step of lead.
"""
from __future__ import annotations

from typing import Dict, List, Optional

import torch

from deserve_amd import _lib

_MIN_WORDS = 1024


class Block:
    """A pinned int32 buffer and the event of the last upload that read it."""

    def __init__(self, words: int) -> None:
        self.tensor = torch.empty((words,), dtype=torch.int32, pin_memory=True)
        self.event: Optional[torch.cuda.Event] = None

    def idle(self) -> bool:
        return self.event is None or self.event.query()


_free: Dict[int, List[Block]] = {}


def take(words: int) -> Block:
    """A block of at least `words` words that no pending upload reads.  It belongs to the
    caller until it is passed to upload()."""
    cap = _MIN_WORDS
    while cap < words:
        cap *= 2
    blocks = _free.setdefault(cap, [])
    for i, blk in enumerate(blocks):
        if blk.idle():
            return blocks.pop(i)
    return Block(cap)


def upload(blk: Block, dst: torch.Tensor, words: int) -> None:
    """Enqueues the copy of the first `words` words of the block to `dst` (int32, on the
    GPU) on the current stream and returns the block to the pool."""
    if dst.dtype != torch.int32 or not dst.is_cuda or not dst.is_contiguous():
        raise ValueError("upload target must be a contiguous int32 tensor on the GPU")
    if words > dst.numel() or words > blk.tensor.numel():
        raise ValueError(f"upload of {words} words into {dst.numel()} from {blk.tensor.numel()}")
    _lib.check(_lib.lib().dskv_upload_words(dst.data_ptr(), blk.tensor.data_ptr(), words,
                                            _lib.current_stream()), "upload_words")
    if blk.event is None:
        blk.event = torch.cuda.Event()
    blk.event.record()
    _free.setdefault(blk.tensor.numel(), []).append(blk)


def to_device(blk: Block, words: int, device: torch.device) -> torch.Tensor:
    """upload() into a fresh device tensor of `words` words (at least one)."""
    dst = torch.empty((max(words, 1),), dtype=torch.int32, device=device)
    upload(blk, dst, words)
    return dst

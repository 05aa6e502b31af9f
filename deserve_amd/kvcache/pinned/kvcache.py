"""(memory, ptr, size) record kept for interface parity
(deserve_worker/kvcache/pinned/kvcache.py:4-8; unused by the reference engine)."""
from dataclasses import dataclass

from deserve_amd.kvcache.pinned.pinned_memory import PinnedMemory


@dataclass
class PinnedKVCache:
    memory: PinnedMemory
    ptr: int
    size: int

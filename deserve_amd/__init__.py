"""deserve_amd - MI355X-native KV-cache hot path of one DeServe pipeline stage.

Host-side mirror of ``deserve_worker.kvcache`` / ``deserve_worker.execution``
(same class and method names) over hand-written gfx950 kernels reached through
the C ABI in ``include/dskv.h`` (``deserve_amd/_lib.py``).
"""
__all__ = ["_lib"]

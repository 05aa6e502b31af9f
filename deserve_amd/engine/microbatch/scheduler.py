"""Import path of deserve_worker/engine/microbatch/scheduler.py; the class lives beside
MicroBatchProcessor."""
from deserve_amd.engine.microbatch.processor import MicroBatchScheduler

__all__ = ["MicroBatchScheduler"]

"""Policy stages of the pipeline scheduler: given the page budget of a step they
decide which tasks execute, which are evicted to host memory and which come back
(deserve_worker/engine/pipeline/stage/__init__.py:7-13).  Pure host logic; the
data movement they request is done by the KV cache manager's swap engine."""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import Tuple

from deserve_amd.task import TaskManager


class Stage(ABC):
    def __init__(self, manager: TaskManager) -> None:
        self.manager = manager

    @abstractmethod
    def process(self, rest_pages: int, request) -> Tuple[int, object]:
        """Takes the pages still free for this step and the step request; returns both, updated."""


def by_length(table) -> list:
    """(task id, tokens) pairs, shortest first; equal lengths keep insertion order."""
    return sorted(table.items(), key=lambda kv: kv[1].shape[0])

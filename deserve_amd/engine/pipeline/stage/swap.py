"""Eviction / reload policy under a page budget
(deserve_worker/engine/pipeline/stage/swap.py:9-107).

Deficit (rest_pages < 0): evict waiting prefills, longest first, then waiting
decodes, longest first, then the tail of the executing decode batch - until the
budget is met.  Surplus: bring evicted prefills back, longest first, then evicted
decodes, each only if it fits, stopping at the first that does not."""
from __future__ import annotations

from typing import Dict, Tuple

from deserve_amd.task import TaskManager

from . import Stage, by_length


class SwapStage(Stage):
    def __init__(self, manager: TaskManager, local_suspended_prefills: Dict[str, object],
                 local_suspended_decodes: Dict[str, object], local_offloaded_prefills: Dict[str, object],
                 local_offloaded_decodes: Dict[str, object]) -> None:
        super().__init__(manager)
        self.local_suspended_prefills = local_suspended_prefills
        self.local_suspended_decodes = local_suspended_decodes
        self.local_offloaded_prefills = local_offloaded_prefills
        self.local_offloaded_decodes = local_offloaded_decodes

    def _evict_waiting(self, rest_pages: int, request, waiting, evicted, pages_of) -> int:
        for task_id, x in reversed(by_length(waiting)):
            if rest_pages >= 0:
                break
            rest_pages += pages_of([task_id])
            del waiting[task_id]
            evicted[task_id] = x
            request.offload_task_ids.append(task_id)
        return rest_pages

    def _evict_executing_tail(self, rest_pages: int, request) -> int:
        """Cuts the decode batch after its first k tasks, k as large as the budget allows
        (at least one task stays)."""
        assert all(n == 1 for n in request.exec_seqlens)
        ids = request.exec_task_ids
        for keep in range(len(ids), 0, -1):
            tail = ids[keep:]
            freed = self.manager.calc_occupied_space(tail) + self.manager.calc_extended_space(tail)
            if rest_pages + freed < 0:
                continue
            cut_xs = request.xs[keep:]
            request.xs = request.xs[:keep]
            request.exec_task_ids = ids[:keep]
            request.exec_seqlens = request.exec_seqlens[:keep]   # the reference leaves these stale
            request.offload_task_ids.extend(tail)
            for i, task_id in enumerate(tail):
                self.local_offloaded_decodes[task_id] = cut_xs[i:i + 1]
                assert self.local_offloaded_decodes[task_id].numel() > 0
            return rest_pages + freed
        # pages are held by other rounds, or the request can never fit
        raise RuntimeError("Unable to fetch enough pages")

    def _reload(self, rest_pages: int, request, evicted, waiting, pages_of) -> int:
        for task_id, x in reversed(by_length(evicted)):
            if rest_pages <= 0:
                break
            need = pages_of([task_id])
            if rest_pages < need:
                break
            rest_pages -= need
            del evicted[task_id]
            waiting[task_id] = x          # waits on the device again; joins a batch later
            request.reload_task_ids.append(task_id)
        return rest_pages

    def process(self, rest_pages: int, request) -> Tuple[int, object]:
        m = self.manager
        if rest_pages < 0:
            rest_pages = self._evict_waiting(rest_pages, request, self.local_suspended_prefills,
                                             self.local_offloaded_prefills, m.calc_initial_space)
            rest_pages = self._evict_waiting(rest_pages, request, self.local_suspended_decodes,
                                             self.local_offloaded_decodes, m.calc_occupied_space)
            if rest_pages < 0:
                rest_pages = self._evict_executing_tail(rest_pages, request)
        else:
            rest_pages = self._reload(rest_pages, request, self.local_offloaded_prefills,
                                      self.local_suspended_prefills, m.calc_initial_space)
            rest_pages = self._reload(rest_pages, request, self.local_offloaded_decodes,
                                      self.local_suspended_decodes, m.calc_occupied_space)
        return rest_pages, request

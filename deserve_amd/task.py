"""Per-request progress record and page arithmetic
(deserve_worker/task.py:26-115).  The reference fixes float16/cuda as module
globals and changes torch's default dtype at import; here they are plain
defaults that every constructor can override, and nothing global is touched."""
from __future__ import annotations

from dataclasses import dataclass, field

import torch

main_dtype = torch.float16
main_device = torch.device("cuda")


@dataclass
class SamplingParams:
    temperature: float = 0.0
    top_p: float = 1.0
    max_seq_len: int = 4096
    max_new_tokens: int = 4096
    dump_probs_num: int = 0

    def model_dump(self) -> dict:
        """The fields as a dict (the reference's pydantic model offers the same call)."""
        return dict(self.__dict__)

    def __setstate__(self, state) -> None:
        # a pickle of the reference's pydantic model carries its fields under "__dict__"
        fields = state.get("__dict__", state) if isinstance(state, dict) else state
        for name in ("temperature", "top_p", "max_seq_len", "max_new_tokens", "dump_probs_num"):
            if name in fields:
                setattr(self, name, fields[name])


@dataclass
class TaskData:
    task_id: str
    start_pos: int
    round: int
    seqlen: int
    initial_seqlen: int
    sampling_params: SamplingParams = field(default_factory=SamplingParams)

    @staticmethod
    def empty(task_id: str, initial_seqlen: int, sampling_params: SamplingParams) -> "TaskData":
        return TaskData(task_id, 0, 0, 0, initial_seqlen, sampling_params)

    def init(self, seqlen: int) -> None:
        self.seqlen = seqlen

    def is_prefill(self) -> bool:
        return self.start_pos >= self.initial_seqlen

    def finished_prefill(self) -> bool:
        return self.start_pos + self.seqlen >= self.initial_seqlen

    def step(self) -> None:
        """Advance past the tokens just processed: decode continues one token at
        a time, an unfinished chunked prefill waits for its next chunk."""
        assert self.seqlen > 0
        self.start_pos += self.seqlen
        self.seqlen = 1 if self.start_pos >= self.initial_seqlen else 0
        self.round += 1


class TaskManager:
    def __init__(self, num_pages: int, page_size: int) -> None:
        self.task_datas: dict[str, TaskData] = {}
        self.page_size = page_size

    def add(self, task_data: TaskData) -> None:
        self.task_datas[task_data.task_id] = task_data

    def get(self, task_id: str) -> TaskData:
        return self.task_datas[task_id]

    def calc_space(self, size: int) -> int:
        return -(-size // self.page_size)

    def _sum(self, task_ids, fn) -> int:
        return sum(fn(self.get(t)) for t in task_ids)

    def calc_occupied_space(self, task_ids: list[str]) -> int:
        return self._sum(task_ids, lambda d: self.calc_space(d.start_pos))

    def calc_initial_space(self, task_ids: list[str]) -> int:
        return self._sum(task_ids, lambda d: self.calc_space(d.initial_seqlen))

    def calc_extended_space(self, task_ids: list[str]) -> int:
        assert all(self.get(t).seqlen > 0 for t in task_ids)
        return self._sum(task_ids, lambda d: self.calc_space(d.start_pos + d.seqlen)
                         - self.calc_space(d.start_pos))

    def calc_seqlens(self, task_ids: list[str]) -> int:
        return self._sum(task_ids, lambda d: d.seqlen)

    def calc_delta_space(self, task_id: str, seqlen: int) -> int:
        d = self.get(task_id)
        return self.calc_space(d.start_pos + seqlen) - self.calc_space(d.start_pos)

    def calc_rest_space(self, task_id: str) -> int:
        d = self.get(task_id)
        return self.calc_space(d.initial_seqlen) - self.calc_space(d.start_pos)

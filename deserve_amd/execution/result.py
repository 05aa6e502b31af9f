"""Result record of one batch step (deserve_worker/execution/result.py:6-13)."""
from dataclasses import dataclass, field

import torch


@dataclass
class BatchResult:
    ongoing_xs: torch.Tensor
    ongoing_task_ids: list
    all_xs: torch.Tensor
    all_task_ids: list
    done_task_ids: list = field(default_factory=list)
    needed_probs: dict = field(default_factory=dict)

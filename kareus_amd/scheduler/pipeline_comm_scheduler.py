"""Steps through one pipeline stage's precomputed schedule, one item per instruction.

The training loop calls ``on_step_begin`` / ``on_instruction_begin(name)`` /
``on_instruction_end(name)`` / ``on_step_end``; the partition engine only reads
``current_schedule``.  State machine and error texts follow
kareus/scheduler/pipeline_comm_scheduler.py: path check ``:36-40``, stage range
``:75-78``, microbatch count in per-microbatch mode ``:83-87``, per-instruction mode
advancing on every instruction and checking its kind ``:104-114``, per-microbatch
mode advancing on forward only ``:115-121``, drained-at-step-end check ``:131-144``.
"""

from __future__ import annotations

import os
from pathlib import Path
from typing import Iterator, List, Optional, Union

from .parser import ScheduleItem, ScheduleItemCP, parse_schedule_file

__all__ = ["PipelineCommScheduler"]

Item = Union[ScheduleItem, ScheduleItemCP]


class PipelineCommScheduler:
    def __init__(
        self,
        configs_pipeline: Union[str, os.PathLike],
        pp_rank: int,
        num_microbatches: int,
        use_activation_checkpointing: bool = False,
        context_parallel: bool = False,
    ) -> None:
        path = Path(str(configs_pipeline))
        if path.suffix != ".py" or not path.exists():
            raise FileNotFoundError(f"configs_pipeline must be an existing .py file, got: {path}")
        self._config_path: Optional[Path] = path.resolve()
        stages = parse_schedule_file(self._config_path, use_activation_checkpointing, context_parallel)
        self._setup(stages, pp_rank, num_microbatches, use_activation_checkpointing, context_parallel)

    @classmethod
    def from_parsed(
        cls,
        parsed: List[List[Item]],
        pp_rank: int,
        num_microbatches: int,
        use_activation_checkpointing: bool = False,
        context_parallel: bool = False,
    ) -> "PipelineCommScheduler":
        """Build from an already parsed schedule (e.g. read once, then shared)."""
        self = cls.__new__(cls)
        self._config_path = None
        self._setup(parsed, pp_rank, num_microbatches, use_activation_checkpointing, context_parallel)
        return self

    def _setup(self, stages, pp_rank, num_microbatches, ac_mode, context_parallel) -> None:
        self._ac_mode = bool(ac_mode)
        self._context_parallel = bool(context_parallel)
        if not 0 <= pp_rank < len(stages):
            raise IndexError(
                f"pp_rank {pp_rank} is out of range for schedule list of length {len(stages)}"
            )
        self._pp_rank = pp_rank
        self._schedule_items: List[Item] = list(stages[pp_rank])
        if not self._ac_mode and num_microbatches != len(self._schedule_items):
            raise ValueError(
                f"Number of microbatches in schedule ({len(self._schedule_items)}) "
                f"does not match num_microbatches ({num_microbatches})"
            )
        self._reset()

    def _reset(self) -> None:
        self._iter_items: Iterator[Item] = iter(self._schedule_items)
        self.current_schedule: Optional[Item] = None

    def on_step_begin(self) -> None:
        pass

    def on_instruction_begin(self, name: str) -> None:
        if self._ac_mode:
            item = next(self._iter_items, None)
            if item is None:
                raise RuntimeError("No more scheduled instructions available for this step")
            expected = "forward" if item.bwd_mlp is None else "backward"
            if expected != name:
                raise RuntimeError(f"Schedule/item mismatch: expected '{expected}', got '{name}'")
            self.current_schedule = item
        elif name == "forward":
            item = next(self._iter_items, None)
            if item is None:
                raise RuntimeError("No more forward microbatches available for this step")
            self.current_schedule = item

    def on_instruction_end(self, name: Optional[str] = None) -> None:
        pass

    def on_step_end(self) -> None:
        extra = next(self._iter_items, None)
        if extra is not None:
            raise RuntimeError(
                f"Schedule returned more items than expected at step end. Next item: {extra}"
            )
        self._reset()

"""Steps through one pipeline stage's frequency plan, one entry per instruction, and pins the
shader clock to it.

The plan is the ``freqs_pipeline_*.py`` file the schedule generator writes next to
``scheds_pipeline_*.py``: per stage a list of ``("forward" | "backward", MHz)`` in the order the
stage executes its 1F1B instructions (tests/kareus/schedules/.../frontier/freqs_pipeline_02328.py:1-4
of the reference).  In the reference the file goes to the Zeus frequency server and a client object
in the training loop switches the clock at every instruction
(tests/artifact/run_kareus.sh:376-381; the hooks are the same four the communication scheduler
gets, kareus/scheduler/pipeline_comm_scheduler.py:97-144).  Here the object reads the file itself
and writes the clock level through sysfs (``kareus_amd.profiling.hardware.set_gpu_frequency``); a
user who may not write those files gets a plan that is stepped through and recorded but not
applied (``applied`` stays False).
"""

from __future__ import annotations

import os
from pathlib import Path
from typing import Callable, Iterator, List, Optional, Tuple, Union

from .parser import parse_frequency_file

__all__ = ["PipelineFrequencyScheduler"]


def _sysfs_setter(device_index: int) -> Callable[[int], bool]:
    from ..profiling.hardware import set_gpu_frequency

    return lambda mhz: set_gpu_frequency(mhz, device_index, settle_s=0.0)


class PipelineFrequencyScheduler:
    """``on_instruction_begin(name)`` takes the next ``(name, MHz)`` of this stage's plan, checks
    the instruction kind and switches the clock when the value differs from the current one.

    ``history`` lists ``(name, MHz, applied)`` for the instructions of the current step;
    ``current_frequency`` is the MHz value last applied (None until a write succeeds).
    """

    def __init__(
        self,
        frequency_file: Union[str, os.PathLike],
        pp_rank: int,
        num_instructions: Optional[int] = None,
        set_frequency: Optional[Callable[[int], bool]] = None,
        reset_frequency: Optional[Callable[[], bool]] = None,
        device_index: int = 0,
    ) -> None:
        path = Path(str(frequency_file))
        if path.suffix != ".py" or not path.exists():
            raise FileNotFoundError(f"frequency_file must be an existing .py file, got: {path}")
        stages = parse_frequency_file(path)
        if not 0 <= pp_rank < len(stages):
            raise IndexError(f"pp_rank {pp_rank} is out of range for frequency list of length {len(stages)}")
        self._plan: List[Tuple[str, int]] = list(stages[pp_rank])
        if num_instructions is not None and num_instructions != len(self._plan):
            raise ValueError(
                f"Number of instructions in the frequency plan ({len(self._plan)}) "
                f"does not match num_instructions ({num_instructions})"
            )
        self._set = set_frequency if set_frequency is not None else _sysfs_setter(device_index)
        if reset_frequency is None:
            from ..profiling.hardware import reset_gpu_clocks

            reset_frequency = lambda: reset_gpu_clocks(device_index)  # noqa: E731
        self._reset_clock = reset_frequency
        self.current_frequency: Optional[int] = None
        self.applied: bool = False
        self.history: List[Tuple[str, int, bool]] = []
        self._iter: Iterator[Tuple[str, int]] = iter(self._plan)

    def on_step_begin(self) -> None:
        self._iter = iter(self._plan)
        self.history = []

    def on_instruction_begin(self, name: str) -> None:
        entry = next(self._iter, None)
        if entry is None:
            raise RuntimeError("No more planned frequencies available for this step")
        expected, mhz = entry
        if expected != name:
            raise RuntimeError(f"Frequency plan mismatch: expected '{expected}', got '{name}'")
        if mhz != self.current_frequency:
            # only a write that went through sets the clock in force; after a failed one the clock
            # is unknown (the setter may have handed it back to the governor), so the next
            # instruction tries again whatever its value
            self.applied = bool(self._set(mhz))
            self.current_frequency = mhz if self.applied else None
        self.history.append((name, mhz, self.current_frequency == mhz))

    def on_instruction_end(self, name: Optional[str] = None) -> None:
        pass

    def on_step_end(self) -> None:
        extra = next(self._iter, None)
        if extra is not None:
            raise RuntimeError(f"Frequency plan has more entries than the step executed. Next entry: {extra}")

    def release(self) -> bool:
        """Hand the clock back to the driver's governor."""
        self.current_frequency = None
        return bool(self._reset_clock())

"""Per-partition time/energy profiling: the measurements Kareus' schedule search is fed with."""

from .hardware import (
    Trial,
    all_configurations,
    append_eval_log,
    available_frequencies_mhz,
    build_eval_record,
    load_eval_log,
    measure,
    measure_batch,
    reset_gpu_clocks,
    set_gpu_frequency,
)
from .partition_executor import DEFAULT_COMM_CHANNELS, PartitionExecutor
from .partition_tests import PARTITION_KEYS, PartitionTest

__all__ = [
    "DEFAULT_COMM_CHANNELS", "PARTITION_KEYS", "PartitionExecutor", "PartitionTest", "Trial",
    "all_configurations", "append_eval_log", "available_frequencies_mhz", "build_eval_record",
    "load_eval_log", "measure", "measure_batch", "reset_gpu_clocks", "set_gpu_frequency",
]

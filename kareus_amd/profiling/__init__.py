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
from .profile_csv import generate_profile_csv, layers_per_stage, pareto_optimal, read_eval_log

__all__ = [
    "DEFAULT_COMM_CHANNELS", "PARTITION_KEYS", "PartitionExecutor", "PartitionTest", "Trial",
    "all_configurations", "generate_profile_csv", "layers_per_stage", "pareto_optimal", "read_eval_log", "append_eval_log", "available_frequencies_mhz", "build_eval_record",
    "load_eval_log", "measure", "measure_batch", "reset_gpu_clocks", "set_gpu_frequency",
]

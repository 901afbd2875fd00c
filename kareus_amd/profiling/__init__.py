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
    nominal_frequency_mhz,
    reset_gpu_clocks,
    set_gpu_frequency,
)
from .partition_executor import DEFAULT_COMM_CHANNELS, PartitionExecutor
from .partition_tests import PARTITION_KEYS, PartitionTest

# the two command-line modules (``python -m kareus_amd.profiling.profile_csv`` / ``.plan_generator``)
# are imported on first use, so that running one as a script does not find it imported already
_LAZY = {
    "generate_profile_csv": "profile_csv", "layers_per_stage": "profile_csv", "pareto_optimal": "profile_csv",
    "read_eval_log": "profile_csv", "generate_plans": "plan_generator", "plan_frontier": "plan_generator",
    "pipeline_frontier": "plan_generator",
}


def __getattr__(name):
    module = _LAZY.get(name)
    if module is None:
        raise AttributeError(f"module {__name__!r} has no attribute {name!r}")
    import importlib

    return getattr(importlib.import_module(f"{__name__}.{module}"), name)


__all__ = [
    "DEFAULT_COMM_CHANNELS", "PARTITION_KEYS", "PartitionExecutor", "PartitionTest", "Trial",
    "all_configurations", "append_eval_log", "available_frequencies_mhz", "build_eval_record",
    "generate_plans", "generate_profile_csv", "layers_per_stage", "load_eval_log", "measure", "measure_batch",
    "nominal_frequency_mhz", "pareto_optimal", "pipeline_frontier", "plan_frontier", "read_eval_log",
    "reset_gpu_clocks", "set_gpu_frequency",
]

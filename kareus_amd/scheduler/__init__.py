from .parser import (
    CommConfig,
    ScheduleItem,
    ScheduleItemCP,
    parse_frequency_file,
    parse_schedule_file,
)
from .pipeline_comm_scheduler import PipelineCommScheduler

__all__ = [
    "CommConfig",
    "ScheduleItem",
    "ScheduleItemCP",
    "parse_schedule_file",
    "parse_frequency_file",
    "PipelineCommScheduler",
]

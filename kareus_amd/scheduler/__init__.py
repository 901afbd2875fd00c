from .parser import (
    CommConfig,
    ScheduleItem,
    ScheduleItemCP,
    parse_frequency_file,
    parse_schedule_file,
)
from .pipeline_comm_scheduler import PipelineCommScheduler
from .pipeline_frequency_scheduler import PipelineFrequencyScheduler

__all__ = [
    "CommConfig",
    "ScheduleItem",
    "ScheduleItemCP",
    "parse_schedule_file",
    "parse_frequency_file",
    "PipelineCommScheduler",
    "PipelineFrequencyScheduler",
]

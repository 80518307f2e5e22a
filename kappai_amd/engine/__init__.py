from .batch import RowBatch, StepEntry, layout_rows
from .engine import Engine, EngineConfig, Metrics, StepOutput
from .scheduler import Request, Scheduled, Scheduler, SchedulerConfig
from .step import StepRunner

__all__ = ["RowBatch", "StepEntry", "layout_rows", "Engine", "EngineConfig", "Metrics",
           "StepOutput", "Request", "Scheduled", "Scheduler", "SchedulerConfig", "StepRunner"]

from ..sampling import SamplingParams
from .batch import BatchError, StepContext, StepEntry, build_context
from .engine import Engine, Request, StepOutput, StepRecord
from .runner import ModelRunner
from .scheduler import Planned, Scheduler, SchedulerError

__all__ = ["SamplingParams", "BatchError", "StepContext", "StepEntry", "build_context", "Engine", "Request",
           "StepOutput", "StepRecord", "ModelRunner", "Planned", "Scheduler", "SchedulerError"]

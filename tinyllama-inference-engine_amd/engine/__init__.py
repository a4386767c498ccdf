from .engine import Engine, parse_dtype
from .scheduler import Request, SamplingParams, Scheduled, Scheduler
from .step import GroupView, ModelRunner, StepContext, StepEntry, StepTimings

__all__ = ["Engine", "parse_dtype", "Request", "SamplingParams", "Scheduled", "Scheduler", "GroupView", "ModelRunner",
           "StepContext", "StepEntry", "StepTimings"]

from .engine import Engine, parse_dtype
from .step import GroupView, ModelRunner, StepContext, StepEntry

__all__ = ["Engine", "parse_dtype", "GroupView", "ModelRunner", "StepContext", "StepEntry"]

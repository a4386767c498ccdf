"""An inference engine for the Llama dense decoder on one MI355X (gfx950).

    from tlie_amd import Engine, StepEntry
    engine = Engine(model_dir, dtype="bfloat16")
    tokens = engine.generate([[1, 15043, 3186]], max_tokens=16)
"""
from . import models as _models  # noqa: F401
from .config import LlamaConfig, ModelSpec, PartSpec
from .engine import Engine, StepEntry
from .errors import EngineError, ErrorCode
from .registry import register
from .weights import WeightStore, write_random_model

__all__ = ["Engine", "StepEntry", "EngineError", "ErrorCode", "LlamaConfig", "ModelSpec", "PartSpec", "register",
           "WeightStore", "write_random_model"]

"""The engine: a model folder in, a step function and generation out.

`Engine(model_dir)` reads config.json, finds the architecture in the registry, checks and loads
the weights, builds the model from its parts, makes the cache pools, and offers
  step(entries)      the step function (see engine/step.py)
  admit / finish     a request's slot and pages
  generate(...)      prompts to tokens through the scheduler and the sampler
"""
from __future__ import annotations

from typing import Hashable, Sequence

import torch

from .. import models as _models  # noqa: F401  (registers architectures and parts)
from ..cache.manager import CacheManager
from ..config.llama import read_config_json
from ..errors import EngineError, ErrorCode, invalid_argument
from ..models.builder import build_model, expected_tensors
from ..registry import config_from_dict
from ..weights.store import WeightStore
from .step import ModelRunner, StepEntry

_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "f32": torch.float32,
           "fp32": torch.float32}


def parse_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name in (torch.bfloat16, torch.float32):
            return name
    elif str(name).lower() in _DTYPES:
        return _DTYPES[str(name).lower()]
    raise EngineError(ErrorCode.INVALID_DTYPE, f"the engine runs in bfloat16 or float32, not {name}")


class Engine:
    def __init__(self, model_dir: str, dtype="bfloat16", max_tokens: int = 4096, page_size: int = 16,
                 max_requests: int = 64, device: str = "cuda:0"):
        """max_tokens: how many positions the cache pools hold in all (rounded up to whole
        pages); max_requests: how many requests can be live at once."""
        if not torch.cuda.is_available():
            raise EngineError(ErrorCode.HIP, "no GPU is visible: the engine has no CPU path")
        self.dtype = parse_dtype(dtype)
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        self.config = config_from_dict(read_config_json(model_dir))
        self.spec = self.config.to_spec()
        store = WeightStore(model_dir)
        weights = store.load(expected_tensors(self.spec), self.dtype, self.device)
        self.model = build_model(self.spec, weights, self.dtype, self.device)
        if max_tokens <= 0:
            raise invalid_argument("max_tokens must be positive")
        num_pages = (max_tokens + page_size - 1) // page_size
        self.cache = CacheManager(self.model.run_needs(), page_size, num_pages, max_requests, self.dtype, self.device,
                                  max_positions=self.spec.max_positions)
        self.runner = ModelRunner(self.model, self.cache)

    # ---- the step function and what goes with it --------------------------------------------------
    def admit(self, request: Hashable) -> int:
        return self.cache.admit(request)

    def finish(self, request: Hashable) -> None:
        self.cache.release(request)

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        return self.runner.step(entries)

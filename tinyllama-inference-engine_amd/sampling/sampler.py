"""Sampling from the step's logits.

reference: greedy is the first index of the maximum and refuses NaN or Inf
(src/operators.cpp:166-175); with temperature > 0 the server draws from the top-p part of
softmax(logits / T) (app/server.cpp:237-277) with a generator seeded per request (:198).  Here the
draw is made on the device by one kernel for all rows, and the uniform number for a row is a
hash of (the request's seed, the index of the token being generated): it is the same whatever
else is in the batch and however the prompt was cut, also after a preemption.
"""
from __future__ import annotations

import torch

from .. import ops
from ..errors import EngineError, ErrorCode

MASK64 = (1 << 64) - 1


def splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & MASK64
    x = ((x ^ (x >> 30)) * 0xBF58476D1CE4E5B9) & MASK64
    x = ((x ^ (x >> 27)) * 0x94D049BB133111EB) & MASK64
    return x ^ (x >> 31)


def uniform01(seed: int, counter: int) -> float:
    """The uniform number in [0, 1) that the kernel uses for (seed, counter): 24 bits."""
    h = splitmix64(splitmix64(seed & MASK64) ^ ((counter * 0xD1342543DE82EF95 + 1) & MASK64))
    return (h >> 40) / 16777216.0


def _signed(value: int) -> int:
    value &= MASK64
    return value - (1 << 64) if value >= (1 << 63) else value


class Sampler:
    def __init__(self, device):
        self.device = device

    def sample(self, logits: torch.Tensor, params: list, counters: list[int]) -> list[int]:
        """One token per row.  params[i] has temperature, top_p and seed; counters[i] is the
        index of the token row i generates.  Raises `numerical_error` on NaN or Inf logits."""
        rows = logits.shape[0]
        if rows == 0:
            return []
        if all(not p.temperature > 0.0 for p in params):
            tokens = ops.sample(logits)
        else:
            temperature = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32, device=self.device)
            top_p = torch.tensor([float(p.top_p) for p in params], dtype=torch.float32, device=self.device)
            seed = torch.tensor([_signed(int(p.seed)) for p in params], dtype=torch.int64, device=self.device)
            counter = torch.tensor([int(c) for c in counters], dtype=torch.int64, device=self.device)
            tokens = ops.sample(logits, temperature, top_p, seed, counter)
        out = tokens.cpu().tolist()
        if any(token < 0 for token in out):
            raise EngineError(ErrorCode.NUMERICAL, "logits contain NaN or Inf")
        return out

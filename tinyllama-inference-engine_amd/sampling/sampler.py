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


class PendingTokens:
    """A step's sampled tokens on their way to the host.  `read()` waits for them."""

    def __init__(self, host: torch.Tensor, event, rows: int):
        self._host, self._event, self.rows = host, event, rows

    def read(self) -> list[int]:
        if self._event is not None:
            self._event.synchronize()
        out = self._host[:self.rows].tolist()
        if any(token < 0 for token in out):
            raise EngineError(ErrorCode.NUMERICAL, "logits contain NaN or Inf")
        return out


class Sampler:
    """Samples on the device into a buffer that stays where it is (`device_tokens`: a decode step
    can take its tokens from there before the host has seen them) and copies the tokens to pinned
    host memory without waiting.  Two sets of host buffers are used in turn: a caller may have at
    most one `PendingTokens` unread when it samples again."""

    def __init__(self, device, capacity: int = 64):
        self.device = torch.device(device)
        self.capacity = capacity
        self.device_tokens = torch.zeros(capacity, dtype=torch.int32, device=self.device)
        self._floats = torch.zeros((2, capacity), dtype=torch.float32, device=self.device)      # temperature, top_p
        self._longs = torch.zeros((2, capacity), dtype=torch.int64, device=self.device)         # seed, counter
        self._host_tokens = [torch.zeros(capacity, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._host_floats = [torch.zeros((2, capacity), dtype=torch.float32, pin_memory=True) for _ in range(2)]
        self._host_longs = [torch.zeros((2, capacity), dtype=torch.int64, pin_memory=True) for _ in range(2)]
        self._events = [torch.cuda.Event(), torch.cuda.Event()]
        self._turn = 0

    def sample_async(self, logits: torch.Tensor, params: list, counters: list[int]) -> PendingTokens:
        """One token per row, left in `device_tokens[:rows]` and on its way to the host.
        params[i] has temperature, top_p and seed; counters[i] is the index of the token row i
        generates."""
        rows = logits.shape[0]
        if rows == 0:
            return PendingTokens(self._host_tokens[0], None, 0)
        if rows > self.capacity:
            raise EngineError(ErrorCode.INVALID_ARGUMENT, f"the sampler was made for {self.capacity} rows, not {rows}")
        turn = self._turn
        self._turn ^= 1
        out = self.device_tokens[:rows]
        if all(not p.temperature > 0.0 for p in params):
            ops.sample(logits, out=out)
        else:
            floats, longs = self._host_floats[turn], self._host_longs[turn]
            floats[0, :rows] = torch.tensor([float(p.temperature) for p in params], dtype=torch.float32)
            floats[1, :rows] = torch.tensor([float(p.top_p) for p in params], dtype=torch.float32)
            longs[0, :rows] = torch.tensor([_signed(int(p.seed)) for p in params], dtype=torch.int64)
            longs[1, :rows] = torch.tensor([int(c) for c in counters], dtype=torch.int64)
            self._floats.copy_(floats, non_blocking=True)
            self._longs.copy_(longs, non_blocking=True)
            ops.sample(logits, self._floats[0, :rows], self._floats[1, :rows], self._longs[0, :rows], self._longs[1, :rows],
                       out=out)
        host = self._host_tokens[turn]
        host[:rows].copy_(out, non_blocking=True)
        self._events[turn].record()
        return PendingTokens(host, self._events[turn], rows)

    def sample(self, logits: torch.Tensor, params: list, counters: list[int]) -> list[int]:
        """One token per row, on the host.  Raises `numerical_error` on NaN or Inf logits."""
        return self.sample_async(logits, params, counters).read()

"""The interfaces of the parts a model is put together from.

A part is built from its `PartSpec` (sizes and constants), says which tensors it expects under a
prefix, takes them, and runs on the tokens of one step.  It does not know which model it is in,
which layer it is, or how the step was cut; what it may need to know about the step (positions,
which sequence a token belongs to, where its cache rows are) arrives in the `StepContext`, and
what the cache manager holds for it arrives in the `Binding`.

    Norm           forward(residual f32 [T, H]) -> [T, H] in the activation type
                   add_forward(residual, delta, rows=None): residual += delta, then forward
    Mixer          forward(x [T, H], ctx, binding) -> Product or tensor [T, H]
                   cache_need() -> CacheNeed | None;  state_need() -> StateNeed | None
    FeedForward    forward(x [T, H], ctx) -> Product or tensor [T, H]
                   (both may opt into the fusions of steps of few rows, see Mixer below)
    PositionEncoding
                   rotary_table() -> (inv_freq, rot_dim) | None   (lets attention fuse it)
                   apply_qk(q, k, positions) -> (q, k)             (any other scheme)
    Block          forward(residual, pending, ctx, binding) -> pending
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any

import torch

from ..config.spec import PartSpec, TensorSpec
from ..ops import NormedRows, Product, ResidualUpdated, as_product


@dataclass(frozen=True)
class CacheNeed:
    """Pages of whatever a mixer keeps per position.  A page of `page_size` positions is a tensor
    of shape (*planes, page_size * width): in each of the prod(planes) planes, `width` values for
    each of the page's positions.  How the positions and values lie inside a plane is the mixer's
    own business (its kernels write and read the pages); the cache manager allocates and numbers
    pages and looks at nothing inside them.  `dtype` None: the activation type of the run.
    `window` None: every position stays; else only the last `window` positions are ever read again
    (pages that no later token can see are given back)."""
    planes: tuple[int, ...]
    width: int
    window: int | None = None
    dtype: torch.dtype | None = None

    def page_shape(self, page_size: int) -> tuple[int, ...]:
        return (*self.planes, page_size * self.width)

    def values_per_position(self) -> int:
        count = self.width
        for plane in self.planes:
            count *= plane
        return count


@dataclass(frozen=True)
class StateNeed:
    """State of fixed size per request: one row of `shape` in an area indexed by request slot."""
    shape: tuple[int, ...]
    dtype: torch.dtype = torch.float32


@dataclass
class Binding:
    """What the cache manager holds for one run of a layer."""
    group: int | None = None            # index of the page group (block table, slot map) in the step context
    cache: torch.Tensor | None = None   # [pages, *need.page_shape(page_size)] of the run whose cache is read
    writes: bool = True                 # this run owns the cache and writes the step's keys and values
    state: torch.Tensor | None = None   # [request slots, *shape] for a mixer with state of its own


class Part:
    # A part whose forward only launches kernels on the current stream, with sizes that depend on
    # nothing but the number of tokens and sequences (no reading of the step's host arrays, no
    # synchronisation), may be recorded into a HIP graph.  Parts say so themselves.
    graph_safe = False

    def __init__(self, spec: PartSpec, dtype: torch.dtype, device):
        self.spec = spec
        self.dtype = dtype              # the activation type: float32 or bfloat16
        self.device = device

    @classmethod
    def tensor_specs(cls, spec: PartSpec, prefix: str) -> list[TensorSpec]:
        return []

    def load(self, weights: dict[str, torch.Tensor], prefix: str) -> None:
        pass


@dataclass
class ResidualTarget:
    """Handed to a mixer or feed-forward that can add its result into the residual itself (in the
    kernel of its last product): the float32 residual, and (weight, eps) of the norm that reads the
    residual next, or None."""
    residual: torch.Tensor
    next_norm: tuple | None = None


class Norm(Part):
    def forward(self, residual: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError

    def lazy_params(self):
        """(weight, eps) when this norm can be folded into the product that follows it (its
        weight applied to the residual by whoever writes the residual, its scale to the product's
        rows), else None."""
        return None

    def add_forward(self, residual: torch.Tensor, delta, rows: torch.Tensor | None = None, lazy: bool = False):
        """Unfused default: add in place, then norm; with `rows`, norm those rows of the sum only.
        `delta` may be a `ResidualUpdated`: then the residual already holds it."""
        if isinstance(delta, ResidualUpdated):
            delta = None
        if rows is not None:
            picked = residual[rows.long()]
            if delta is not None:
                picked = picked + as_product(delta).dense(torch.float32)[rows.long()]
            return self.forward(picked.contiguous())
        if delta is not None:
            residual += as_product(delta).dense(torch.float32)
        return self.forward(residual)


class PositionEncoding(Part):
    def rotary_table(self):
        return None

    def apply_qk(self, q: torch.Tensor, k: torch.Tensor, positions: torch.Tensor):
        return q, k


class Mixer(Part):
    def cache_need(self) -> CacheNeed | None:
        return None

    def state_need(self) -> StateNeed | None:
        return None

    def forward(self, x: torch.Tensor, ctx: Any, binding: Binding):
        raise NotImplementedError

    # A mixer (or feed-forward) may offer two things to a block that runs a step of few rows:
    #   takes_normed_rows(rows) -> True: `x` may be a `NormedRows` (the norm before it is folded
    #       into its first product);
    #   adds_to_residual = True: `forward(..., into=ResidualTarget)` adds the result into the
    #       residual itself and returns a `ResidualUpdated` (or, when it cannot for this step, its
    #       result as usual).
    adds_to_residual = False

    def takes_normed_rows(self, rows: int) -> bool:
        return False


class FeedForward(Part):
    adds_to_residual = False

    def takes_normed_rows(self, rows: int) -> bool:
        return False

    def forward(self, x: torch.Tensor, ctx: Any):
        raise NotImplementedError


__all__ = ["CacheNeed", "StateNeed", "Binding", "Part", "Norm", "PositionEncoding", "Mixer", "FeedForward",
           "Product", "as_product", "NormedRows", "ResidualUpdated", "ResidualTarget"]

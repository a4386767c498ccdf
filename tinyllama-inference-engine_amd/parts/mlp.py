"""The SiLU-gated feed-forward: down(silu(gate(x)) * up(x)) (src/model.cpp:187-196 of the
reference; SiluMultiply, src/operators.cpp:157-159).  gate and up are one product over the
weight [2 * inter, hidden] whose rows alternate gate and up (g0, u0, g1, u1, ...): the product of
few rows then has a gate and its up in one lane and applies the activation itself."""
from __future__ import annotations

from functools import partial

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
from ..weights.arena import keep_in
from .base import FeedForward
from .linear import Linear


@register("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    """spec: hidden_size, intermediate_size, activation ("silu").
    Tensors: `<prefix>{gate,up,down}_proj.weight`."""
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.hidden = int(spec["hidden_size"])
        self.inter = int(spec["intermediate_size"])
        if spec.get("activation", "silu") != "silu":
            raise invalid_config(f"gated_mlp: activation '{spec['activation']}' is not implemented")
        self.gate_up = self.down = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        hidden, inter = int(spec["hidden_size"]), int(spec["intermediate_size"])
        return [TensorSpec(prefix + "gate_proj.weight", (inter, hidden)),
                TensorSpec(prefix + "up_proj.weight", (inter, hidden)),
                TensorSpec(prefix + "down_proj.weight", (hidden, inter))]

    def load(self, weights, prefix):
        gate, up = weights[prefix + "gate_proj.weight"], weights[prefix + "up_proj.weight"]
        keep = partial(keep_in, weights)
        self.gate_up = Linear(torch.stack([gate, up], dim=1).reshape(2 * self.inter, self.hidden), None, self.dtype, keep=keep)
        self.down = Linear(weights[prefix + "down_proj.weight"], None, self.dtype, keep=keep)

    adds_to_residual = True

    def takes_normed_rows(self, rows: int) -> bool:
        return self.gate_up.takes_rows(rows)

    def forward(self, x, ctx, into=None):
        hidden = self.gate_up(x, gated=True)
        if isinstance(hidden, ops.Product):
            hidden = ops.silu_mul(hidden, self.dtype, interleaved=True)
        return self.down(hidden, into=into)

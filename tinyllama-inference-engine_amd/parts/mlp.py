"""The SiLU-gated feed-forward: down(silu(gate(x)) * up(x)) (src/model.cpp:187-196 of the
reference; SiluMultiply, src/operators.cpp:157-159).  gate and up are one product over the
concatenated weight [2 * inter, hidden]."""
from __future__ import annotations

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..errors import invalid_config
from ..registry import register
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
        self.gate_up = Linear(torch.cat([weights[prefix + "gate_proj.weight"], weights[prefix + "up_proj.weight"]], dim=0),
                              None, self.dtype)
        self.down = Linear(weights[prefix + "down_proj.weight"], None, self.dtype)

    def forward(self, x, ctx):
        return self.down(ops.silu_mul(self.gate_up(x), self.dtype))

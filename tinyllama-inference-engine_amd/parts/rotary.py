"""Rotary positions, half-split pairing: the pair (i, i + d/2) of every head is turned by
angle = float(position) * theta^(-2i/d) (src/operators.cpp:58-73 of the reference).  The
frequencies are made once, in float32 as the reference forms them (`std::pow` on floats,
:63-64); the angle, sine and cosine are float32 in the kernel."""
from __future__ import annotations

import torch

from ..config.spec import PartSpec
from ..errors import invalid_config
from ..registry import register
from .base import PositionEncoding


@register("position_encoding", "rotary")
class Rotary(PositionEncoding):
    """spec: head_dim, theta, optionally rot_dim (default head_dim: the whole head turns)."""
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.head_dim = int(spec["head_dim"])
        self.rot_dim = int(spec.get("rot_dim", self.head_dim))
        self.theta = float(spec["theta"])
        if self.rot_dim % 2 != 0 or not 0 < self.rot_dim <= self.head_dim:
            raise invalid_config(f"rotary: rot_dim {self.rot_dim} must be even and at most head_dim {self.head_dim}")
        if not self.theta > 0:
            raise invalid_config("rotary: theta must be positive")
        index = torch.arange(self.rot_dim // 2, dtype=torch.float32)
        exponent = (-2.0 * index) / float(self.rot_dim)
        self.inv_freq = torch.pow(torch.tensor(self.theta, dtype=torch.float32), exponent).to(device)

    def rotary_table(self):
        return self.inv_freq, self.rot_dim


@register("position_encoding", "none")
class NoPositions(PositionEncoding):
    """No position encoding in the mixer (keys are cached as projected)."""
    graph_safe = True

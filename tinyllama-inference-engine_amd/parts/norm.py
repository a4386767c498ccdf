"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w (src/operators.cpp:22-45 of the reference; its
device form, src/cuda/kernels.cu:67-84).  The residual it reads is float32; the sum of squares,
the scale and the product are float32; the output is in the activation type."""
from __future__ import annotations

import torch

from .. import ops
from ..config.spec import PartSpec, TensorSpec
from ..registry import register
from ..weights.arena import keep_in
from .base import Norm, ResidualUpdated, as_product


@register("norm", "rms_norm")
class RMSNorm(Norm):
    """spec: size, eps.  Tensor: `<prefix>weight` [size]."""
    graph_safe = True

    def __init__(self, spec: PartSpec, dtype, device):
        super().__init__(spec, dtype, device)
        self.size = int(spec["size"])
        self.eps = float(spec["eps"])
        self.weight = None

    @classmethod
    def tensor_specs(cls, spec, prefix):
        return [TensorSpec(prefix + "weight", (int(spec["size"]),), init="norm")]

    def load(self, weights, prefix):
        self.weight = keep_in(weights, weights[prefix + "weight"].contiguous())

    def forward(self, residual):
        return ops.add_rmsnorm(residual, None, self.weight, self.eps, self.dtype)

    def lazy_params(self):
        return self.weight, self.eps

    def add_forward(self, residual, delta, rows=None, lazy=False):
        if isinstance(delta, ResidualUpdated):
            # the residual holds the sum already; if its writer also left this norm's inputs and the
            # reader can fold the norm into its product, nothing is launched here
            if lazy and rows is None and delta.normed is not None:
                return delta.normed
            delta = None
        product = as_product(delta) if delta is not None else None
        return ops.add_rmsnorm(residual, product, self.weight, self.eps, self.dtype, rows=rows)

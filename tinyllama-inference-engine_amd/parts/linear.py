"""y = x . W^T (+ b), W stored [out, in] as the reference stores and applies it
(src/model.cpp:65-72; src/cuda/kernels.cu:359-363).

Which kernel runs is decided here and nowhere else:
  float32 activations            the true 32-bit kernel (plain FMAs, no matrix instruction)
  bfloat16, weight kept float32  the same kernel on widened values
  bfloat16                       the tiled MFMA kernels when they take the sizes, else the plain one
"""
from __future__ import annotations

import torch

from .. import ops
from ..ops import Product


class Linear:
    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None, dtype: torch.dtype):
        self.weight = weight.contiguous()
        self.bias = bias.contiguous() if bias is not None else None
        if self.bias is not None and self.bias.dtype != self.weight.dtype:
            self.bias = self.bias.to(self.weight.dtype)
        self.dtype = dtype
        self.out_features, self.in_features = self.weight.shape

    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype | None = None) -> Product:
        out_dtype = out_dtype or self.dtype
        return ops.gemm_generic(x, self.weight, self.bias, out_dtype)

"""y = x . W^T (+ b), W stored [out, in] as the reference stores and applies it
(src/model.cpp:65-72; src/cuda/kernels.cu:359-363).

Which kernel runs is decided here and nowhere else:
  float32 activations            the true 32-bit kernel (plain FMAs, no matrix instruction)
  bfloat16, weight kept float32  the same kernel on widened values
  bfloat16, at most 64 rows      the skinny MFMA kernel (W streamed once, split-K partial sums)
  bfloat16, more rows            the library's product (as the reference uses a library for its
                                 products: cublasGemmEx, src/cuda/kernels.cu:342-368), bfloat16 out
  anything those refuse          the plain kernel
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

    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype | None = None, whole: bool = False) -> Product:
        """out_dtype: what a dense result is stored in (the skinny kernel's partial sums are float32
        whatever it says).  whole: the caller has no kernel that adds partial sums up, so the
        product must come as one array (the skinny kernel then does not split K)."""
        out_dtype = out_dtype or self.dtype
        if ops.gemm_skinny_takes(x, self.weight) and (not whole or out_dtype == torch.float32):
            split_len = (self.in_features + 63) // 64 * 64 if whole else None
            return ops.gemm_skinny(x, self.weight, self.bias, split_len=split_len)
        if x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and out_dtype == torch.bfloat16:
            ops._device_tensor(x, "x", torch.bfloat16)
            if x.dim() != 2 or x.shape[1] != self.in_features:
                raise ops.invalid_shape(f"linear: x {list(x.shape)} does not fit weight {list(self.weight.shape)}")
            if self.bias is not None:
                return Product(torch.addmm(self.bias, x, self.weight.t()), 1)
            return Product(torch.mm(x, self.weight.t()), 1)
        return ops.gemm_generic(x, self.weight, self.bias, out_dtype)

"""y = x . W^T (+ b), W stored [out, in] as the reference stores and applies it
(src/model.cpp:65-72; src/cuda/kernels.cu:359-363).

Which kernel runs is decided here and nowhere else:
  float32 activations            the true 32-bit kernel (plain FMAs, no matrix instruction)
  bfloat16, weight kept float32  the same kernel on widened values
  bfloat16, at most 16 rows      the rows kernel when the caller folds something in: the norm before the
                                 product, the SiLU gate or the add into the residual after it
  bfloat16, at most 64 rows      the skinny MFMA kernel (W streamed once, split-K partial sums; the gated
                                 feed-forward's first product keeps K whole and applies the SiLU gate itself)
  bfloat16, more rows            the library's product (as the reference uses a library for its
                                 products: cublasGemmEx, src/cuda/kernels.cu:342-368), bfloat16 out, or
                                 float32 for the output head: hipBLASLt called directly
                                 (`ops.library_mm`), the plain kernel where that fails
  anything those refuse          the plain kernel
"""
from __future__ import annotations

import torch

from .. import ops
from ..ops import Product


class Linear:
    def __init__(self, weight: torch.Tensor, bias: torch.Tensor | None, dtype: torch.dtype, keep=None):
        """keep: what gives a tensor its place for good (`keep_in` of the mapping that the part loads
        from); without it the tensors stay where they are."""
        keep = keep or (lambda tensor: tensor)
        self.weight = keep(weight.contiguous())
        if bias is not None and bias.dtype != self.weight.dtype:
            bias = bias.to(self.weight.dtype)
        self.bias = keep(bias.contiguous()) if bias is not None else None
        self.dtype = dtype
        self.out_features, self.in_features = self.weight.shape

    def takes_rows(self, rows: int) -> bool:
        """Whether a step of `rows` rows can go to the rows kernel (and so may bring a `NormedRows`,
        ask for the gate, or for the add into the residual)."""
        return ops.gemm_rows_takes(rows, self.weight, self.dtype)

    def __call__(self, x, out_dtype: torch.dtype | None = None, whole: bool = False, into=None, gated: bool = False,
                 rope=None):
        """out_dtype: what a dense result is stored in (the skinny kernel's partial sums are float32
        whatever it says).  whole: the caller has no kernel that adds partial sums up, so the
        product must come as one array (the skinny kernel then does not split K).
        into (a `ResidualTarget`): add the result into the residual, if the kernel for this step can
        (then a `ResidualUpdated` comes back, else the result as usual).  gated: the weight's rows
        alternate gate and up; if the kernel for this step can, silu(gate) * up comes back as a
        tensor, else the product as usual.  rope (an `ops.RopeTarget`; the weight's rows are in
        paired order): if the kernel for this step can, q and k are rotated, k and v written to the
        cache and q comes back as a tensor, else the product as usual."""
        out_dtype = out_dtype or self.dtype
        if self.takes_rows(x.shape[0]):
            if into is not None:
                return ops.gemm_rows(x, self.weight, self.bias, "residual", residual=into.residual, next_norm=into.next_norm)
            if gated:
                return ops.gemm_rows(x, self.weight, self.bias, "silu")
            if rope is not None:
                return ops.gemm_rows(x, self.weight, self.bias, "rope", rope=rope)
            if isinstance(x, ops.NormedRows):
                return ops.gemm_rows(x, self.weight, self.bias, "store")
        if isinstance(x, ops.NormedRows):
            raise ops.invalid_argument("this product cannot fold the norm before it; ask takes_rows() first")
        if gated and ops.gemm_skinny_takes(x, self.weight) and self.out_features % 2 == 0:
            return ops.gemm_skinny(x, self.weight, self.bias, gated=True)     # all of K in a workgroup: the gate is applied there
        if ops.gemm_skinny_takes(x, self.weight) and (not whole or out_dtype == torch.float32):
            split_len = (self.in_features + 63) // 64 * 64 if whole else None
            return ops.gemm_skinny(x, self.weight, self.bias, split_len=split_len)
        if x.dtype == torch.bfloat16 and self.weight.dtype == torch.bfloat16 and out_dtype in (torch.bfloat16, torch.float32):
            ops._device_tensor(x, "x", torch.bfloat16)
            if x.dim() != 2 or x.shape[1] != self.in_features:
                raise ops.invalid_shape(f"linear: x {list(x.shape)} does not fit weight {list(self.weight.shape)}")
            if self.bias is not None:
                # the library's product comes without the bias: it joins the float32 sums in a kernel of this
                # library's own, as in the kernels that add it themselves, and the sum is rounded once
                return Product(ops.add_bias(ops.library_mm(x, self.weight, torch.float32), self.bias, out_dtype), 1)
            return Product(ops.library_mm(x, self.weight, out_dtype), 1)   # (float32: the output head's logits for many rows)
        return ops.gemm_generic(x, self.weight, self.bias, out_dtype)

"""A projection y = x W^T (+ b) (+ residual), W stored [out, in].

Not a part of its own: mixers and feed-forwards own their projections and
call this helper, which picks the kernel from the types and sizes at hand:

* float32 weights (the 32-bit path, or a tensor the file stores in 32-bit):
  the plain kernel, true float32 throughout;
* bfloat16 weights and activations: the MFMA kernels (a skinny one for a few
  rows, a tiled one for many) when the sizes fit them, else the plain kernel.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor], fast: bool = True):
        if weight.dim() != 2:
            raise ValueError("a projection weight must be [out, in]")
        if bias is not None and bias.numel() != weight.shape[0]:
            raise ValueError(f"bias has {bias.numel()} elements, the projection has {weight.shape[0]} outputs")
        self.weight = weight.contiguous()
        self.bias = None if bias is None else bias.contiguous()
        self.fast = fast
        self.n_out, self.n_in = weight.shape

    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype, resid: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
        w = self.weight
        if w.dtype == torch.float32 and x.dtype != torch.float32:
            x = ops.cast(x, torch.float32)
        if self.fast and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
            y = ops.gemm_bf16(x, w, self.bias, resid, out_dtype, out)
            if y is not None:
                return y
        return ops.gemm_plain(x, w, self.bias, resid, out_dtype, out)

    def gated(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """silu(x Wg^T) * (x Wu^T) for a stacked weight [Wg; Wu]: one fused kernel on the
        matrix cores when the sizes allow, else the product in float32 and the activation kernel."""
        w = self.weight
        if self.fast and w.dtype == torch.bfloat16 and x.dtype == torch.bfloat16:
            y = ops.gemm_bf16(x, w, None, None, out_dtype, gated=True)
            if y is not None:
                return y
        return ops.silu_mul(self(x, torch.float32), out_dtype)

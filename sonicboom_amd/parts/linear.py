"""A projection y = x W^T (+ b) (+ residual), W stored [out, in].

Not a part of its own: mixers and feed-forwards own their projections and
call this helper, which picks the kernel from the types and sizes at hand:

* float32 weights (the 32-bit path, or a tensor the file stores in 32-bit):
  the plain kernel, true float32 throughout;
* bfloat16 weights and activations: the matrix-core kernels (two that stream
  the weights once for few rows, a tiled one for more).  For them the weight is
  re-laid once, when the projection is built, into the tile order the matrix
  cores read (:func:`sonicboom_amd.ops.pack_weight`) and the row-major copy is
  dropped.  An inner size that is not a multiple of 8 keeps the row-major
  weight and the plain kernel.

``gated=True`` marks a stacked weight [W_gate; W_up] whose product is
act(x W_gate^T) * (x W_up^T), ``activation`` naming the gate's ("silu" or "gelu_tanh").
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops


class Linear:
    def __init__(self, weight: torch.Tensor, bias: Optional[torch.Tensor], fast: bool = True,
                 gated: bool = False, activation: str = "silu"):
        if weight.dim() != 2:
            raise ValueError("a projection weight must be [out, in]")
        self.gated = gated
        self.activation = activation
        ops.gate_code(activation)             # an unknown name is refused when the part is built
        self.rows, self.n_in = weight.shape
        self.n_out = self.rows // 2 if gated else self.rows
        if gated and self.rows % 2:
            raise ValueError("a gated projection stacks two matrices of equal height")
        if bias is not None and bias.numel() != self.n_out:
            raise ValueError(f"bias has {bias.numel()} elements, the projection has {self.n_out} outputs")
        self.bias = None if bias is None else bias.contiguous()
        self.packed = None
        self.weight = weight.contiguous()
        if fast and weight.is_cuda and weight.dtype == torch.bfloat16 and self.n_in % 8 == 0:
            self.packed = ops.pack_weight(self.weight, gated)
            self.weight = None

    def _row_major(self) -> torch.Tensor:
        if self.weight is None:
            raise RuntimeError("this projection only keeps its packed weight")
        return self.weight

    def __call__(self, x: torch.Tensor, out_dtype: torch.dtype, resid: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.gated:
            return self.gated_product(x, out_dtype)
        if self.packed is not None:
            if x.dtype != torch.bfloat16:
                x = ops.cast(x, torch.bfloat16)
            return ops.gemm_bf16(x, self.packed, self.bias, resid, out_dtype, out,
                                 packed_shape=(self.rows, self.n_in))
        w = self._row_major()
        if w.dtype == torch.float32 and x.dtype != torch.float32:
            x = ops.cast(x, torch.float32)
        return ops.gemm_plain(x, w, self.bias, resid, out_dtype, out)

    def partial(self, x: torch.Tensor) -> Optional[torch.Tensor]:
        """The raw product in K slices, float32 [slices, rows, out] (bias and residual left to the
        consumer), when a kernel that cuts K over the grid takes this call (few rows, or a few
        hundred against a narrow matrix); else None."""
        if self.packed is None or self.gated or x.dtype != torch.bfloat16:
            return None
        return ops.gemm_bf16_partial(x, self.packed, packed_shape=(self.rows, self.n_in))

    def add_into(self, x: torch.Tensor, resid: torch.Tensor, then_norm=None, out_dtype=None):
        """resid += x W^T (+ b).  With ``then_norm`` (an RMS norm part) tries to return
        then_norm(resid) in ``out_dtype`` from the same pass; None when the caller has to norm."""
        part = self.partial(x)
        if part is not None and ops.reduce_resid_norm_ok(self.n_out):
            fuse = then_norm is not None and getattr(then_norm, "fusable", False)
            return ops.reduce_resid_norm(part, self.bias, resid, then_norm.weight if fuse else None,
                                         then_norm.eps if fuse else 0.0, out_dtype if fuse else None)
        self(x, torch.float32, resid=resid, out=resid)
        return None

    def gated_product(self, x: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
        """act(x Wg^T) * (x Wu^T): one fused kernel on the matrix cores, or the product in
        float32 followed by the activation kernel."""
        if self.packed is not None:
            if x.dtype != torch.bfloat16:
                x = ops.cast(x, torch.bfloat16)
            return ops.gemm_bf16(x, self.packed, None, None, out_dtype, gated=self.activation,
                                 packed_shape=(self.rows, self.n_in))
        w = self._row_major()
        if w.dtype == torch.float32 and x.dtype != torch.float32:
            x = ops.cast(x, torch.float32)
        return ops.gate_mul(ops.gemm_plain(x, w, None, None, torch.float32), out_dtype, self.activation)

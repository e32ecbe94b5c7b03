"""RMS norm (/root/reference/core/src/nn/norm.cpp:25-42)."""
from __future__ import annotations

from .. import ops
from .base import Part, register_part
from .spec import PartSpec, TensorSpec


def rmsnorm_spec(weight_name: str, width: int, eps: float) -> PartSpec:
    return PartSpec("norm", "rmsnorm", {"width": width, "eps": float(eps)},
                    {"weight": TensorSpec(weight_name, (width,), init=(1.0, 0.02))})


@register_part("norm", "rmsnorm")
class RMSNorm(Part):
    """y = (x * 1/sqrt(mean(x^2) + eps)) * w; the weight multiplies as it is."""
    category = "norm"
    fusable = True      # a projection's last pass may apply this norm (it exposes weight and eps)

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.width = int(spec.params["width"])
        self.eps = float(spec.params["eps"])
        self.weight = tensors.get("weight")

    def forward(self, x, out_dtype, rows=None):
        return ops.rmsnorm(x, self.weight, self.eps, out_dtype, rows)

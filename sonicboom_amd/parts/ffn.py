"""Gated dense feed-forward: y = W_down (act(W_gate f) * (W_up f)).

/root/reference/core/src/model/emit.cpp:364-374; the activation is a parameter
of the spec: "silu", g / (1 + exp(-g)) (/root/reference/core/src/nn/activation.cpp:41-50),
or "gelu_tanh", 0.5 g (1 + tanh(sqrt(2/pi) g (1 + 0.044715 g^2))) (:27-36); the product
kernels apply either in their epilogue.  The gate and up matrices
are stacked into one [2*inner, width] matrix when the part is built, so a
step runs one product for both; its float32 result feeds the activation
kernel, whose output is rounded once to the activation type.
"""
from __future__ import annotations

import torch

from .base import Part, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec

ACTIVATIONS = ("silu", "gelu_tanh")    # the gates the product kernels apply in their epilogue


def gated_ffn_spec(prefix: str, width: int, inner: int, activation: str = "silu") -> PartSpec:
    return PartSpec("ffn", "gated_dense", {"width": width, "inner": inner, "activation": activation}, {
        "gate_weight": TensorSpec(prefix + "gate_proj.weight", (inner, width)),
        "up_weight": TensorSpec(prefix + "up_proj.weight", (inner, width)),
        "down_weight": TensorSpec(prefix + "down_proj.weight", (width, inner)),
    })


@register_part("ffn", "gated_dense")
class GatedDenseFFN(Part):
    category = "ffn"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width, self.inner = int(p["width"]), int(p["inner"])
        self.activation = p.get("activation", "silu")
        if self.activation not in ACTIVATIONS:
            raise ValueError(f"unknown activation {self.activation!r}; known: {ACTIVATIONS}")
        g, u = tensors["gate_weight"], tensors["up_weight"]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        self.gate_up = Linear(torch.cat([g, u], dim=0), None, rt.fast_kernels, gated=True,
                              activation=self.activation)
        self.down = Linear(tensors["down_weight"], None, rt.fast_kernels)

    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only

    def forward(self, h, x, ctx, then_norm=None):
        """x += ffn(h).  Returns then_norm(x) when the down projection could apply the norm in
        its last pass, else None."""
        mid = self.gate_up.gated_product(h, self.rt.act_dtype)
        return self.down.add_into(mid, x, then_norm, self.rt.act_dtype)

"""Arrangement of norms, mixer and feed-forward in a block.

``prenorm`` (/root/reference/core/src/model/emit.cpp:436-459 without the
optional post-norms): x += mixer(norm(x)); x += ffn(norm(x)).  Mixer and
feed-forward add their result into the float32 residual stream themselves,
which lets their last projection fuse the addition.
"""
from __future__ import annotations

from .base import Part, register_part
from .spec import PartSpec


def prenorm_block_spec(mixer_norm: PartSpec, mixer: PartSpec, ffn_norm: PartSpec, ffn: PartSpec) -> PartSpec:
    return PartSpec("block", "prenorm", {}, {}, {
        "mixer_norm": mixer_norm, "mixer": mixer, "ffn_norm": ffn_norm, "ffn": ffn})


@register_part("block", "prenorm")
class PreNormBlock(Part):
    category = "block"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.mixer_norm = parts["mixer_norm"]
        self.mixer = parts["mixer"]
        self.ffn_norm = parts["ffn_norm"]
        self.ffn = parts["ffn"]

    def forward(self, x, ctx, binding) -> None:
        act = self.rt.act_dtype
        self.mixer.forward(self.mixer_norm.forward(x, act), x, ctx, binding)
        self.ffn.forward(self.ffn_norm.forward(x, act), x, ctx)

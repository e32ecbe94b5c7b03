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
        self.first_norm = self.mixer_norm      # what the block before may apply in its last pass
        self.mixer = parts["mixer"]
        self.ffn_norm = parts["ffn_norm"]
        self.ffn = parts["ffn"]

    def forward(self, x, ctx, binding, h=None, next_norm=None):
        """Run the block on the residual stream ``x`` in place.  ``h`` is mixer_norm(x) when the
        previous block has already computed it; ``next_norm`` is the norm the next block starts
        with.  Returns next_norm(x) when the feed-forward's last pass produced it, else None.
        Mixers and feed-forwards that can apply a norm in their last pass say so with
        ``fuses_norm``; the others are simply followed by the norm."""
        act = self.rt.act_dtype
        if h is None:
            h = self.mixer_norm.forward(x, act)
        f = None
        if getattr(self.mixer, "fuses_norm", False):
            f = self.mixer.forward(h, x, ctx, binding, then_norm=self.ffn_norm)
        else:
            self.mixer.forward(h, x, ctx, binding)
        trace = getattr(ctx, "trace", None)
        if trace is not None:
            trace("after_mixer", x)
        if f is None:
            f = self.ffn_norm.forward(x, act)
        out = None
        if getattr(self.ffn, "fuses_norm", False):
            out = self.ffn.forward(f, x, ctx, then_norm=next_norm)
        else:
            self.ffn.forward(f, x, ctx)
        if trace is not None:
            trace("after_ffn", x)
        return out

"""Token embedding and the output head.

Embedding: a row lookup into the float32 residual stream, no scale
(/root/reference/core/src/model/emit.cpp:237-248).  Head: logits = W h in
float32; the matrix is the embedding table when the spec says the model ties
them (/root/reference/core/src/model/exec.cpp:516-517).
"""
from __future__ import annotations

import torch

from .. import ops
from .base import Part, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec


def embedding_spec(name: str, vocab: int, width: int) -> PartSpec:
    return PartSpec("embedding", "lookup", {"vocab": vocab, "width": width},
                    {"table": TensorSpec(name, (vocab, width))})


def head_spec(name: str, vocab: int, width: int) -> PartSpec:
    """``name`` may be the embedding table's name: the head then shares it."""
    return PartSpec("head", "linear", {"vocab": vocab, "width": width},
                    {"weight": TensorSpec(name, (vocab, width))})


@register_part("embedding", "lookup")
class Embedding(Part):
    category = "embedding"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.table = tensors["table"]
        self.vocab, self.width = self.table.shape

    def forward(self, ids: torch.Tensor, ctx=None) -> torch.Tensor:
        """``ctx``: the step's context, for embeddings that look at more than the ids (the
        rows' positions, say); this one does not."""
        return ops.embed(self.table, ids)


@register_part("head", "linear")
class LinearHead(Part):
    category = "head"

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        self.proj = Linear(tensors["weight"], None, rt.fast_kernels)
        self.vocab = int(spec.params["vocab"])

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return self.proj(h, torch.float32)

"""Interfaces of the parts a model is assembled from, and their registry.

A part is built from its :class:`~sonicboom_amd.parts.spec.PartSpec`, the
tensors the spec names and a :class:`Runtime`.  It knows its own sizes and
constants and nothing about the model it sits in.  Parts of the same category
are interchangeable: the engine only uses the interface of the category.

Interfaces (``x`` is the float32 residual stream [rows, width], ``h`` a normed
copy in the activation type, ``ctx`` the step's
:class:`~sonicboom_amd.engine.step.StepContext`):

* **norm**      ``forward(x, out_dtype, rows=None) -> tensor``
* **position**  ``rotary_tables() -> (inv_freq, freq_factors, rot_dims) | None``
                and, for encodings that are not rotary, ``apply(qkv, ctx, heads_q,
                heads_kv, head_dim)`` acting in place on float32 qkv rows;
                ``score_scale`` multiplies the attention scale.
* **mixer**     ``cache_spec() -> KVSpec | RowsSpec | None``, ``state_spec() -> StateSpec | None``,
                ``forward(h, x, ctx, binding)`` adds the mixer's output into ``x``.
* **ffn**       ``forward(h, x, ctx)`` adds the feed-forward's output into ``x``.
                Mixers and feed-forwards may set ``fuses_norm`` (their ``forward`` then
                takes ``then_norm=`` and may return the normed stream) and ``graph_safe``
                (their launches depend on device buffers only, so a decode step may be
                recorded once and replayed).
* **block**     ``mixer`` attribute and ``forward(x, ctx, binding, h=None, next_norm=None)``;
                optionally ``first_norm``, the norm the block starts with (the block before
                may then hand over ``h`` = first_norm(x) from its last pass), and calls of
                ``ctx.trace(name, x)`` after its mixer and feed-forward when that is set.
* **embedding** ``forward(ids, ctx) -> x`` (``ctx.row_pos`` for embeddings that add a position's row)
* **head**      ``forward(h) -> float32 logits [rows, vocab]``
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Dict, Optional, Tuple

import torch

from .spec import PartSpec

CATEGORIES = ("norm", "position", "mixer", "ffn", "block", "embedding", "head")


@dataclass(frozen=True)
class Runtime:
    """Where and in which precision parts run.  ``act_dtype`` is the type of
    normed activations, queries and the cache: float32 for the 32-bit path,
    bfloat16 for serving.  The residual stream is float32 in both."""
    device: torch.device
    act_dtype: torch.dtype
    fast_kernels: bool = True     # MFMA kernels where sizes allow (bfloat16 only)

    @property
    def cache_dtype(self) -> torch.dtype:
        return self.act_dtype


@dataclass(frozen=True)
class KVSpec:
    """What a mixer keeps per token: keys and values of ``kv_heads`` heads of
    ``head_dim``; ``window`` > 0 when only the last ``window`` keys are read."""
    kv_heads: int
    head_dim: int
    window: int = 0

    def key(self):
        return (int(self.kv_heads), int(self.head_dim), int(self.window))


@dataclass(frozen=True)
class RowsSpec:
    """What a mixer keeps per token when that is not keys and values of heads: one row of
    ``shape`` (a compressed key-value vector, say) in the cache's dtype, paged like keys;
    ``window`` > 0 when only the last ``window`` rows are read.  The mixer's binding then
    carries the rows as ``k_cache`` [pages, PAGE, *shape] and no ``v_cache``."""
    shape: Tuple[int, ...]
    window: int = 0

    def key(self):
        return ("rows", tuple(int(n) for n in self.shape), int(self.window))


@dataclass(frozen=True)
class StateSpec:
    """Per-sequence state of fixed size (zeroed when a slot is handed out)."""
    shape: Tuple[int, ...]
    dtype: torch.dtype = torch.float32


class Part:
    category = ""

    def __init__(self, spec: PartSpec, tensors: Dict[str, Optional[torch.Tensor]],
                 parts: Dict[str, "Part"], rt: Runtime):
        self.spec = spec
        self.rt = rt


class Mixer(Part):
    category = "mixer"

    def cache_spec(self) -> "Optional[KVSpec | RowsSpec]":
        return None

    def state_spec(self) -> Optional[StateSpec]:
        return None

    def forward(self, h, x, ctx, binding) -> None:
        raise NotImplementedError


_REGISTRY: Dict[Tuple[str, str], Callable] = {}


def register_part(category: str, kind: str):
    """Class decorator: make ``kind`` available to specs of ``category``."""
    if category not in CATEGORIES:
        raise ValueError(f"unknown part category {category!r}; categories are {CATEGORIES}")

    def deco(cls):
        _REGISTRY[(category, kind)] = cls
        return cls
    return deco


def registered_parts():
    return sorted(_REGISTRY)


def build_part(spec: PartSpec, tensors: Dict[str, torch.Tensor], rt: Runtime) -> Part:
    """Instantiate ``spec`` (nested parts first) with tensors looked up by name."""
    try:
        cls = _REGISTRY[(spec.category, spec.kind)]
    except KeyError:
        kinds = [k for c, k in _REGISTRY if c == spec.category]
        raise KeyError(f"no {spec.category} part of kind {spec.kind!r}; registered: {sorted(kinds)}") from None
    nested = {role: build_part(p, tensors, rt) for role, p in spec.parts.items()}
    own = {role: tensors.get(t.name) for role, t in spec.tensors.items()}
    return cls(spec, own, nested, rt)

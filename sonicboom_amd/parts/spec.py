"""Descriptions of a model as data.

An architecture turns its typed configuration into a :class:`ModelSpec`: a
tree of :class:`PartSpec` (kind, constants, tensors) for the embedding, every
block and the head, plus the order in which blocks run.  Nothing in a spec
touches a GPU, so specs are built and checked on any machine.  The engine
instantiates each spec through the part registry; the weight loader reads the
tensors a spec names.  This is the recipe idea of the reference
(/root/reference/core/include/sonicboom/model/recipe.h:51-205): layer kinds as
values that carry their own sizes and constants.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple


@dataclass(frozen=True)
class TensorSpec:
    """One tensor of the model file.

    ``kind`` is "float" (kept in bfloat16, or in float32 when stored so or when
    the whole model runs in 32-bit) or "int" (kept as int32).  ``init`` is
    (mean, std) of the seeded random mode.  An ``optional`` tensor may be
    absent from the file; the part then receives None.
    """
    name: str
    shape: Tuple[int, ...]
    kind: str = "float"
    optional: bool = False
    init: Tuple[float, float] = (0.0, 0.02)


@dataclass
class PartSpec:
    """A part: its category ("mixer", "ffn", "norm", "position", "block",
    "embedding", "head"), its kind within the category, its constants, the
    tensors it owns by role, and the parts nested in it by role."""
    category: str
    kind: str
    params: Dict[str, object] = field(default_factory=dict)
    tensors: Dict[str, TensorSpec] = field(default_factory=dict)
    parts: Dict[str, "PartSpec"] = field(default_factory=dict)

    def all_tensors(self) -> List[TensorSpec]:
        out = list(self.tensors.values())
        for p in self.parts.values():
            out += p.all_tensors()
        return out


@dataclass(frozen=True)
class OrderEntry:
    """One execution of a block.

    ``block`` indexes ``ModelSpec.blocks`` (the same block may be named by
    several entries).  ``cache`` names the cache entry the mixer uses: entries
    with the same number share keys and values; the one with ``writes_cache``
    stores them, the others only read.  ``None`` means the mixer keeps nothing
    per token.  Per-sequence state of fixed size belongs to the entry itself.
    """
    block: int
    cache: Optional[int] = None
    writes_cache: bool = True


@dataclass
class ModelSpec:
    architecture: str
    width: int
    vocab: int
    embedding: PartSpec
    blocks: List[PartSpec]
    order: List[OrderEntry]
    final_norm: PartSpec
    head: PartSpec
    max_positions: int = 0                    # 0 = not bounded by the model
    stop_tokens: Tuple[int, ...] = ()
    # Names that may be in the file without being used (a tied head's copy).
    ignorable_tensors: Tuple[str, ...] = ()

    def all_tensors(self) -> List[TensorSpec]:
        seen, out = set(), []
        parts = [self.embedding, *self.blocks, self.final_norm, self.head]
        for p in parts:
            for t in p.all_tensors():
                if t.name not in seen:
                    seen.add(t.name)
                    out.append(t)
        return out

    def validate(self) -> None:
        caches_written = {}
        for i, e in enumerate(self.order):
            if not 0 <= e.block < len(self.blocks):
                raise ValueError(f"order entry {i} names block {e.block}, the model has {len(self.blocks)}")
            if e.cache is not None and e.writes_cache:
                if e.cache in caches_written:
                    raise ValueError(
                        f"order entries {caches_written[e.cache]} and {i} both write cache {e.cache}")
                caches_written[e.cache] = i
        for i, e in enumerate(self.order):
            if e.cache is not None and not e.writes_cache:
                w = caches_written.get(e.cache)
                if w is None or w > i:
                    raise ValueError(f"order entry {i} reads cache {e.cache} before any entry has written it")

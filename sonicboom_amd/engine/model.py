"""A decoder built from a model spec: embedding, blocks in their run order, final norm, head."""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Optional

import torch

from ..cache.paged import GroupSpec, PagedCache, group_entries
from ..config.registry import architecture_of, load_config
from ..parts import ModelSpec, Runtime, build_part
from ..weights import open_tensors, random_source

DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def require_gpu(device=None) -> torch.device:
    """The HIP device to run on; there is no CPU path."""
    if not torch.cuda.is_available():
        raise RuntimeError("sonicboom_amd needs a HIP GPU (gfx950): torch reports none, and there is no CPU path")
    return torch.device(device or "cuda:0")


@dataclass
class LayerBinding:
    """What one order entry's mixer is handed in a step."""
    entry: int                       # index in the run order
    group: Optional[int]             # cache group (None: the mixer keeps no keys)
    k_cache: Optional[torch.Tensor]
    v_cache: Optional[torch.Tensor]
    writes_cache: bool
    state: Optional[torch.Tensor]    # [max_slots, *shape] or None


class DecoderModel:
    def __init__(self, spec: ModelSpec, tensors: Dict[str, torch.Tensor], rt: Runtime, config=None):
        spec.validate()
        self.spec, self.rt, self.config = spec, rt, config
        self.width, self.vocab = spec.width, spec.vocab
        self.embedding = build_part(spec.embedding, tensors, rt)
        self.head = build_part(spec.head, tensors, rt)
        self.final_norm = build_part(spec.final_norm, tensors, rt)
        shared = {t.name for t in spec.embedding.all_tensors() + spec.head.all_tensors()
                  + spec.final_norm.all_tensors()}
        self.blocks = []
        for b in spec.blocks:
            self.blocks.append(build_part(b, tensors, rt))
            for t in b.all_tensors():          # the block has packed what it needs
                if t.name not in shared:
                    tensors.pop(t.name, None)
        self.order = list(spec.order)
        for e in self.order:
            mixer = self.blocks[e.block].mixer
            if e.cache is not None and not e.writes_cache and hasattr(mixer, "query_only"):
                mixer.query_only()
        for b in self.blocks:
            if hasattr(b.mixer, "finish_build"):
                b.mixer.finish_build()
        # heights of the runs of rows that the mixers' kernels take together (a mixer says so with
        # a row_tile attribute: a height, or several); a step's context describes its rows in runs
        # of each of them
        heights = set()
        for b in self.blocks:
            asked = getattr(b.mixer, "row_tile", 0) or ()
            heights.update((int(asked),) if isinstance(asked, int) else (int(h) for h in asked))
        self.row_tiles = sorted(heights)
        # What every cache entry stores, and which order entries want per-sequence state.
        self.cache_specs: Dict[int, tuple] = {}
        self.state_specs: Dict[int, tuple] = {}
        for i, e in enumerate(self.order):
            mixer = self.blocks[e.block].mixer
            if e.cache is not None:
                cs = mixer.cache_spec()
                if cs is None:
                    raise ValueError(f"order entry {i} names cache {e.cache} but its mixer keeps no keys")
                need = cs.key()          # (kv heads, head size, window), or ("rows", shape, window)
                if e.writes_cache:
                    self.cache_specs[e.cache] = need
                elif self.cache_specs.get(e.cache, need)[:2] != need[:2]:
                    raise ValueError(f"order entry {i} reads cache {e.cache} whose heads (or rows) differ from its own")
            ss = mixer.state_spec()
            if ss is not None:
                self.state_specs[i] = (tuple(ss.shape), ss.dtype)
        self.groups: List[GroupSpec] = group_entries(self.cache_specs)

    # ---- construction --------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, dtype: str = "bfloat16", device=None, fast_kernels: bool = True):
        """The model of a folder with config.json and model.safetensors; its class is chosen by config.json."""
        arch, cfg = load_config(folder)          # configuration errors first: they need no GPU
        spec = arch.build_spec(cfg)
        dev = require_gpu(device)
        tensors = open_tensors(folder, spec, dtype, dev)      # read as the parts ask for them
        try:
            return cls(spec, tensors, Runtime(dev, DTYPES[dtype], fast_kernels), cfg)
        finally:
            tensors.close()

    @classmethod
    def from_random(cls, config, seed: int, dtype: str = "bfloat16", device=None, fast_kernels: bool = True,
                    stored: Optional[str] = None):
        """Random weights drawn on the device, for a typed configuration or a config.json dict: the
        model that a folder written by ``write_random_model(folder, config, seed, stored or dtype)``
        gives when it is loaded as ``dtype``, to the bit."""
        d = config if isinstance(config, dict) else config.to_dict()
        arch = architecture_of(d)
        cfg = arch.config_class.from_dict(d)
        spec = arch.build_spec(cfg)
        dev = require_gpu(device)
        tensors = random_source(spec, seed, dtype, dev, stored)       # drawn as the parts ask for them
        return cls(spec, tensors, Runtime(dev, DTYPES[dtype], fast_kernels), cfg)

    # ---- cache -----------------------------------------------------------------
    def new_cache(self, max_tokens: int, max_slots: Optional[int] = None, step_rows: int = 0) -> PagedCache:
        return PagedCache(self.groups, max_tokens, self.rt.cache_dtype, self.rt.device,
                          self.state_specs, max_slots, step_rows=step_rows)

    def bindings(self, cache: PagedCache) -> List[LayerBinding]:
        out = []
        for i, e in enumerate(self.order):
            k = v = g = None
            if e.cache is not None:
                k, v, g = cache.entry_views(e.cache)
            out.append(LayerBinding(i, g, k, v, e.writes_cache and e.cache is not None, cache.state.get(i)))
        return out

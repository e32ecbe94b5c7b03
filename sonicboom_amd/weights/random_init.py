"""Seeded random weights.

``write_random_model`` makes a model folder (config.json, model.safetensors)
from a configuration and a seed; ``random_tensors`` makes the same kind of
weights straight on a device, for sizes too large to route through a file.
Each tensor is drawn as mean + std * N(0,1) with the (mean, std) of its
:class:`~sonicboom_amd.parts.spec.TensorSpec`: projections and biases
N(0, 0.02), norm weights 1 + N(0, 0.02).  In a folder, tensor number i of the
spec comes from a Philox generator keyed by (seed, i), so the file does not
depend on the order or the machine that wrote it.
"""
from __future__ import annotations

import json
import os
from typing import Dict

import numpy as np
import torch

from ..config.registry import architecture_of
from ..parts.spec import ModelSpec
from .safetensors_io import f32_to_bf16_bits, write_safetensors


def _draw(seed: int, index: int, shape, mean: float, std: float) -> np.ndarray:
    gen = np.random.Generator(np.random.Philox(key=[int(seed) & (2**64 - 1), index]))
    a = gen.standard_normal(size=shape, dtype=np.float32)
    return (a * np.float32(std) + np.float32(mean)).astype(np.float32)


def random_arrays(spec: ModelSpec, seed: int) -> Dict[str, np.ndarray]:
    """float32 arrays (int32 zeros for integer tables) for every tensor of the spec."""
    out = {}
    for i, t in enumerate(spec.all_tensors()):
        if t.kind == "int":
            out[t.name] = np.zeros(t.shape, dtype=np.int32)
        else:
            out[t.name] = _draw(seed, i, t.shape, *t.init)
    return out


def write_random_model(folder: str, config, seed: int, dtype: str = "bfloat16",
                       float32_tensors=()) -> ModelSpec:
    """Write ``config.json`` and ``model.safetensors`` for a typed configuration
    (or a config.json dict).  ``dtype`` is the stored type of floating tensors;
    names in ``float32_tensors`` are stored in float32 regardless."""
    if dtype not in ("bfloat16", "float32"):
        raise ValueError("stored dtype must be bfloat16 or float32")
    d = config if isinstance(config, dict) else config.to_dict()
    arch = architecture_of(d)
    cfg = arch.config_class.from_dict(d)
    spec = arch.build_spec(cfg)
    os.makedirs(folder, exist_ok=True)
    d = dict(d)
    d["torch_dtype"] = dtype
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(d, f, indent=2, sort_keys=True)

    def entries():
        for name, a in random_arrays(spec, seed).items():
            if a.dtype == np.int32:
                yield name, "I32", a
            elif dtype == "float32" or name in float32_tensors:
                yield name, "F32", a
            else:
                yield name, "BF16", f32_to_bf16_bits(a)
    write_safetensors(os.path.join(folder, "model.safetensors"), entries(),
                      metadata={"format": "pt", "seed": seed})
    return spec


def random_source(spec: ModelSpec, seed: int, dtype: str, device):
    """The spec's tensors drawn on ``device`` as they are asked for (a model of 145 GB is then
    built block by block without its row-major weights ever standing whole beside the packed
    ones).  Tensor number i of the spec comes from torch's generator seeded by (seed, i): the
    values do not depend on the order of asking.  Another stream of numbers than the folder
    writer's, the same distributions."""
    from .loader import LazyTensors
    tdt = torch.float32 if dtype == "float32" else torch.bfloat16
    specs = {t.name: (i, t) for i, t in enumerate(spec.all_tensors())}

    def make(name):
        i, t = specs[name]
        if t.kind == "int":
            return torch.zeros(t.shape, dtype=torch.int32, device=device)
        gen = torch.Generator(device=device)
        gen.manual_seed((int(seed) * 1000003 + i) & (2**63 - 1))
        mean, std = t.init
        a = torch.empty(t.shape, dtype=torch.float32, device=device)
        a.normal_(mean, std, generator=gen)
        return a.to(tdt)
    return LazyTensors(specs, make)


def random_tensors(spec: ModelSpec, seed: int, dtype: str, device) -> Dict[str, torch.Tensor]:
    """All of :func:`random_source` at once, as a dict."""
    return random_source(spec, seed, dtype, device).materialize()

"""Seeded random weights.

``write_random_model`` makes a model folder (config.json, model.safetensors)
from a configuration and a seed; ``random_source`` draws the same weights
straight on a device, for sizes too large to route through a file.
Each tensor is drawn as mean + std * N(0,1) with the (mean, std) of its
:class:`~sonicboom_amd.parts.spec.TensorSpec`: projections and biases
N(0, 0.02), norm weights 1 + N(0, 0.02).  Element e of tensor number i of the
spec is a function of (seed, i, e) alone (:mod:`.random_stream`: Philox4x32-10
keyed by the seed, Box and Muller), computed to the same bits by NumPy here and
by the kernel ``sb_random_normal`` on the GPU: a folder written from (config,
seed, dtype) and a model drawn on the device from the same three are the same
model, whatever the order, the machine or the side that drew it.
"""
from __future__ import annotations

import json
import os
from typing import Dict

import numpy as np
import torch

from ..config.registry import architecture_of
from ..parts.spec import ModelSpec
from . import random_stream
from .safetensors_io import f32_to_bf16_bits, write_safetensors


# tensors of at least this many elements are drawn by the GPU's kernel when a folder is written
# on a machine that has one (same bits, a few hundred times faster than NumPy)
DEVICE_DRAW_FROM = 1 << 22


def _draw(seed: int, index: int, shape, mean: float, std: float, device=None) -> np.ndarray:
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    if device is not None and n >= DEVICE_DRAW_FROM:
        from .. import ops
        return ops.random_normal(shape, seed, index, mean, std, torch.float32, device).cpu().numpy()
    return random_stream.draw(seed, index, shape, mean, std)


def random_arrays(spec: ModelSpec, seed: int, device=None) -> Dict[str, np.ndarray]:
    """float32 arrays (int32 zeros for integer tables) for every tensor of the spec."""
    return dict(iter_random_arrays(spec, seed, device))


def iter_random_arrays(spec: ModelSpec, seed: int, device=None):
    """(name, array) for every tensor of the spec, one at a time: float32 arrays, int32 zeros for
    integer tables.  ``device``: a GPU that draws the large tensors (same bits as the host)."""
    for i, t in enumerate(spec.all_tensors()):
        if t.kind == "int":
            yield t.name, np.zeros(t.shape, dtype=np.int32)
        else:
            yield t.name, _draw(seed, i, t.shape, *t.init, device=device)


def write_random_model(folder: str, config, seed: int, dtype: str = "bfloat16",
                       float32_tensors=(), device="auto") -> ModelSpec:
    """Write ``config.json`` and ``model.safetensors`` for a typed configuration
    (or a config.json dict).  ``dtype`` is the stored type of floating tensors;
    names in ``float32_tensors`` are stored in float32 regardless.  ``device``: the GPU that
    draws the large tensors ("auto": the first one if there is one; None: the host draws all);
    the file is the same either way."""
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

    if device == "auto":
        device = "cuda:0" if torch.cuda.is_available() else None

    def entries():
        for name, a in iter_random_arrays(spec, seed, device):
            if a.dtype == np.int32:
                yield name, "I32", a
            elif dtype == "float32" or name in float32_tensors:
                yield name, "F32", a
            else:
                yield name, "BF16", f32_to_bf16_bits(a)
    write_safetensors(os.path.join(folder, "model.safetensors"), entries(),
                      metadata={"format": "pt", "seed": seed})
    return spec


def random_source(spec: ModelSpec, seed: int, dtype: str, device, stored=None):
    """The spec's tensors drawn on ``device`` as they are asked for (a model of 145 GB is then
    built block by block without its row-major weights ever standing whole beside the packed
    ones).  Tensor number i of the spec is drawn by ``sb_random_normal`` under (seed, i): the
    values do not depend on the order of asking, and they are the bits that
    :func:`write_random_model` stores for the same (configuration, seed, dtype).  ``stored``
    (default: ``dtype``) is the type such a folder would be stored in: "bfloat16" with a ``dtype``
    of "float32" gives the float32 model of a bfloat16 folder."""
    from .. import ops
    from .loader import LazyTensors
    out_dt = torch.float32 if dtype == "float32" else torch.bfloat16
    tdt = out_dt if stored is None else (torch.float32 if stored == "float32" else torch.bfloat16)
    specs = {t.name: (i, t) for i, t in enumerate(spec.all_tensors())}

    def make(name):
        i, t = specs[name]
        if t.kind == "int":
            return torch.zeros(t.shape, dtype=torch.int32, device=device)
        mean, std = t.init
        if torch.device(device).type == "cpu":          # the host's own function: the same bits
            return torch.from_numpy(random_stream.draw(seed, i, t.shape, mean, std)).to(tdt).to(out_dt)
        return ops.random_normal(t.shape, seed, i, mean, std, tdt, device).to(out_dt)
    return LazyTensors(specs, make)


def random_tensors(spec: ModelSpec, seed: int, dtype: str, device, stored=None) -> Dict[str, torch.Tensor]:
    """All of :func:`random_source` at once, as a dict."""
    return random_source(spec, seed, dtype, device, stored).materialize()

"""Weights from a model folder, by tensor name.

The folder holds ``model.safetensors``, or several shards named by
``model.safetensors.index.json``'s ``weight_map``.  Every tensor the model
spec names is looked up by name and its shape checked; every problem of the
whole file set is collected and reported in ONE error, one line each — missing
tensors, unexpected tensors, wrong shapes, wrong kinds — as the reference's
binder accumulates its messages (/root/reference/core/src/model/loader.cpp:325-408,
:875-947).

Types: floating tensors are kept in bfloat16; a tensor the file stores in 32
bits (or 64) stays float32; integer tables become int32.  With
``dtype="float32"`` every floating tensor is widened to float32.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List

import numpy as np
import torch

from ..parts.spec import ModelSpec, TensorSpec
from .safetensors_io import SafetensorsError, SafetensorsFile, bf16_bits_to_f32

SINGLE = "model.safetensors"
INDEX = "model.safetensors.index.json"
_FLOAT = ("F64", "F32", "F16", "BF16")
_INT = ("I64", "I32", "I16", "I8", "U8", "BOOL")


class WeightError(ValueError):
    """The files of a model folder do not hold the tensors the model needs."""


def open_files(folder: str) -> Dict[str, SafetensorsFile]:
    """tensor name -> open file that holds it."""
    single, index = os.path.join(folder, SINGLE), os.path.join(folder, INDEX)
    files: Dict[str, SafetensorsFile] = {}
    owner: Dict[str, SafetensorsFile] = {}
    try:
        if os.path.exists(index):
            with open(index) as f:
                weight_map = json.load(f).get("weight_map")
            if not isinstance(weight_map, dict):
                raise WeightError(f"format: {index} has no weight_map object")
            for name, shard in weight_map.items():
                if shard not in files:
                    files[shard] = SafetensorsFile(os.path.join(folder, shard))
                owner[name] = files[shard]
            for shard, sf in files.items():
                for name in sf.tensors:
                    owner.setdefault(name, sf)
        elif os.path.exists(single):
            sf = SafetensorsFile(single)
            files[SINGLE] = sf
            owner = {name: sf for name in sf.tensors}
        else:
            raise WeightError(f"io: {folder} holds neither {SINGLE} nor {INDEX}")
    except (SafetensorsError, json.JSONDecodeError) as e:
        for sf in files.values():
            sf.close()
        raise WeightError(str(e)) from None
    return owner


def check_against_spec(found: Dict[str, tuple], wanted: List[TensorSpec], ignorable=()) -> List[str]:
    """Problems of a file set, one line each.  ``found`` maps name -> (dtype name, shape)."""
    problems = []
    names = {t.name for t in wanted}
    for t in wanted:
        if t.name not in found:
            if not t.optional:
                problems.append(f"missing tensor: {t.name} (the model wants shape {list(t.shape)})")
            continue
        dtype, shape = found[t.name]
        if tuple(shape) != tuple(t.shape):
            problems.append(f"tensor shape mismatch: {t.name} (the file has {list(shape)} {dtype}, "
                            f"the model wants {list(t.shape)})")
        elif (t.kind == "float" and dtype not in _FLOAT) or (t.kind == "int" and dtype not in _INT):
            problems.append(f"tensor type mismatch: {t.name} (the file has {dtype}, the model wants "
                            f"{'a floating' if t.kind == 'float' else 'an integer'} type)")
    for name in sorted(found):
        if name not in names and name not in ignorable:
            problems.append(f"unexpected tensor: {name} (shape {list(found[name][1])})")
    return problems


def _to_torch(raw: np.ndarray, file_dtype: str, kind: str, mode: str) -> torch.Tensor:
    if kind == "int":
        return torch.from_numpy(raw.astype(np.int32))
    if file_dtype in ("F64", "F32"):
        return torch.from_numpy(raw.astype(np.float32, copy=False))
    if file_dtype == "BF16":
        if mode == "float32":
            return torch.from_numpy(bf16_bits_to_f32(raw))
        return torch.from_numpy(raw.view(np.int16)).view(torch.bfloat16)
    # F16
    t = torch.from_numpy(raw.astype(np.float32))
    return t if mode == "float32" else t.to(torch.bfloat16)


class LazyTensors:
    """name -> tensor, made when it is first asked for and kept until it is popped.

    A model is built part by part; each part packs its tensors into the layout its kernels read
    and the model pops the originals.  Making a tensor only when its part asks for it keeps one
    part's worth of originals alive at a time, on the host and on the device, whatever the
    model's size.  ``get``, ``pop``, ``in`` and ``keys`` are what the builders use of a dict."""

    def __init__(self, names, make, close=None):
        self._names = set(names)
        self._make = make
        self._close = close
        self._kept: Dict[str, torch.Tensor] = {}

    def get(self, name, default=None):
        if name in self._kept:
            return self._kept[name]
        if name not in self._names:
            return default
        t = self._kept[name] = self._make(name)
        return t

    def __getitem__(self, name):
        t = self.get(name)
        if t is None:
            raise KeyError(name)
        return t

    def __contains__(self, name):
        return name in self._names

    def pop(self, name, default=None):
        self._names.discard(name)
        return self._kept.pop(name, default)

    def keys(self):
        return sorted(self._names)

    def materialize(self) -> Dict[str, torch.Tensor]:
        return {name: self.get(name) for name in self.keys()}

    def close(self) -> None:
        if self._close is not None:
            self._close()
            self._close = None
        self._names = set(self._kept)


def open_tensors(folder: str, spec: ModelSpec, dtype: str, device) -> LazyTensors:
    """The tensors ``spec`` names, read from the folder's files one by one as they are asked for
    and put on ``device``.  Everything is checked first: raises :class:`WeightError` listing every
    missing, unexpected, ill-shaped and ill-typed tensor.  ``close()`` the result when the model
    is built."""
    if dtype not in ("float32", "bfloat16"):
        raise ValueError(f"dtype must be float32 or bfloat16, not {dtype}")
    owner = open_files(folder)

    def close():
        for sf in set(owner.values()):
            sf.close()
    try:
        wanted = {t.name: t for t in spec.all_tensors()}
        found = {name: (sf.tensors[name].dtype, sf.tensors[name].shape) for name, sf in owner.items()}
        problems = check_against_spec(found, list(wanted.values()), spec.ignorable_tensors)
        if problems:
            raise WeightError(f"{folder}: {len(problems)} problem(s) with the weights\n" + "\n".join(problems))
    except BaseException:
        close()
        raise

    def make(name):
        sf, t = owner[name], wanted[name]
        return _to_torch(sf.raw(name), sf.tensors[name].dtype, t.kind, dtype).to(device)
    return LazyTensors([n for n in wanted if n in owner], make, close)


def load_tensors(folder: str, spec: ModelSpec, dtype: str, device) -> Dict[str, torch.Tensor]:
    """All tensors ``spec`` names, on ``device``; raises :class:`WeightError`
    listing every missing, unexpected and ill-shaped tensor."""
    source = open_tensors(folder, spec, dtype, device)
    try:
        return source.materialize()
    finally:
        source.close()

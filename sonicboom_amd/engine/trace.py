"""Dumps of a step's named intermediates, as text, and their comparison.

The format is the reference's (/root/reference/tools/baseline/sonicboom_dump.cpp:36-43,
/root/reference/tools/baseline/compare_dumps.cpp:5-19)::

    # <comment>
    @ <name> f32 <d0> <d1> <d2> <d3>
    <value>            (%.9g, one per line, d0*d1*d2*d3 of them)

A step's dump holds, in the order of the computation: ``embedding``, for every entry of the
run order ``entry<i>.after_mixer`` and ``entry<i>.after_ffn`` (the float32 residual stream of the
step's rows, [rows, width] flattened row by row), and ``logits`` of the wanted rows.  Two dumps
of the same step are compared name by name in that order, which points at the first layer where
two runs part (:func:`compare`; relative error ``|a-b| / max(|a|, |b|, 1e-12)``).
"""
from __future__ import annotations

import math
from typing import Dict, List, Tuple

import numpy as np


class DumpWriter:
    """``writer(name, tensor)`` appends one named tensor to a dump file."""

    def __init__(self, path: str, comment: str = ""):
        self._f = open(path, "w")
        if comment:
            self._f.write(f"# {comment}\n")

    def __call__(self, name: str, tensor) -> None:
        a = tensor.detach().float().cpu().numpy() if hasattr(tensor, "detach") else np.asarray(tensor, np.float32)
        a = np.ascontiguousarray(a, dtype=np.float32).reshape(-1)
        self._f.write(f"@ {name} f32 {a.size} 1 1 1\n")
        if a.size:
            self._f.write("\n".join("%.9g" % v for v in a.tolist()))
            self._f.write("\n")

    def close(self) -> None:
        self._f.close()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()


def read_dump(path: str) -> List[Tuple[str, np.ndarray]]:
    """[(name, float32 values)] in file order.  A name may hold spaces: the last five fields of
    a header are the type and four sizes."""
    out: List[Tuple[str, np.ndarray]] = []
    name, want, vals = None, 0, []
    with open(path) as f:
        for line in f:
            if not line.strip() or line[0] == "#":
                continue
            if line[0] == "@":
                if name is not None:
                    out.append((name, _finish(vals, want, name, path)))
                fields = line[1:].split()
                if len(fields) < 6:
                    raise ValueError(f"{path}: bad header: {line.strip()}")
                name = " ".join(fields[:-5])
                want = int(np.prod([int(d) for d in fields[-4:]]))
                vals = []
            elif name is not None:
                vals.append(line)
    if name is not None:
        out.append((name, _finish(vals, want, name, path)))
    return out


def _finish(lines, want, name, path) -> np.ndarray:
    a = np.array([float(v) for v in lines], dtype=np.float32)
    if a.size != want:
        raise ValueError(f"{path}: tensor {name} announces {want} values and holds {a.size}")
    return a


def compare(ref: List[Tuple[str, np.ndarray]], cand: List[Tuple[str, np.ndarray]], tol: float = 1e-4):
    """Per name of ``ref`` (in its order; the k-th occurrence of a name matches the k-th of the
    other dump): rows of (name, values, largest absolute error, largest relative error, root
    mean square error, within tolerance).  Returns (rows, first name out of tolerance or None,
    names only in ref, names only in cand)."""
    by_name: Dict[str, List[np.ndarray]] = {}
    for n, a in cand:
        by_name.setdefault(n, []).append(a)
    seen: Dict[str, int] = {}
    rows, first_bad, only_ref = [], None, []
    for n, a in ref:
        k = seen.get(n, 0)
        seen[n] = k + 1
        if n not in by_name or k >= len(by_name[n]):
            only_ref.append(n)
            continue
        b = by_name[n][k]
        if a.size != b.size:
            rows.append((n, a.size, math.inf, math.inf, math.inf, False))
            first_bad = first_bad or n
            continue
        a64, b64 = a.astype(np.float64), b.astype(np.float64)
        diff = np.abs(a64 - b64)
        rel = diff / np.maximum(np.maximum(np.abs(a64), np.abs(b64)), 1e-12)
        bad_values = ~(np.isfinite(a64) & np.isfinite(b64))
        max_abs = float(diff[~bad_values].max()) if (~bad_values).any() else 0.0
        max_rel = float(rel[~bad_values].max()) if (~bad_values).any() else 0.0
        rms = float(np.sqrt((diff[~bad_values] ** 2).mean())) if (~bad_values).any() else 0.0
        # within tolerance: every value close in relative or in absolute terms
        ok = not bad_values.any() and bool((np.minimum(rel, diff) <= tol).all())
        rows.append((n, a.size, max_abs, max_rel, rms, ok))
        if not ok and first_bad is None:
            first_bad = n
    only_cand = [n for n in by_name if n not in seen]
    return rows, first_bad, only_ref, only_cand

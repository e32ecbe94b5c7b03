"""Position encodings a mixer can be given.

``rope``: rotate-half (NEOX) rotary encoding,
/root/reference/core/src/nn/rope.cpp:26-83.  Its constants — base, rotated
width, per-pair divisors of long-context scaling, the multiplier of the
attention scale — are parameters; the per-pair factor
``expf(-2 i / n * logf(base))`` is computed here in float32 exactly as the
reference writes it and handed to the kernel as a table.

``none``: no encoding.
"""
from __future__ import annotations

import math
from typing import Optional, Sequence

import numpy as np
import torch

from .base import Part, register_part
from .spec import PartSpec


def rope_spec(head_dim: int, base: float, rot_dims: int = 0,
              freq_factors: Optional[Sequence[float]] = None, score_scale: float = 1.0) -> PartSpec:
    return PartSpec("position", "rope", {
        "head_dim": head_dim, "base": float(base), "rot_dims": int(rot_dims),
        "freq_factors": None if freq_factors is None else [float(f) for f in freq_factors],
        "score_scale": float(score_scale)})


def scaled_rope_tables(kind: str, factor: float, head_dim: int, base: float, original_ctx: int,
                       beta_fast: float = 32.0, beta_slow: float = 1.0, attention_factor: float = 1.0,
                       rot_dims: int = 0):
    """Per-pair angle divisors and the score multiplier of linear / YaRN scaling.

    /root/reference/core/src/model/loader.cpp:226-311: alpha(i) =
    fs*(1-ramp(i)) + ramp(i) for YaRN and fs for linear, fs = 1/factor, the
    divisor is 1/alpha; YaRN's magnitude m = (1 + 0.1 ln factor) * attention
    factor multiplies the scores by m^2 (full rotation only).
    """
    n_rot = head_dim if rot_dims == 0 else rot_dims
    fs = 1.0 / factor
    yarn = kind == "yarn"
    lo = hi = 0.0
    if yarn:
        def corr(beta):
            return n_rot * math.log(original_ctx / (beta * 2.0 * math.pi)) / (2.0 * math.log(base))
        lo = max(0.0, math.floor(corr(beta_fast)))
        hi = min(n_rot - 1.0, math.ceil(corr(beta_slow)))
    table = []
    for i in range(n_rot // 2):
        alpha = fs
        if yarn:
            y = (i - lo) / max(0.001, hi - lo)
            ramp = 1.0 - min(1.0, max(0.0, y))
            alpha = fs * (1.0 - ramp) + ramp
        table.append(float(np.float32(1.0 / alpha)) if alpha > 0.0 else 1.0)
    score = 1.0
    if yarn:
        if n_rot != head_dim:
            raise ValueError("YaRN scaling with a partly rotated head is not supported")
        m = (1.0 if factor <= 1.0 else 1.0 + 0.1 * math.log(factor)) * attention_factor
        score = float(np.float32(m * m))
    return table, score


class Position(Part):
    category = "position"
    score_scale = 1.0

    def rotary_tables(self):
        """(inv_freq, freq_factors, rot_dims) for the fused rotate-and-store
        kernel, or None when the encoding is not rotary."""
        return None

    def apply(self, qkv, ctx, heads_q, heads_kv, head_dim) -> None:
        """In-place encoding of float32 qkv rows for encodings that are not rotary."""
        raise NotImplementedError


@register_part("position", "none")
class NoPosition(Position):
    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)

    def rotary_tables(self):
        return (None, None, 0)


@register_part("position", "rope")
class Rope(Position):
    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.head_dim = int(p["head_dim"])
        self.rot_dims = int(p.get("rot_dims") or 0) or self.head_dim
        if self.rot_dims % 2 or self.rot_dims > self.head_dim:
            raise ValueError(f"rotary width {self.rot_dims} must be even and at most the head size {self.head_dim}")
        self.score_scale = float(p.get("score_scale", 1.0))
        n = self.rot_dims
        log_base = np.log(np.float32(p["base"])).astype(np.float32)
        i = np.arange(n // 2, dtype=np.float32)
        expo = (np.float32(-2.0) * i / np.float32(n)).astype(np.float32)
        inv = np.exp((expo * log_base).astype(np.float32)).astype(np.float32)
        self.inv_freq = torch.from_numpy(inv).to(rt.device)
        ff = p.get("freq_factors")
        self.freq_factors = None
        if ff is not None:
            if len(ff) < n // 2:
                raise ValueError(f"freq_factors has {len(ff)} entries, {n // 2} pairs rotate")
            self.freq_factors = torch.tensor(list(ff)[: n // 2], dtype=torch.float32, device=rt.device)

    def rotary_tables(self):
        return (self.inv_freq, self.freq_factors, self.rot_dims)

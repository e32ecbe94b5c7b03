"""The one stream of random numbers that seeded weights come from, on the host.

Element e of tensor number i under a 64-bit seed is a function of (seed, i, e) alone:
Philox4x32-10 with the seed as its key and the counter (e // 4 low word, e // 4 high word, i, 0)
gives four words; words 0 and 1 make the standard normals of elements 4c and 4c + 1, words 2
and 3 those of 4c + 2 and 4c + 3 (Box and Muller: radius from the first word, angle from the
second, cosine branch then sine branch).  The value is float32(mean + std * z), rounded once
more to bfloat16 where the tensor is stored so.

The kernel ``sb_random_normal`` (csrc/random_fill.hip) computes the same function on the GPU,
to the bit.  That holds because nothing here or there uses a library's logarithm, sine or
cosine: both sides run the same sequence of float64 additions, multiplications, divisions and
one square root, each rounded once as IEEE 754 says (no fused multiply-add on either side), with
the series and the constants below.  ``tests/test_gpu_random_stream.py`` compares the float64
values bit for bit.
"""
from __future__ import annotations

import numpy as np

from ..sampling.philox import philox4x32_10

LN2 = float.fromhex("0x1.62e42fefa39efp-1")
QUARTER_PI_OVER_2_30 = float.fromhex("0x1.921fb54442d18p-1") / float(1 << 30)     # (pi / 4) / 2^30
LOG_TERMS = 11            # 2 s (1 + s^2/3 + ... + s^20/21), |s| <= 0.1716
SIN_COEFFS = tuple((-1.0) ** k / float(np.prod(np.arange(1, 2 * k + 2, dtype=np.float64))) for k in range(8))
COS_COEFFS = tuple((-1.0) ** k / float(np.prod(np.arange(1, 2 * k + 1, dtype=np.float64))) for k in range(9))
LOG_COEFFS = tuple(1.0 / (2 * k + 1) for k in range(LOG_TERMS))
CHUNK = 1 << 16           # counters worked on at a time (stays in the cache)


def _neg2_log_u(word: np.ndarray) -> np.ndarray:
    """-2 ln((word + 0.5) / 2^32) in float64, by the sequence of operations the kernel runs."""
    x = (word.astype(np.float64) * 2.0 + 1.0)            # odd integer below 2^33: exact
    m, e = np.frexp(x)                                   # x = m 2^e, 0.5 <= m < 1: exact
    low = m < 0.7071067811865476
    m = np.where(low, m * 2.0, m)
    e = np.where(low, e - 1, e)
    s = (m - 1.0) / (m + 1.0)
    s2 = s * s
    p = np.full_like(s, LOG_COEFFS[-1])
    for c in LOG_COEFFS[-2::-1]:
        p = p * s2 + c
    ln = (e - 33).astype(np.float64) * LN2 + (2.0 * s) * p
    return -2.0 * ln


def _cos_sin(word: np.ndarray):
    """cos and sin of 2 pi (word + 0.5) / 2^32: the angle is reduced in integers to an eighth of
    a turn, both series run on at most pi / 4."""
    y = word.astype(np.uint64) * np.uint64(2) + np.uint64(1)          # angle = 2 pi y / 2^33
    octant = (y >> np.uint64(30)).astype(np.int64)
    r = (y & np.uint64((1 << 30) - 1)).astype(np.int64)
    odd = (octant & 1) == 1
    r = np.where(odd, (1 << 30) - r, r)
    phi = r.astype(np.float64) * QUARTER_PI_OVER_2_30
    p2 = phi * phi
    sp = np.full_like(phi, SIN_COEFFS[-1])
    for c in SIN_COEFFS[-2::-1]:
        sp = sp * p2 + c
    sp = sp * phi
    cp = np.full_like(phi, COS_COEFFS[-1])
    for c in COS_COEFFS[-2::-1]:
        cp = cp * p2 + c
    swap = (octant == 1) | (octant == 2) | (octant == 5) | (octant == 6)
    cos = np.where(swap, sp, cp)
    sin = np.where(swap, cp, sp)
    cos = np.where((octant >= 2) & (octant <= 5), -cos, cos)
    sin = np.where(octant >= 4, -sin, sin)
    return cos, sin


def standard_normals(seed: int, tensor_index: int, count: int, first: int = 0) -> np.ndarray:
    """float64 standard normals of elements ``first`` ... ``first + count - 1`` of a tensor."""
    seed = int(seed) & (2 ** 64 - 1)
    c_first, c_end = first // 4, (first + count + 3) // 4
    out = np.empty((c_end - c_first) * 4, dtype=np.float64)
    for a in range(c_first, c_end, CHUNK):
        b = min(c_end, a + CHUNK)
        c = np.arange(a, b, dtype=np.uint64)
        w = philox4x32_10(c & np.uint64(0xFFFFFFFF), c >> np.uint64(32), np.uint64(tensor_index), np.uint64(0), seed)
        z = out[(a - c_first) * 4:(b - c_first) * 4].reshape(-1, 4)
        for pair in (0, 1):
            radius = np.sqrt(_neg2_log_u(w[2 * pair]))
            cos, sin = _cos_sin(w[2 * pair + 1])
            z[:, 2 * pair] = radius * cos
            z[:, 2 * pair + 1] = radius * sin
    skip = first - c_first * 4
    return out[skip:skip + count]


def draw(seed: int, tensor_index: int, shape, mean: float, std: float) -> np.ndarray:
    """float32 array of ``shape``: float32(mean + std * z) in the tensor's row-major order."""
    n = int(np.prod(shape, dtype=np.int64)) if len(shape) else 1
    z = standard_normals(seed, tensor_index, n)
    return (z * float(std) + float(mean)).astype(np.float32).reshape(shape)

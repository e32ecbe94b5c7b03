"""Plain sampling, written from ``core/src/nn/sampling.cpp`` of the reference
(paths under ``/root/reference``).  Pure Python loops, float32 through NumPy
scalars where the reference computes in float, float64 where it uses double.
Shares no code with ``sonicboom_amd.sampling``.
"""
from __future__ import annotations

import math

import numpy as np

F32 = np.float32

K_CANDIDATES = 256      # core/include/sonicboom/nn/sampling.h:68
K_LOGIT_WINDOW = 30.0   # core/include/sonicboom/nn/sampling.h:61

_M0, _M1 = 0xD2511F53, 0xCD9E8D57   # core/src/nn/sampling.cpp:28-29
_W0, _W1 = 0x9E3779B9, 0xBB67AE85   # core/src/nn/sampling.cpp:30-31
_MASK = 0xFFFFFFFF


def philox4x32_10(counter, key: int):
    """core/src/nn/sampling.cpp:207-227."""
    c0, c1, c2, c3 = [int(c) & _MASK for c in counter]
    k0, k1 = key & _MASK, (key >> 32) & _MASK
    for _ in range(10):
        p0 = _M0 * c0
        p1 = _M1 * c2
        hi0, lo0 = p0 >> 32, p0 & _MASK
        hi1, lo1 = p1 >> 32, p1 & _MASK
        c0, c1, c2, c3 = hi1 ^ c1 ^ k0, lo1, hi0 ^ c3 ^ k1, lo0
        k0 = (k0 + _W0) & _MASK
        k1 = (k1 + _W1) & _MASK
    return [c0, c1, c2, c3]


def _counts(history, last_n: int, vocab: int):
    window = min(len(history), int(last_n))
    count = {}
    for t in history[len(history) - window:]:
        if 0 <= t < vocab:
            count[t] = count.get(t, 0) + 1
    return count


def penalize(logits, temperature_path: bool, repeat_penalty=1.0, repeat_last_n=64,
             presence_penalty=0.0, frequency_penalty=0.0, history=()):
    """core/src/nn/sampling.cpp:43-70 (greedy form) and :77-104 (single-rounding
    form); both give v>0 ? v/rp : v*rp, then v -= freq*count + presence."""
    adv = np.array(logits, dtype=F32, copy=True)
    rp, pp, fp = F32(repeat_penalty), F32(presence_penalty), F32(frequency_penalty)
    if len(history) == 0 or (rp == 1 and pp == 0 and fp == 0):
        return adv
    for t, c in _counts(list(history), repeat_last_n, adv.shape[0]).items():
        v = adv[t]
        if rp != 1:
            v = F32(v / rp) if v > 0 else F32(v * rp)
        if temperature_path:
            # fma(freq, c, presence) then fma(-1, adjust, v): one rounding each.
            adjust = F32(np.float64(fp) * np.float64(c) + np.float64(pp))
            v = F32(np.float64(v) - np.float64(adjust))
        else:
            v = F32(v - F32(F32(fp * F32(c)) + pp))
        adv[t] = v
    return adv


def allowed_by(mask, i: int) -> bool:
    """core/src/nn/sampling.cpp:266-274: bit i & 7 of byte i >> 3; an id past the
    bitmap is not allowed; an empty mask allows everything."""
    if not mask:
        return True
    byte = i >> 3
    return byte < len(mask) and bool((mask[byte] >> (i & 7)) & 1)


def select_candidates(logits, temperature, history=(), mask=None, **pen):
    """core/src/nn/sampling.cpp:257-285: z = l_adj / T as one float32 division
    over the ids the mask allows, the 256 largest z (ties to the lower id),
    ordered (z descending, id ascending)."""
    adv = penalize(logits, True, history=history, **pen)
    T = F32(temperature)
    cands = [(i, F32(adv[i] / T)) for i in range(adv.shape[0]) if allowed_by(mask, i)]
    cands.sort(key=lambda c: (-float(c[1]), c[0]))
    return cands[:K_CANDIDATES]


def filter_candidates(cands, top_k=0, top_p=1.0, min_p=0.0):
    """core/src/nn/sampling.cpp:157-203: window 30, top-k, min-p, nucleus."""
    if not cands:
        return []
    m = cands[0][1]
    floor_z = F32(m - F32(K_LOGIT_WINDOW))
    out = [c for c in cands if c[1] >= floor_z]
    if top_k > 0 and len(out) > top_k:
        out = out[:top_k]
    if min_p > 0.0:
        cutoff = F32(m + F32(math.log(F32(min_p))))
        out = [c for c in out if not (c[1] < cutoff)]
    if 0.0 < top_p < 1.0 and out:
        total = sum(math.exp(float(c[1]) - float(m)) for c in out)
        if total > 0.0:
            acc = 0.0
            keep = 0
            while keep < len(out):
                acc += math.exp(float(out[keep][1]) - float(m))
                if acc / total >= float(F32(top_p)):
                    keep += 1
                    break
                keep += 1
            keep = max(keep, 1)
            out = out[:min(keep, len(out))]
    return out


def draw(cands, seed: int, position: int) -> int:
    """core/src/nn/sampling.cpp:294-311: Gumbel-max with a Philox word keyed by
    (position, candidate id), u = (bits + 0.5) / 2^32, g = -ln(-ln u), the
    largest z + g in float64 wins, ties to the lower id."""
    best, best_score = -1, -math.inf
    for tid, z in cands:
        bits = philox4x32_10([position & _MASK, (position >> 32) & _MASK, tid, 0], seed)
        u = (float(bits[0]) + 0.5) / 4294967296.0
        g = -math.log(-math.log(u))
        score = float(z) + g
        if best < 0 or score > best_score or (score == best_score and tid < best):
            best, best_score = tid, score
    return best


def sample_token(logits, position: int, temperature=0.0, seed=0, top_k=0, top_p=1.0,
                 min_p=0.0, repeat_penalty=1.0, repeat_last_n=64, presence_penalty=0.0,
                 frequency_penalty=0.0, history=(), mask=None) -> int:
    """core/src/nn/sampling.cpp:314-352 (the mask as a filter over the ids, not
    through the compacted list, which selects the same)."""
    pen = dict(repeat_penalty=repeat_penalty, repeat_last_n=repeat_last_n,
               presence_penalty=presence_penalty, frequency_penalty=frequency_penalty)
    if not temperature > 0.0:
        adv = penalize(logits, False, history=history, **pen)
        best = -1
        for i in range(adv.shape[0]):
            if allowed_by(mask, i) and (best < 0 or adv[i] > adv[best]):
                best = i
        return best
    cands = select_candidates(logits, temperature, history=history, mask=mask, **pen)
    kept = filter_candidates(cands, top_k=top_k, top_p=top_p, min_p=min_p)
    return draw(kept, seed, position)


def surviving_ids(logits, temperature, history=(), top_k=0, top_p=1.0, min_p=0.0, **pen):
    """The candidate set the filters leave, ascending ids
    (core/include/sonicboom/nn/sampling.h:113-120)."""
    if not temperature > 0.0:
        return list(range(len(logits)))
    cands = select_candidates(logits, temperature, history=history, **pen)
    return sorted(c[0] for c in filter_candidates(cands, top_k, top_p, min_p))

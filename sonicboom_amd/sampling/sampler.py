"""Choosing the next token of every sequence of a step.

The order of stages is the reference's
(/root/reference/core/include/sonicboom/nn/sampling.h:93-98): penalties over the
last ``repeat_last_n`` tokens of the history, the mask of constrained decoding (a
bitmap of the ids a row may choose from, when the caller brings one), then either the argmax
(temperature 0, ties to the lowest id) or: the 256 best candidates by
z = logit / temperature, a window of 30 below the best, top-k, min-p, top-p,
and a Gumbel-max draw with a Philox4x32-10 word keyed by (seed, position of
the token being produced, candidate id).  All of it runs on the device over the
whole batch: penalties, argmax, the candidate selection, and the filters and the
draw over each row's 256 candidates (a wave a row, the running sums of top-p and
the Gumbel scores in float64, /root/reference/core/src/nn/sampling.cpp:157-203,
:287-312); a step's tokens come back in one small copy.  The same filters and draw
on the host, row by row and for all rows at once in array arithmetic, are
:func:`filter_candidates`, :func:`gumbel_draw` and :func:`draw_rows`: what the
tests hold the device kernel to, beside the plain sampler.
Every sequence draws from its own (seed, position) stream, so its tokens do
not depend on what else is in the batch.
"""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from .. import ops
from .params import SamplingParams
from .philox import philox4x32_10

LOGIT_WINDOW = np.float32(30.0)     # /root/reference/core/include/sonicboom/nn/sampling.h:61
CANDIDATES = 256                    # /root/reference/core/include/sonicboom/nn/sampling.h:68


def penalty_items(histories: Sequence[Sequence[int]], last_n: int, vocab: int):
    """(row, token, count) triples of the tokens in each history's trailing window."""
    rows, toks, counts = [], [], []
    for r, h in enumerate(histories):
        window = min(len(h), last_n)
        if window == 0:
            continue
        seen = {}
        for t in h[len(h) - window:]:
            if 0 <= t < vocab:
                seen[t] = seen.get(t, 0) + 1
        for t, c in seen.items():
            rows.append(r)
            toks.append(t)
            counts.append(c)
    return rows, toks, counts


def filter_candidates(ids: np.ndarray, z: np.ndarray, p: SamplingParams):
    """Window, top-k, min-p and nucleus over candidates ordered (z descending, id ascending)."""
    if ids.size == 0:
        return ids, z
    m = z[0]
    keep = int(np.count_nonzero(z >= np.float32(m - LOGIT_WINDOW)))
    if p.top_k > 0:
        keep = min(keep, p.top_k)
    ids, z = ids[:keep], z[:keep]
    if p.min_p > 0.0:
        cutoff = np.float32(m + np.log(np.float32(p.min_p)))
        ok = ~(z < cutoff)
        ids, z = ids[ok], z[ok]
    if 0.0 < p.top_p < 1.0 and ids.size:
        e = np.exp(z.astype(np.float64) - np.float64(m))
        acc = np.cumsum(e)            # sequential, like the reference's running sums
        total = acc[-1]
        if total > 0.0:
            reached = np.nonzero(acc / total >= np.float64(np.float32(p.top_p)))[0]
            n = int(reached[0]) + 1 if reached.size else ids.size
            ids, z = ids[:max(n, 1)], z[:max(n, 1)]
    return ids, z


def gumbel_draw(ids: np.ndarray, z: np.ndarray, seed: int, position: int) -> int:
    """The candidate with the largest z + g, g = -ln(-ln u), u from Philox word 0
    of counter (position lo, position hi, id, 0); ties go to the lower id."""
    if ids.size == 0:
        return -1
    w0, _, _, _ = philox4x32_10(position & 0xFFFFFFFF, (position >> 32) & 0xFFFFFFFF, ids.astype(np.uint64), 0, seed)
    u = (w0.astype(np.float64) + 0.5) / 4294967296.0
    score = z.astype(np.float64) - np.log(-np.log(u))
    best = score.max()
    return int(ids[score == best].min())


def draw_rows(ids: np.ndarray, z: np.ndarray, positions: Sequence[int], p: SamplingParams) -> List[int]:
    """:func:`filter_candidates` and :func:`gumbel_draw` for every row of a step at once:
    ``ids`` and ``z`` are [rows, candidates], each row ordered (z descending, id ascending).  The
    same arithmetic element by element (the kept candidates of a row are always a prefix of it,
    so masks stand in for the slices), hence the same tokens; a step of 64 rows costs what one
    row costs in the row-by-row form."""
    n, k = z.shape
    if k == 0:
        return [-1] * n
    ids = np.asarray(ids)
    z = np.asarray(z, dtype=np.float32)
    cols = np.arange(k)[None, :]
    m = z[:, :1]
    keep = np.count_nonzero(z >= (m - LOGIT_WINDOW), axis=1)
    if p.top_k > 0:
        keep = np.minimum(keep, p.top_k)
    live = cols < keep[:, None]
    if p.min_p > 0.0:
        cutoff = m + np.log(np.float32(p.min_p))
        live &= ~(z < cutoff)
    if 0.0 < p.top_p < 1.0:
        count = live.sum(axis=1)
        e = np.where(live, np.exp(z.astype(np.float64) - m.astype(np.float64)), 0.0)
        acc = np.cumsum(e, axis=1)                    # row by row, in order
        total = acc[np.arange(n), np.maximum(count, 1) - 1]
        usable = (count > 0) & (total > 0.0)
        with np.errstate(divide="ignore", invalid="ignore"):
            reached = (acc / total[:, None] >= np.float64(np.float32(p.top_p))) & live
        n_keep = np.where(reached.any(axis=1), reached.argmax(axis=1) + 1, count)
        n_keep = np.where(usable, np.maximum(n_keep, 1), count)
        live &= cols < n_keep[:, None]
    pos = np.asarray([int(q) for q in positions], dtype=np.uint64)
    w0 = philox4x32_10((pos & np.uint64(0xFFFFFFFF))[:, None], (pos >> np.uint64(32))[:, None],
                       ids.astype(np.uint64), 0, p.seed)[0]
    u = (w0.astype(np.float64) + 0.5) / 4294967296.0
    score = np.where(live, z.astype(np.float64) - np.log(-np.log(u)), -np.inf)
    best = score.max(axis=1)
    tie = (score == best[:, None]) & live
    chosen = np.where(tie, ids.astype(np.int64), np.iinfo(np.int64).max).min(axis=1)
    return [int(c) if a else -1 for c, a in zip(chosen, live.any(axis=1))]


class Sampler:
    def __init__(self, params: SamplingParams):
        self.params = params.validated()

    def device_draw(self, vocab: int):
        """What a decode loop needs to draw on the device inside its own recorded step
        (temperature, candidates, top_k, ln min_p or None, top_p or None, seed): None when the
        choice is greedy or needs the host (penalties over the histories)."""
        p = self.params
        if not p.temperature > 0.0 or p.has_penalties:
            return None
        return (float(p.temperature), min(CANDIDATES, vocab), int(p.top_k), self._log_min_p(), self._top_p(),
                int(p.seed))

    # the cut-offs as the host form rounds them: ln(min_p) in float32, top_p through float32
    def _log_min_p(self) -> Optional[float]:
        return float(np.log(np.float32(self.params.min_p))) if self.params.min_p > 0.0 else None

    def _top_p(self) -> Optional[float]:
        return float(np.float64(np.float32(self.params.top_p))) if 0.0 < self.params.top_p < 1.0 else None

    def pick(self, logits: torch.Tensor, positions: Sequence[int], histories: Sequence[Sequence[int]],
             masks: Optional[Sequence[Optional[bytes]]] = None) -> List[int]:
        """One token per row of float32 ``logits`` [rows, vocab] (modified in place when
        penalties or masks apply).  ``positions[r]`` is the absolute position the new token of
        row r will take; ``histories[r]`` its prompt and generated tokens so far; ``masks[r]``
        the bitmap of the ids row r may choose from (bit i & 7 of byte i >> 3 for id i, ids past
        the bitmap not allowed; None or empty: no constraint), applied after the penalties
        (/root/reference/core/src/nn/sampling.cpp:266-274, :334-339).  -1 for a row that may
        choose nothing."""
        p = self.params
        n, vocab = logits.shape
        sampled = p.temperature > 0.0
        if p.has_penalties:
            rows, toks, counts = penalty_items(histories, p.repeat_last_n, vocab)
            if rows:
                dev = logits.device
                items = torch.tensor([rows, toks, counts], dtype=torch.int32).to(dev)
                ops.penalize(logits, items[0].contiguous(), items[1].contiguous(), items[2].contiguous(),
                             p.repeat_penalty, p.presence_penalty, p.frequency_penalty, exact=sampled)
        nothing_allowed = [False] * n
        if masks is not None and any(masks):
            n_bytes = (vocab + 7) // 8
            bitmaps = np.zeros((n, n_bytes), dtype=np.uint8)
            for r, mask in enumerate(masks):
                if not mask:
                    bitmaps[r] = 0xFF
                    continue
                row = np.frombuffer(bytes(mask), dtype=np.uint8)[:n_bytes]
                bitmaps[r, :row.size] = row
                if vocab % 8:
                    bitmaps[r, -1] &= (1 << (vocab % 8)) - 1
                nothing_allowed[r] = not bitmaps[r].any()
            ops.mask_logits(logits, torch.from_numpy(bitmaps).to(logits.device))
        if not sampled:
            tokens = ops.argmax(logits).tolist()
            return [-1 if none else t for t, none in zip(tokens, nothing_allowed)]
        k = min(CANDIDATES, vocab)
        ids_d, z_d = ops.top_candidates(logits, p.temperature, k)
        tokens = ops.draw(ids_d, z_d, positions, p.top_k, self._log_min_p(), self._top_p(), p.seed).tolist()
        return [-1 if none else t for t, none in zip(tokens, nothing_allowed)]

"""Helpers of the GPU tests: plain logits per request, the three ways of cutting a
request into steps, and the comparison of logits."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from plain import qwen2_plain  # noqa: E402

_PLAIN_MODELS = {}
_PLAIN_LOGITS = {}


def plain_model(folder):
    if folder not in _PLAIN_MODELS:
        _PLAIN_MODELS[folder] = qwen2_plain.load_model(folder)
    return _PLAIN_MODELS[folder]


def plain_logits(folder, tokens):
    """Logits [n, vocab] of the plain implementation for one whole request."""
    key = (folder, tuple(tokens))
    if key not in _PLAIN_LOGITS:
        cfg, w = plain_model(folder)
        _PLAIN_LOGITS[key] = qwen2_plain.forward(cfg, w, list(tokens))
    return _PLAIN_LOGITS[key]


# Tolerances, fixed: float32 differs from the plain implementation by the
# rounding of float32 sums (the plain one sums in float64); bfloat16 by the
# rounding of activations to 8 bits of mantissa at every part's boundary.
TOL = {"float32": dict(atol=5e-5, rtol=5e-5), "bfloat16": dict(atol=3e-2, rtol=3e-2)}


def assert_logits_close(got, want, dtype, what=""):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: logits are not finite"
    tol = TOL[dtype]
    scale = max(1.0, float(np.abs(want).max()))
    err = np.abs(got - want)
    bound = tol["atol"] * scale + tol["rtol"] * np.abs(want)
    if not (err <= bound).all():
        i = np.unravel_index(np.argmax(err - bound), err.shape)
        raise AssertionError(f"{what}: logits differ at {i}: got {got[i]:.6g}, want {want[i]:.6g} "
                             f"(|diff| {err[i]:.3g} > {bound[i]:.3g}); max |diff| {err.max():.3g}")
    return float(err.max())


def run_whole(engine, tokens):
    """One request alone: all its tokens in one step, logits at every position."""
    from sonicboom_amd.engine import StepEntry
    s = engine.alloc_slot()
    try:
        return engine.step([StepEntry(s, tokens, range(len(tokens)))]).cpu().numpy()
    finally:
        engine.free_slot(s)


def run_tail_one_by_one(engine, tokens, tail=32):
    """The request's head in one step, its last ``tail`` tokens one by one."""
    from sonicboom_amd.engine import StepEntry
    tail = min(tail, len(tokens) - 1)
    head = len(tokens) - tail
    s = engine.alloc_slot()
    try:
        rows = [engine.step([StepEntry(s, tokens[:head], range(head))]).cpu().numpy()]
        for t in tokens[head:]:
            rows.append(engine.step([StepEntry(s, [t], [0])]).cpu().numpy())
        return np.concatenate(rows, axis=0)
    finally:
        engine.free_slot(s)


def run_batch(engine, requests, prompt_lens):
    """Requests that start together: prompts (the first ``prompt_lens[i]`` tokens) in one step,
    then one token each per step; shorter requests end earlier.  Returns logits per request,
    from its last prompt position to its end."""
    from sonicboom_amd.engine import StepEntry
    slots = [engine.alloc_slot() for _ in requests]
    got = [[] for _ in requests]
    try:
        out = engine.step([StepEntry(s, r[:n], range(n)) for s, r, n in zip(slots, requests, prompt_lens)]).cpu().numpy()
        off = 0
        for i, n in enumerate(prompt_lens):
            got[i].append(out[off:off + n])
            off += n
        pos = list(prompt_lens)
        live = [i for i in range(len(requests)) if pos[i] < len(requests[i])]
        for i in range(len(requests)):
            if i not in live:
                engine.free_slot(slots[i])
                slots[i] = None
        while live:
            out = engine.step([StepEntry(slots[i], [requests[i][pos[i]]], [0]) for i in live]).cpu().numpy()
            for k, i in enumerate(live):
                got[i].append(out[k:k + 1])
                pos[i] += 1
            for i in list(live):
                if pos[i] >= len(requests[i]):
                    live.remove(i)
                    engine.free_slot(slots[i])
                    slots[i] = None
        return [np.concatenate(g, axis=0) for g in got]
    finally:
        for s in slots:
            if s is not None:
                engine.free_slot(s)

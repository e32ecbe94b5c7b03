"""Helpers of the GPU tests: plain logits per request, the three ways of cutting a
request into steps, and the comparison of logits."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))
from plain import qwen2_plain  # noqa: E402

_PLAIN_MODELS = {}
_PLAIN_LOGITS = {}


def plain_model(folder, wide=False):
    """The plain implementation's (configuration, weights) of a folder.  ``wide`` keeps the
    matrices in float64 (the same values: every float32 is one), which spares the plain products
    their conversion at every call; it pays for models of real layer sizes."""
    if folder not in _PLAIN_MODELS:
        cfg, w = qwen2_plain.load_model(folder)
        if wide:
            w = {k: (v.astype(np.float64) if v.ndim == 2 else v) for k, v in w.items()}
        _PLAIN_MODELS[folder] = (cfg, w)
    return _PLAIN_MODELS[folder]


def plain_logits(folder, tokens):
    """Logits [n, vocab] of the plain implementation for one whole request."""
    key = (folder, tuple(tokens))
    if key not in _PLAIN_LOGITS:
        cfg, w = plain_model(folder)
        _PLAIN_LOGITS[key] = qwen2_plain.forward(cfg, w, list(tokens))
    return _PLAIN_LOGITS[key]


def forget_plain(folder):
    """Drop what is cached for a folder (large models)."""
    _PLAIN_MODELS.pop(folder, None)
    for key in [k for k in _PLAIN_LOGITS if k[0] == folder]:
        del _PLAIN_LOGITS[key]


# Tolerances, fixed.  float32 differs from the plain implementation by the rounding of float32
# sums (the plain one sums in float64).  bfloat16 rounds activations to 8 bits of mantissa at
# every part's boundary; what that does to a logit is measured against the spread of the logits
# (their standard deviation), not against 1, and in two ways: no logit may be off by more than
# a fraction of the spread plus a fraction of itself, and the root mean square of all differences,
# which rounding keeps small and a systematic mistake does not, has a tighter bound of its own.
# On the "sharp" models (conftest.SHARP_QK) scores of ten and more make the softmax amplify the
# rounding of queries and keys: measured on the GPU over the whole suite the largest difference
# was 0.287 spreads and the root mean square 0.0233, against 0.0257 and 0.0055 on the tiny models
# of plain random weights; the bounds of both kinds are what was measured times 1.4.
# "wide" is for models of real layer sizes, where a row of 3,584 and a sum over 18,944 products
# round more often: measured 0.066 and 0.013 there (the largest over two layers of the 7B, 14B and
# 72B sizes; the 7B sizes alone 0.058 and 0.0095), where the smallest of the mistakes that
# tests/test_plain.py::test_sharp_models_show_attention_mistakes plants, a dropped query bias,
# moves the plain logits by 0.20 and 0.031 (a wrong scale by 4.6 and 0.88): the bounds are what
# was measured times 1.4, and that mistake is 2.2 and 1.7 times beyond them.
F32_TOL = dict(atol=5e-5, rtol=5e-5)
BF16_MAX = {"tiny": 0.036, "wide": 0.09, "sharp": 0.4}     # largest difference, in spreads (plus BF16_REL * |logit|)
BF16_RMS = {"tiny": 0.008, "wide": 0.018, "sharp": 0.033}   # root mean square of the differences, in spreads
BF16_REL = 0.02
# the largest of both that the bfloat16 comparisons of this run have seen, by kind (the summary
# at the end of a test run prints them: what the bounds above are set from)
BF16_SEEN = {}


def bf16_limits(want, sharp=False):
    """(bound on every |difference|, bound on their root mean square) for logits ``want``;
    ``sharp``: False / "tiny", True / "sharp", or "wide"."""
    kind = {False: "tiny", True: "sharp"}.get(sharp, sharp)
    want = np.asarray(want, dtype=np.float64)
    spread = float(want.std())
    return BF16_MAX[kind] * spread + BF16_REL * np.abs(want), BF16_RMS[kind] * spread


def assert_logits_close(got, want, dtype, what="", sharp=False):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    assert np.isfinite(got).all(), f"{what}: logits are not finite"
    err = np.abs(got - want)
    if dtype == "float32":
        bound = F32_TOL["atol"] * max(1.0, float(np.abs(want).max())) + F32_TOL["rtol"] * np.abs(want)
    else:
        bound, rms_bound = bf16_limits(want, sharp)
        rms = float(np.sqrt((err ** 2).mean())) if err.size else 0.0
        spread = float(want.std())
        if err.size and spread > 0:
            kind = {False: "tiny", True: "sharp"}.get(sharp, sharp)
            seen = BF16_SEEN.setdefault(kind, [0.0, 0.0])
            seen[0] = max(seen[0], float((err - BF16_REL * np.abs(want)).max()) / spread)
            seen[1] = max(seen[1], rms / spread)
        assert rms <= rms_bound, f"{what}: root mean square difference {rms:.3g} > {rms_bound:.3g}"
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

"""The plain implementation pinned by what fixes it beside the reference's text: vectors
the reference's own tests hold, special cases that reduce to a library routine, and
invariants.  Each case is chosen so that a plausible mistake fails it (a wrong sign or
pairing in the rotation, eps outside the root, a norm in the wrong place, the bias after
the rotation, a wrong head mapping)."""
import math

import numpy as np
import pytest
import torch

from plain import qwen2_plain as P

F32 = np.float32


def rng(seed=0):
    return np.random.default_rng(seed)


# ---- RMS norm ------------------------------------------------------------------------------
def test_rms_norm_reference_vectors():
    """/root/reference/tests/core/test_nn.cpp:172-219."""
    assert np.allclose(P.rms_norm(np.array([[2, 2, 2, 2]], F32), None, 0.0), 1.0, atol=1e-6)
    assert np.allclose(P.rms_norm(np.array([[2, 2, 2, 2]], F32), np.full(4, 3, F32), 0.0), 3.0, atol=1e-6)
    # eps inside the root, added to the mean: mean 0.25 + 0.75 = 1 exactly
    assert np.array_equal(P.rms_norm(np.array([[1, 0, 0, 0]], F32), None, 0.75), np.array([[1, 0, 0, 0]], F32))


def test_rms_norm_invariants():
    for n in (64, 201, 338):                       # test_nn.cpp:192-208
        x = rng(n).uniform(-4, 4, size=(3, n)).astype(F32)
        y = P.rms_norm(x, None, 0.0)
        assert np.allclose(np.sqrt((y.astype(np.float64) ** 2).mean(-1)), 1.0, atol=1e-4)
        assert np.allclose(P.rms_norm(x * F32(7.5), None, 0.0), y, atol=1e-5)      # scale free without eps
        want = x / np.linalg.norm(x.astype(np.float64), axis=-1, keepdims=True) * math.sqrt(n)
        assert np.allclose(y, want, atol=1e-5)
    # the weight multiplies as it is (not 1 + w)
    x = rng(1).standard_normal((2, 8)).astype(F32)
    assert np.allclose(P.rms_norm(x, np.zeros(8, F32), 1e-6), 0.0)


# ---- rotation --------------------------------------------------------------------------------
def test_rope_reference_vectors():
    """/root/reference/tests/core/test_nn.cpp:221-290."""
    x = np.array([[0.5, -1.25, 2.0, 3.5]], F32)
    assert np.array_equal(P.rope_neox(x, [0], 4, 10000.0), x)                        # position 0: identity
    # head size 2, base 1: theta = pos, so pos = pi/2 is a quarter turn ... positions are integers
    # here, so the same is reached through the frequency table: theta = 1 / (2/pi)
    q = P.rope_neox(np.array([[1.0, 0.0]], F32), [1], 2, 1.0, freq_factors=[2.0 / math.pi])
    assert np.allclose(q, [[0.0, 1.0]], atol=1e-6)
    # pairs are (i, i + half): with both angles pi/2, (x0, x2) -> (-x2, x0) and (x1, x3) -> (-x3, x1);
    # an interleaved (2i, 2i+1) pairing would give (-x1, x0, -x3, x2) instead
    ff = [2.0 / math.pi, 2.0 / math.pi]
    y = P.rope_neox(np.array([[1.0, 0.0, 2.0, 3.0]], F32), [1], 4, 1.0, freq_factors=ff)
    assert np.allclose(y, [[-2.0, -3.0, 1.0, 0.0]], atol=1e-6)
    # a huge divisor freezes its pair (test_nn.cpp:272-289)
    y = P.rope_neox(np.array([[1.0, 0.0, 2.0, 3.0]], F32), [1], 4, 1.0, freq_factors=[2.0 / math.pi, 1e30])
    assert np.allclose(y, [[-2.0, 0.0, 1.0, 3.0]], atol=1e-5)
    with pytest.raises(ValueError):
        P.rope_neox(np.zeros((1, 6), F32), [1], 6, 10000.0, rot_dims=3)


def test_rope_invariants():
    r = rng(2)
    hd = 32
    q = r.standard_normal((1, hd)).astype(F32)
    k = r.standard_normal((1, hd)).astype(F32)
    # an orthogonal transform: the norm is kept (test_nn.cpp:243-258)
    for pos in (1, 7, 1000):
        assert abs(np.linalg.norm(P.rope_neox(q, [pos], hd, 1e4)) - np.linalg.norm(q)) < 1e-4
    # only distances count: <rope(q, m), rope(k, n)> depends on m - n
    def dot(m, n):
        return (P.rope_neox(q, [m], hd, 1e4) @ P.rope_neox(k, [n], hd, 1e4).T).item()
    assert abs(dot(5, 2) - dot(105, 102)) < 1e-4 and abs(dot(5, 2) - dot(40, 37)) < 1e-4
    assert abs(dot(5, 2) - dot(2, 5)) > 1e-3                    # and on its sign
    # every head is rotated alike; a partly rotated head keeps its tail
    two = np.concatenate([q, q], axis=1)
    out = P.rope_neox(two, [9], hd, 1e4)
    assert np.array_equal(out[:, :hd], out[:, hd:])
    part = P.rope_neox(q, [9], hd, 1e4, rot_dims=16)
    assert np.array_equal(part[:, 16:], q[:, 16:]) and not np.allclose(part[:, :16], q[:, :16])
    # the angle of pair i is pos * base^(-2i/n)
    one = np.zeros((1, hd), F32)
    one[0, 3] = 1.0
    y = P.rope_neox(one, [11], hd, 1e4)
    theta = 11 * 1e4 ** (-2 * 3 / hd)
    assert np.allclose([y[0, 3], y[0, 3 + hd // 2]], [math.cos(theta), math.sin(theta)], atol=1e-5)


def test_yarn_table_limits():
    cfg = {"_head_dim": 64, "rope_theta": 1e4, "max_position_embeddings": 4096,
           "rope_scaling": {"type": "yarn", "factor": 8.0, "original_max_position_embeddings": 512}}
    ff, mult = P.rope_scaling(cfg)
    assert ff[0] == 1.0 and abs(ff[-1] - 8.0) < 1e-6 and all(a <= b + 1e-6 for a, b in zip(ff, ff[1:]))
    assert abs(mult - (1 + 0.1 * math.log(8.0)) ** 2) < 1e-6
    lin, m1 = P.rope_scaling({"_head_dim": 8, "rope_theta": 1e4, "rope_scaling": {"type": "linear", "factor": 4.0}})
    assert lin == [4.0] * 4 and m1 == 1.0
    assert P.rope_scaling({"_head_dim": 8, "rope_theta": 1e4}) == (None, 1.0)


# ---- softmax and attention -------------------------------------------------------------------
def test_softmax_vectors():
    """/root/reference/tests/core/test_nn.cpp:292-330."""
    assert np.allclose(P.softmax(np.array([1, 2, 3], F32)), [0.09003057, 0.24472847, 0.66524096], atol=1e-7)
    assert np.allclose(P.softmax(np.array([0, 0], F32)), [0.5, 0.5])
    x = rng(3).standard_normal(9).astype(F32)
    assert np.allclose(P.softmax(x), P.softmax(x + F32(100.0)), atol=1e-6)          # shift invariant
    assert np.isfinite(P.softmax(np.array([1e4, 1e4 - 1], F32))).all()


def attn(q, k, v, hq, hkv, hd, scale=1.0, causal=True, window=0, qpos=None):
    q, k, v = (np.asarray(a, F32) for a in (q, k, v))
    nq, nk = q.shape[0], k.shape[0]
    return P.attention(q, k, v, np.arange(nq) if qpos is None else qpos, np.arange(nk), hq, hkv, hd, scale,
                       causal, window)


def test_attention_reference_vectors():
    """/root/reference/tests/core/test_nn.cpp:402-511."""
    assert np.allclose(attn([[1.0]], [[1.0]], [[5.0]], 1, 1, 1, causal=False), [[5.0]])
    assert np.allclose(attn([[1, 0, 0, 0]], [[1, 0, 0, 0]], [[1, 2, 3, 4]], 1, 1, 4, causal=False), [[1, 2, 3, 4]])
    assert np.allclose(attn([[1], [1]], [[1], [1]], [[2], [4]], 1, 1, 1).flatten(), [2.0, 3.0])    # causal
    assert np.allclose(attn([[1, 1, 1, 1]], [[1, 1]], [[1, 2]], 4, 2, 1, causal=False), [[1, 1, 2, 2]])   # GQA map
    assert abs(attn([[1], [1], [1]], [[1], [1], [1]], [[1], [2], [4]], 1, 1, 1, window=2)[2, 0] - 3.0) < 1e-6
    assert abs(attn([[2.0]], [[2.0], [0.0]], [[1.0], [3.0]], 1, 1, 1, 1.0, causal=False)[0, 0] - 1.0360) < 1e-3
    assert abs(attn([[2.0]], [[2.0], [0.0]], [[1.0], [3.0]], 1, 1, 1, 0.5, causal=False)[0, 0] - 1.2384) < 1e-3
    with pytest.raises(ValueError):
        attn([[1, 1, 1]], [[1, 1]], [[1, 1]], 3, 2, 1)
    # a row that sees no key is zero (attention.cpp:74-78)
    assert np.array_equal(attn([[1.0]], [[1.0]], [[5.0]], 1, 1, 1, qpos=[-1]), [[0.0]])


def test_attention_equals_the_library_routine_without_mask_or_rotation():
    r = rng(4)
    n, h, hd = 7, 3, 8
    q, k, v = (r.standard_normal((n, h * hd)).astype(F32) for _ in range(3))
    scale = 1 / math.sqrt(hd)
    got = attn(q, k, v, h, h, hd, scale, causal=False)
    tq, tk, tv = (torch.from_numpy(a).view(n, h, hd).transpose(0, 1).double() for a in (q, k, v))
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv).transpose(0, 1).reshape(n, h * hd)
    assert np.allclose(got, want.numpy(), atol=2e-6)
    want_c = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True)
    assert np.allclose(attn(q, k, v, h, h, hd, scale), want_c.transpose(0, 1).reshape(n, h * hd).numpy(), atol=2e-6)


def test_attention_invariants():
    r = rng(5)
    n, hq, hkv, hd = 9, 4, 2, 8
    q = r.standard_normal((n, hq * hd)).astype(F32)
    k = r.standard_normal((n, hkv * hd)).astype(F32)
    v = r.standard_normal((n, hkv * hd)).astype(F32)
    base = attn(q, k, v, hq, hkv, hd, 0.3)
    # equal scores: the causal running mean of the values
    mean = attn(np.zeros_like(q), k, v, hq, hkv, hd, 0.3)
    want = np.cumsum(v.reshape(n, hkv, hd), axis=0) / np.arange(1, n + 1)[:, None, None]
    assert np.allclose(mean.reshape(n, hq, hd)[:, ::2], want, atol=1e-5)
    # grouped heads equal full heads with keys and values repeated per group
    rep = lambda a: np.repeat(a.reshape(n, hkv, hd), hq // hkv, axis=1).reshape(n, hq * hd)  # noqa: E731
    assert np.allclose(base, attn(q, rep(k), rep(v), hq, hq, hd, 0.3), atol=1e-6)
    # causality: a later key does not change earlier rows
    k2, v2 = k.copy(), v.copy()
    k2[6:], v2[6:] = 9.0, -9.0
    assert np.array_equal(attn(q, k2, v2, hq, hkv, hd, 0.3)[:6], base[:6])
    # a window of one sees only the row's own key
    assert np.allclose(attn(q, k, v, hq, hkv, hd, 0.3, window=1), rep(v), atol=1e-6)


# ---- feed-forward ----------------------------------------------------------------------------
def test_silu_and_swiglu():
    """/root/reference/tests/core/test_nn.cpp:52-66."""
    s = P.silu(np.array([0.0, 1.0, -1.0, 100.0, -100.0], F32))
    assert s[0] == 0.0 and abs(s[1] - 0.7310586) < 1e-6 and abs(s[2] + 0.26894143) < 1e-6
    assert s[3] == 100.0 and abs(s[4]) < 1e-30
    r = rng(6)
    f = r.standard_normal((3, 8)).astype(F32)
    wg, wu, wd = (r.standard_normal(sh).astype(F32) for sh in ((12, 8), (12, 8), (8, 12)))
    assert np.array_equal(P.swiglu(f, np.zeros_like(wg), wu, wd), np.zeros((3, 8), F32))     # silu(0) = 0
    assert np.array_equal(P.swiglu(f, wg, wu, np.zeros_like(wd)), np.zeros((3, 8), F32))
    g, u = f @ wg.T, f @ wu.T
    want = (torch.nn.functional.silu(torch.from_numpy(g).double()).numpy() * u) @ wd.T
    assert np.allclose(P.swiglu(f, wg, wu, wd), want, atol=1e-4)
    # the gate, not the up projection, goes through the activation
    assert not np.allclose(P.swiglu(f, wg, wu, wd), P.swiglu(f, wu, wg, wd), atol=1e-3)


# ---- the whole model ---------------------------------------------------------------------------
@pytest.fixture(scope="module")
def models(model_folders):
    return {k: P.load_model(v) for k, v in model_folders.items()}


def test_residual_stack_without_branches(models):
    """With every output and down projection zero the blocks add nothing: the logits are
    head(norm(embedding)) per token, wherever the token stands."""
    cfg, w = models["B"]
    w = dict(w)
    for name in w:
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            w[name] = np.zeros_like(w[name])
    tokens = [3, 77, 3, 200]
    got = P.forward(cfg, w, tokens)
    want = P.linear(P.rms_norm(w["model.embed_tokens.weight"][tokens], w["model.norm.weight"], cfg["rms_norm_eps"]),
                    w["lm_head.weight"])
    assert np.allclose(got, want, atol=1e-6) and np.allclose(got[0], got[2], atol=1e-6)


def test_bias_precedes_rotation(models):
    """With zero q and k matrices, queries and keys are rotated biases, so the scores are
    sum(b_q R(delta) b_k): they depend on the distance.  A bias added after the rotation
    would give scores that do not."""
    cfg, w = models["A"]
    hd, hq, hkv = cfg["_head_dim"], cfg["num_attention_heads"], cfg["num_key_value_heads"]
    p = "model.layers.0.self_attn."
    bq, bk = w[p + "q_proj.bias"], w[p + "k_proj.bias"]
    h = np.zeros((5, cfg["hidden_size"]), F32)
    q = P.rope_neox(P.linear(h, np.zeros_like(w[p + "q_proj.weight"]), bq), np.arange(5), hd, cfg["rope_theta"])
    k = P.rope_neox(P.linear(h, np.zeros_like(w[p + "k_proj.weight"]), bk), np.arange(5), hd, cfg["rope_theta"])
    s = q.reshape(5, hq, hd)[:, 0] @ k.reshape(5, hkv, hd)[:, 0].T
    assert abs(s[4, 2] - s[3, 1]) < 1e-6 and abs(s[4, 2] - s[2, 0]) < 1e-6      # same distance, same score
    assert abs(s[4, 2] - s[4, 3]) > 1e-7                                         # another distance differs


def _zero_qk_bias(w, prefix):
    w = dict(w)
    for r in ("q_proj", "k_proj", "v_proj"):
        w[prefix + r + ".bias"] = np.zeros_like(w[prefix + r + ".bias"])
    return w


def test_self_attention_default_scale_is_the_library_routines(models):
    """P.self_attention itself (not a scale passed in by the test) against torch's
    scaled_dot_product_attention with its default scale, 1/sqrt(head size): biases zero, and the
    rotation frozen by a linear position scaling of 1e30 (every angle is 0), so what is left is
    projections, causal grouped attention and the output projection.  A scale of 1, of
    1/head size or of 1/sqrt(width) fails this."""
    for name in ("A", "B"):
        cfg, w = models[name]
        cfg = dict(cfg, rope_scaling={"type": "linear", "factor": 1e30})
        hq, hkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["_head_dim"]
        p = "model.layers.1.self_attn."
        w = _zero_qk_bias(w, p)
        n = 11
        # activations large enough for scores of a few units: a wrong scale then matters
        h = (rng(12).standard_normal((n, cfg["hidden_size"])) * 12.0).astype(F32)
        got = P.self_attention(h, np.arange(n), w, p, cfg)
        hh = torch.from_numpy(h).double()
        q, k, v = (hh @ torch.from_numpy(w[p + r + ".weight"]).double().T for r in ("q_proj", "k_proj", "v_proj"))
        q = q.view(n, hq, hd).transpose(0, 1)
        k = k.view(n, hkv, hd).transpose(0, 1).repeat_interleave(hq // hkv, dim=0)
        v = v.view(n, hkv, hd).transpose(0, 1).repeat_interleave(hq // hkv, dim=0)
        a = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True)
        want = a.transpose(0, 1).reshape(n, hq * hd) @ torch.from_numpy(w[p + "o_proj.weight"]).double().T
        assert np.allclose(got, want.numpy(), atol=2e-5), name
        wrong = torch.nn.functional.scaled_dot_product_attention(q, k, v, is_causal=True, scale=1.0)
        wrong = wrong.transpose(0, 1).reshape(n, hq * hd) @ torch.from_numpy(w[p + "o_proj.weight"]).double().T
        assert np.abs(wrong.numpy() - want.numpy()).max() > 1e-2, "the case cannot tell the scales apart"


def test_self_attention_rotates_after_the_bias(models):
    """Through P.self_attention, with zero q and k matrices: queries and keys are rotated
    biases, so the score of (row m, key n) is scale * sum over pairs of
    (qa ka + qb kb) cos(t (m - n)) + (qa kb - qb ka) sin(t (m - n)) with the biases' halves a, b:
    a function of the distance.  Biases added after the rotation would give every pair of rows
    the same score, and the output would be the causal running mean of the values."""
    cfg, w = models["A"]
    hq, hkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["_head_dim"]
    half, group = hd // 2, hq // hkv
    p = "model.layers.0.self_attn."
    w = dict(w)
    w[p + "q_proj.weight"] = np.zeros_like(w[p + "q_proj.weight"])
    w[p + "k_proj.weight"] = np.zeros_like(w[p + "k_proj.weight"])
    r = rng(13)
    w[p + "q_proj.bias"] = r.standard_normal(hq * hd).astype(F32) * F32(1.5)
    w[p + "k_proj.bias"] = r.standard_normal(hkv * hd).astype(F32) * F32(1.5)
    n = 9
    h = r.standard_normal((n, cfg["hidden_size"])).astype(F32) * F32(5.0)
    got = P.self_attention(h, np.arange(n), w, p, cfg)
    # the closed form, in float64
    theta = float(cfg["rope_theta"]) ** (-2.0 * np.arange(half) / hd)
    bq = w[p + "q_proj.bias"].astype(np.float64).reshape(hq, hd)
    bk = w[p + "k_proj.bias"].astype(np.float64).reshape(hkv, hd)
    v = (h.astype(np.float64) @ w[p + "v_proj.weight"].astype(np.float64).T + w[p + "v_proj.bias"]).reshape(n, hkv, hd)
    out = np.zeros((n, hq, hd))
    for hh in range(hq):
        g = hh // group
        qa, qb, ka, kb = bq[hh, :half], bq[hh, half:], bk[g, :half], bk[g, half:]
        for m in range(n):
            d = m - np.arange(m + 1)
            s = ((qa * ka + qb * kb)[None, :] * np.cos(d[:, None] * theta[None, :])
                 + (qa * kb - qb * ka)[None, :] * np.sin(d[:, None] * theta[None, :])).sum(-1) / math.sqrt(hd)
            e = np.exp(s - s.max())
            out[m, hh] = (e / e.sum()) @ v[: m + 1, g]
    want = out.reshape(n, hq * hd) @ w[p + "o_proj.weight"].astype(np.float64).T
    assert np.allclose(got, want, atol=2e-5)
    mean = np.cumsum(v, axis=0) / np.arange(1, n + 1)[:, None, None]
    mean = np.repeat(mean, group, axis=1).reshape(n, hq * hd) @ w[p + "o_proj.weight"].astype(np.float64).T
    assert np.abs(mean - want).max() > 1e-2, "the case cannot tell the orders apart"
    # only distances count: all positions shifted, same output
    assert np.allclose(P.self_attention(h, np.arange(n) + 37, w, p, cfg), got, atol=1e-5)


def test_sharp_models_show_attention_mistakes(models, sharp_folders):
    """What the engine's bfloat16 comparisons can see.  A wrong attention scale (1 for
    1/sqrt(head size) and the like: times 4), a rope base ten times too big, a dropped query bias
    and positions that slip by one each move the plain logits of the "sharp" models by several
    times what the bfloat16 comparisons allow there, in the largest difference and in the root
    mean square; on the models of plain N(0, 0.02) weights most of them hide below the bounds."""
    from helpers import bf16_limits
    mistakes = ("scale", "base", "bias", "position")

    def moved(c, ww, tokens, what, sharp):
        base = P.forward(c, ww, tokens)
        c2, w2 = dict(c), dict(ww)
        att, rope = P.attention, P.rope_neox
        try:
            if what == "scale":
                P.attention = lambda q, k, v, qp, kp, a, b, hd, scale, **kw: att(q, k, v, qp, kp, a, b, hd,
                                                                                 scale * 4.0, **kw)
            elif what == "base":
                c2["rope_theta"] = c["rope_theta"] * 10.0
            elif what == "bias":
                for key in w2:
                    if key.endswith("q_proj.bias"):
                        w2[key] = np.zeros_like(w2[key])
            elif what == "position":
                P.rope_neox = lambda x, pos, *a, **kw: rope(x, [q + (1 if q % 7 == 3 else 0) for q in pos], *a, **kw)
            diff = np.abs(P.forward(c2, w2, tokens) - base)
        finally:
            P.attention, P.rope_neox = att, rope
        bound, rms_bound = bf16_limits(base, sharp)
        return float((diff / bound).max()), float(np.sqrt((diff ** 2).mean())) / rms_bound

    for name in ("A", "B"):
        cfg, w = P.load_model(sharp_folders[name])
        tokens = [int(t) for t in rng(14).integers(0, cfg["vocab_size"], size=65)]
        for what in mistakes:
            by_max, by_rms = moved(cfg, w, tokens, what, True)
            assert by_max > 4.0 and by_rms > 5.0, \
                f"sharp {name}: a wrong {what} is {by_max:.2f} bounds at its largest, {by_rms:.2f} in the mean"
        soft_cfg, soft_w = models[name]
        hidden = [what for what in mistakes if max(moved(soft_cfg, soft_w, tokens, what, False)) < 1.0]
        assert hidden, "the models of plain random weights were expected to hide some of these mistakes"


def test_head_choice_and_causality(models):
    cfg_a, w_a = models["A"]                    # tied: the head is the embedding
    cfg_b, w_b = models["B"]                    # untied
    tokens = [1, 2, 3, 4, 5, 6]
    la = P.forward(cfg_a, w_a, tokens)
    x = w_a["model.embed_tokens.weight"]
    assert la.shape == (6, cfg_a["vocab_size"]) and "lm_head.weight" not in w_a
    lb = P.forward(cfg_b, w_b, tokens)
    swapped = dict(w_b)
    swapped["lm_head.weight"] = w_b["model.embed_tokens.weight"]
    assert not np.allclose(P.forward(cfg_b, swapped, tokens), lb, atol=1e-3)
    # logits at position t do not change when later tokens change
    other = tokens[:3] + [9, 9, 9]
    assert np.array_equal(P.forward(cfg_b, w_b, other)[:3], lb[:3])
    assert not np.allclose(P.forward(cfg_b, w_b, other)[3:], lb[3:], atol=1e-4)
    with pytest.raises(ValueError):
        P.forward(cfg_b, w_b, [cfg_b["vocab_size"]])          # test_nn.cpp:603
    del x


def test_norm_placement(models):
    """The norms stand before the branches: scaling a block's input leaves the attention branch
    unchanged (eps aside) while the residual carries the scale."""
    cfg, w = models["A"]
    cfg = dict(cfg, rms_norm_eps=0.0)
    x = rng(8).standard_normal((4, cfg["hidden_size"])).astype(F32)
    pos = np.arange(4)
    y1 = P.block(x, pos, w, 0, cfg)
    h = P.rms_norm(x, w["model.layers.0.input_layernorm.weight"], 0.0)
    o = P.self_attention(h, pos, w, "model.layers.0.self_attn.", cfg)
    h3 = P.rms_norm(x * F32(3.0), w["model.layers.0.input_layernorm.weight"], 0.0)
    assert np.allclose(h, h3, atol=1e-5)
    x1 = o + x
    f = P.rms_norm(x1, w["model.layers.0.post_attention_layernorm.weight"], 0.0)
    y = P.swiglu(f, w["model.layers.0.mlp.gate_proj.weight"], w["model.layers.0.mlp.up_proj.weight"],
                 w["model.layers.0.mlp.down_proj.weight"]) + x1
    assert np.allclose(y1, y, atol=1e-6)


def test_greedy_stops_after_the_stop_token(models):
    cfg, w = models["A"]
    free = P.greedy(cfg, w, [5, 6, 7], 6)
    assert len(free) == 6
    stopped = P.greedy(cfg, w, [5, 6, 7], 6, stop=(free[2],))
    assert stopped == free[:free.index(free[2]) + 1]
    assert P.argmax(np.array([0.5, 0.5, 0.1])) == 0             # ties to the lowest id


def test_attention_in_blocks_of_rows_is_the_plain_attention():
    """The form that long sequences use: the same numbers as the loop over rows (the row sums of
    the exponentials may round differently by an ulp: numpy sums a row of a matrix pairwise as it
    sums a vector, so they do not)."""
    rng = np.random.default_rng(12)
    for n, hq, hkv, hd in ((70, 4, 2, 16), (300, 3, 1, 32), (129, 2, 2, 8)):
        q, k, v = (rng.standard_normal((n, h * hd)).astype(np.float32) * 1.5 for h in (hq, hkv, hkv))
        pos = np.arange(n)
        want = P.attention(q, k, v, pos, pos, hq, hkv, hd, 0.3)
        for rows in (1, 64, 1000):
            got = P.attention_causal_blocked(q, k, v, hq, hkv, hd, 0.3, rows_at_once=rows)
            assert np.allclose(got, want, rtol=0, atol=2e-6), np.abs(got - want).max()

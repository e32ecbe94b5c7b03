"""A plain, slow implementation of the Qwen2.5 dense decoder.

Whole sequences, no cache, one function per part, NumPy only.  It shares no
code with ``sonicboom_amd``: it reads ``config.json`` with :mod:`json` and the
weights with the ``safetensors`` package, and every formula is written from the
reference's CPU kernels (cited file:line, all under ``/root/reference``).

Arithmetic follows the reference's default CPU mode: activations are float32,
dot products and the mean of squares accumulate in float64 and are rounded to
float32 once (``core/src/nn/cpu_reduce.h:55-57``, ``:75-80``).  The reference
rounds cached K and V through fp16 (``core/src/model/emit.cpp:291-293``); that
is a storage choice of its cache and is left out here, as the engine's 32-bit
path keeps K and V unrounded.
"""
from __future__ import annotations

import json
import math
import os

import numpy as np

F32 = np.float32
F64 = np.float64


# --------------------------------------------------------------------------
# parts
# --------------------------------------------------------------------------
def embedding(table: np.ndarray, tokens) -> np.ndarray:
    """x0[t, :] = E[token[t], :]; no sqrt(width) scale for Qwen2.

    core/src/model/emit.cpp:237-248 (scale only when ``scale_embedding``),
    core/src/model/recipe.cpp:65-70 (Qwen2 leaves ``scale_embedding`` false),
    core/src/nn/embedding.cpp:23-28 (row lookup).
    """
    tokens = np.asarray(tokens, dtype=np.int64)
    if tokens.size and (tokens.min() < 0 or tokens.max() >= table.shape[0]):
        raise ValueError("token id out of range")
    return table[tokens].astype(F32)


def rms_norm(x: np.ndarray, weight, eps: float) -> np.ndarray:
    """y_i = (x_i * inv) * w_i with inv = 1 / sqrt(mean(x^2) + eps).

    core/src/nn/norm.cpp:25-42: eps is added to the mean inside the square
    root, the product order is (x*inv)*w, the weight multiplies as it is.
    core/src/nn/cpu_reduce.h:55-57: each x*x is a float32 product, summed in
    float64, the mean is rounded to float32.
    """
    x = np.asarray(x, dtype=F32)
    sq = (x * x).astype(F32).astype(F64)
    mean = (sq.sum(axis=-1, keepdims=True) / F64(x.shape[-1])).astype(F32)
    inv = (F32(1.0) / np.sqrt(mean + F32(eps), dtype=F32)).astype(F32)
    y = (x * inv).astype(F32)
    if weight is not None:
        y = (y * np.asarray(weight, dtype=F32)).astype(F32)
    return y


def linear(x: np.ndarray, weight: np.ndarray, bias=None) -> np.ndarray:
    """y[o] = sum_i W[o, i] x[i], then y += b.

    core/include/sonicboom/quant/quantized_matmul.h:74-77 (W is [out, in] row
    major), core/src/nn/cpu_reduce.h:75-80 (float64 accumulation, one rounding),
    core/src/nn/elementwise.cpp:52-59 (add_bias is a separate float32 add).
    """
    y = (np.asarray(x, dtype=F64) @ np.asarray(weight, dtype=F64).T).astype(F32)
    if bias is not None:
        y = (y + np.asarray(bias, dtype=F32)).astype(F32)
    return y


def rope_neox(x: np.ndarray, positions, head_dim: int, base: float,
              rot_dims: int = 0, freq_factors=None) -> np.ndarray:
    """Rotate pairs (i, i + half) of every head of ``x`` [n, heads*head_dim].

    core/src/nn/rope.cpp:26-56: theta_i = float(pos) * expf(-2 i / n * logf(base))
    (divided by freq_factors[i] when a table exists), then
    (x_i, x_{i+half}) <- (x_i c - x_{i+half} s, x_i s + x_{i+half} c), all in
    float32.  core/src/nn/rope.cpp:58-83: the leading ``rot_dims`` values of
    each head rotate (0 = the whole head) and n is that width.
    """
    x = np.array(x, dtype=F32, copy=True)
    n_rows = x.shape[0]
    heads = x.shape[1] // head_dim
    dims = head_dim if rot_dims == 0 else rot_dims
    if dims % 2 or dims > head_dim or dims == 0:
        raise ValueError("rotary width must be even and at most head_dim")
    half = dims // 2
    log_base = np.log(F32(base)).astype(F32)
    i = np.arange(half, dtype=F32)
    expo = (F32(-2.0) * i / F32(dims)).astype(F32)
    inv = np.exp((expo * log_base).astype(F32)).astype(F32)          # [half]
    pos = np.asarray(positions, dtype=np.int64).astype(F32)[:, None]  # [n, 1]
    theta = (pos * inv[None, :]).astype(F32)
    if freq_factors is not None:
        theta = (theta / np.asarray(freq_factors, dtype=F32)[None, :half]).astype(F32)
    c = np.cos(theta).astype(F32)[:, None, :]
    s = np.sin(theta).astype(F32)[:, None, :]
    xv = x.reshape(n_rows, heads, head_dim)
    x0 = xv[:, :, :half].copy()
    x1 = xv[:, :, half:dims].copy()
    xv[:, :, :half] = (x0 * c - x1 * s).astype(F32)
    xv[:, :, half:dims] = (x0 * s + x1 * c).astype(F32)
    return xv.reshape(n_rows, heads * head_dim)


def softmax(x: np.ndarray) -> np.ndarray:
    """core/src/nn/softmax.cpp: exp(x - max) / sum, float32."""
    x = np.asarray(x, dtype=F32)
    e = np.exp((x - x.max()).astype(F32)).astype(F32)
    return (e / e.sum(dtype=F32)).astype(F32)


def attention(q: np.ndarray, k: np.ndarray, v: np.ndarray, q_positions,
              k_positions, n_heads_q: int, n_heads_kv: int, head_dim: int,
              scale: float, causal: bool = True, window: int = 0) -> np.ndarray:
    """Grouped-query attention of rows q over keys k, values v.

    core/src/nn/attention.cpp:26-105: query head h reads kv head h // group;
    s_j = dot(q, k_j) * scale; key j is hidden when (causal and j > i) or
    (window > 0 and i >= j + window); m = max, e_j = exp(s_j - m),
    p_j = e_j * (1 / sum e), out = sum_j p_j v_j; a row with no visible key
    is zero (:74-78).  Positions here are absolute, so i and j are the
    positions of the query row and of the key.
    """
    if n_heads_q % n_heads_kv:
        raise ValueError("query heads must be a multiple of kv heads")
    group = n_heads_q // n_heads_kv
    nq, nk = q.shape[0], k.shape[0]
    qv = np.asarray(q, dtype=F32).reshape(nq, n_heads_q, head_dim)
    kv = np.asarray(k, dtype=F32).reshape(nk, n_heads_kv, head_dim)
    vv = np.asarray(v, dtype=F32).reshape(nk, n_heads_kv, head_dim)
    qp = np.asarray(q_positions, dtype=np.int64)
    kp = np.asarray(k_positions, dtype=np.int64)
    out = np.zeros((nq, n_heads_q, head_dim), dtype=F32)
    for i in range(nq):
        hidden = np.zeros(nk, dtype=bool)
        if causal:
            hidden |= kp > qp[i]
        if window > 0:
            hidden |= qp[i] >= kp + window
        vis = ~hidden
        if not vis.any():
            continue
        for h in range(n_heads_q):
            kh = h // group
            s = (kv[vis, kh, :].astype(F64) @ qv[i, h, :].astype(F64)).astype(F32)
            s = (s * F32(scale)).astype(F32)
            m = s.max()
            e = np.exp((s - m).astype(F32)).astype(F32)
            inv = F32(1.0) / e.sum(dtype=F32)
            p = (e * inv).astype(F32)
            out[i, h, :] = (p.astype(F64) @ vv[vis, kh, :].astype(F64)).astype(F32)
    return out.reshape(nq, n_heads_q * head_dim)


def attention_causal_blocked(q: np.ndarray, k: np.ndarray, v: np.ndarray, n_heads_q: int, n_heads_kv: int,
                             head_dim: int, scale: float, rows_at_once: int = 256) -> np.ndarray:
    """:func:`attention` for the one case that long sequences need (row i at position i over keys
    0..i, no window), a block of rows at a time with matrix products instead of a loop over rows:
    the same formula and the same precisions (float64 sums rounded once, float32 scores, maximum,
    exponentials and weights), thousands of times faster.  tests/test_plain.py holds it to
    :func:`attention`."""
    group = n_heads_q // n_heads_kv
    n = q.shape[0]
    qv = np.asarray(q, dtype=F32).reshape(n, n_heads_q, head_dim)
    kv = np.asarray(k, dtype=F32).reshape(n, n_heads_kv, head_dim).astype(F64)
    vv = np.asarray(v, dtype=F32).reshape(n, n_heads_kv, head_dim).astype(F64)
    out = np.zeros((n, n_heads_q, head_dim), dtype=F32)
    for r0 in range(0, n, rows_at_once):
        r1 = min(n, r0 + rows_at_once)
        hidden = np.arange(r1)[None, :] > np.arange(r0, r1)[:, None]
        for h in range(n_heads_q):
            kh = h // group
            s = (qv[r0:r1, h, :].astype(F64) @ kv[:r1, kh, :].T).astype(F32)
            s = (s * F32(scale)).astype(F32)
            s[hidden] = -np.inf
            e = np.exp((s - s.max(axis=1, keepdims=True)).astype(F32)).astype(F32)
            inv = F32(1.0) / e.sum(axis=1, keepdims=True, dtype=F32)
            p = (e * inv).astype(F32)
            out[r0:r1, h, :] = (p.astype(F64) @ vv[:r1, kh, :]).astype(F32)
    return out.reshape(n, n_heads_q * head_dim)


def silu(x: np.ndarray) -> np.ndarray:
    """core/src/nn/activation.cpp:41-50: x / (1 + exp(-x)) in float32."""
    x = np.asarray(x, dtype=F32)
    with np.errstate(over="ignore"):
        return (x / (F32(1.0) + np.exp(-x).astype(F32))).astype(F32)


def swiglu(f: np.ndarray, w_gate, w_up, w_down) -> np.ndarray:
    """u = Wup f; g = silu(Wgate f); y = Wdown (g * u).

    core/src/model/emit.cpp:364-374; core/src/nn/elementwise.cpp:23-27 (mul).
    """
    u = linear(f, w_up)
    g = silu(linear(f, w_gate))
    return linear((g * u).astype(F32), w_down)


def rope_scaling(cfg: dict):
    """(freq_factors or None, multiplier of the attention scores) from config.json's
    ``rope_scaling`` {type|rope_type, factor, original_max_position_embeddings,
    beta_fast, beta_slow, attention_factor}.

    core/src/model/loader.cpp:226-311: theta(i) = pos * base^(-2i/d) / ff[i] with
    ff[i] = 1/alpha(i); linear: alpha = 1/factor; YaRN: alpha = fs (1 - ramp) + ramp
    with ramp(i) = 1 - clamp((i - lo) / max(0.001, hi - lo), 0, 1),
    corr(beta) = d ln(orig / (2 pi beta)) / (2 ln base), lo = max(0, floor(corr(beta_fast))),
    hi = min(d - 1, ceil(corr(beta_slow))); YaRN multiplies the scores by m^2,
    m = (1 + 0.1 ln factor) * attention_factor for factor > 1.
    """
    rs = cfg.get("rope_scaling")
    if not rs:
        return None, 1.0
    kind = rs.get("rope_type", rs.get("type"))
    if kind in (None, "none", "default"):
        return None, 1.0
    d = cfg["_head_dim"]
    base = float(cfg["rope_theta"])
    factor = float(rs["factor"])
    fs = 1.0 / factor
    ff = []
    if kind == "linear":
        return [F32(factor)] * (d // 2), 1.0
    assert kind == "yarn", kind
    orig = rs.get("original_max_position_embeddings", cfg.get("max_position_embeddings"))
    corr = lambda beta: d * math.log(orig / (beta * 2.0 * math.pi)) / (2.0 * math.log(base))  # noqa: E731
    lo = max(0.0, math.floor(corr(float(rs.get("beta_fast", 32.0)))))
    hi = min(d - 1.0, math.ceil(corr(float(rs.get("beta_slow", 1.0)))))
    for i in range(d // 2):
        y = (i - lo) / max(0.001, hi - lo)
        ramp = 1.0 - min(1.0, max(0.0, y))
        alpha = fs * (1.0 - ramp) + ramp
        ff.append(F32(1.0 / alpha))
    m = (1.0 if factor <= 1.0 else 1.0 + 0.1 * math.log(factor)) * float(rs.get("attention_factor", 1.0))
    return ff, float(F32(m * m))


def self_attention(h: np.ndarray, positions, w: dict, prefix: str, cfg: dict) -> np.ndarray:
    """q = Wq h + bq, rotated; k = Wk h + bk, rotated; v = Wv h + bv;
    causal GQA with scale 1/sqrt(head_dim); o = Wo attn (no bias).

    core/src/model/emit.cpp:255-308 (both matmuls, both biases, the bias
    precedes the rotation, V is not rotated, the output projection has no
    bias for Qwen2), core/src/model/recipe.cpp:65-70 and :153-167 (q/k/v bias,
    score scale 1/sqrt(head_dim)), core/src/model/loader.cpp:656-671, :945 (head_dim
    = width / heads, every layer global: no window).
    """
    hq, hkv, hd = cfg["num_attention_heads"], cfg["num_key_value_heads"], cfg["_head_dim"]
    q = linear(h, w[prefix + "q_proj.weight"], w[prefix + "q_proj.bias"])
    k = linear(h, w[prefix + "k_proj.weight"], w[prefix + "k_proj.bias"])
    v = linear(h, w[prefix + "v_proj.weight"], w[prefix + "v_proj.bias"])
    ff, score_mult = rope_scaling(cfg)
    q = rope_neox(q, positions, hd, cfg["rope_theta"], freq_factors=ff)
    k = rope_neox(k, positions, hd, cfg["rope_theta"], freq_factors=ff)
    # core/src/model/recipe.cpp:165-167: the architecture's 1/sqrt(head_dim) times YaRN's magnitude term
    scale = F32(F32(1.0) / np.sqrt(F32(hd))) * F32(score_mult)
    pos = np.asarray(positions)
    if len(pos) > 4096 and np.array_equal(pos, np.arange(len(pos))):
        a = attention_causal_blocked(q, k, v, hq, hkv, hd, float(scale))     # the same, in blocks of rows
    else:
        a = attention(q, k, v, positions, positions, hq, hkv, hd, float(scale),
                      causal=True, window=0)
    return linear(a, w[prefix + "o_proj.weight"])


def block(x: np.ndarray, positions, w: dict, layer: int, cfg: dict) -> np.ndarray:
    """x1 = attn(norm(x)) + x;  x2 = ffn(norm(x1)) + x1.

    core/src/model/emit.cpp:436-459: pre-norms only for Qwen2, operand order of
    the adds is (branch, residual).
    """
    p = f"model.layers.{layer}."
    eps = cfg["rms_norm_eps"]
    h = rms_norm(x, w[p + "input_layernorm.weight"], eps)
    o = self_attention(h, positions, w, p + "self_attn.", cfg)
    x1 = (o + x).astype(F32)
    f = rms_norm(x1, w[p + "post_attention_layernorm.weight"], eps)
    y = swiglu(f, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
               w[p + "mlp.down_proj.weight"])
    return (y + x1).astype(F32)


def lm_head(x: np.ndarray, w: dict, cfg: dict) -> np.ndarray:
    """logits = Wout rmsnorm(x); the head is the embedding matrix when the
    model ties them or the file has no separate head.

    core/src/model/emit.cpp:512-524 (final norm, output matmul, no softcap for
    Qwen2), core/src/model/exec.cpp:516-517 (fall back to token_embd).
    """
    hn = rms_norm(x, w["model.norm.weight"], cfg["rms_norm_eps"])
    if cfg.get("tie_word_embeddings", False) or "lm_head.weight" not in w:
        head = w["model.embed_tokens.weight"]
    else:
        head = w["lm_head.weight"]
    return linear(hn, head)


# --------------------------------------------------------------------------
# the model
# --------------------------------------------------------------------------
def load_model(folder: str):
    """config.json as a dict (plus the derived ``_head_dim``) and the tensors of
    model.safetensors as float32 arrays."""
    from safetensors import safe_open

    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    cfg["_head_dim"] = cfg["hidden_size"] // cfg["num_attention_heads"]
    w = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            w[name] = f.get_tensor(name).float().numpy()
    return cfg, w


def forward(cfg: dict, w: dict, tokens) -> np.ndarray:
    """Logits [n, vocab] of one whole sequence, positions 0..n-1."""
    positions = np.arange(len(tokens), dtype=np.int64)
    x = embedding(w["model.embed_tokens.weight"], tokens)
    for layer in range(cfg["num_hidden_layers"]):
        x = block(x, positions, w, layer, cfg)
    return lm_head(x, w, cfg)


def greedy(cfg: dict, w: dict, prompt, n_new: int, stop=()):
    """Greedy continuation, the whole sequence recomputed for every token.
    The stop token is emitted and ends the sequence
    (core/src/model/gemma4_plan.cpp:1631-1637, :1770-1774)."""
    seq = list(prompt)
    out = []
    for _ in range(n_new):
        logits = forward(cfg, w, seq)[-1]
        t = argmax(logits)
        out.append(t)
        seq.append(t)
        if t in stop:
            break
    return out


def argmax(x) -> int:
    """core/src/nn/sampling.cpp:238-244: first maximum wins."""
    x = np.asarray(x)
    best = 0
    for i in range(1, x.shape[0]):
        if x[i] > x[best]:
            best = i
    return best

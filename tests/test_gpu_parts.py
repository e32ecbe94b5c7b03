"""Each part alone against the plain implementation's function of the same part, at sizes
other than the tiny models'; then architectures that exist only in this file — a mixer with
per-sequence state, another position encoding, windowed layers with a cache group of their
own, a layer that reads another layer's cache, a layer that runs twice — registered, built
and stepped without a change to the framework's files."""
import math

import numpy as np
import pytest
import torch

from plain import qwen2_plain as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
F32, BF16 = torch.float32, torch.bfloat16
TOL = {F32: dict(atol=3e-5, rtol=1e-4), BF16: dict(atol=3e-2, rtol=3e-2)}


def runtime(dtype):
    from sonicboom_amd.parts import Runtime
    return Runtime(torch.device(DEV), dtype, True)


def rand(*shape, scale=1.0, seed=0, dtype=F32):
    g = torch.Generator().manual_seed(seed + 13 * len(shape) + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def tensors_for(spec, dtype, seed=0, scale=0.08):
    """Random tensors for every tensor a part spec names; returns (device dict, float64 numpy dict)."""
    dev, ref = {}, {}
    for i, t in enumerate(spec.all_tensors()):
        mean = t.init[0]
        a = (rand(*t.shape, scale=scale, seed=seed + i) + mean).to(dtype)
        dev[t.name] = a.to(DEV)
        ref[t.name] = a.float().numpy()
    return dev, ref


def close(got, want, dtype, what=""):
    got = got.detach().float().cpu().numpy().astype(np.float64)
    want = np.asarray(want, dtype=np.float64)
    tol = TOL[dtype]
    scale = max(1.0, np.abs(want).max())
    err = np.abs(got - want)
    assert got.shape == want.shape and (err <= tol["atol"] * scale + tol["rtol"] * np.abs(want)).all(), \
        f"{what}: max |diff| {err.max():.3g}"


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_norm_embedding_head_alone(dtype):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.embedding import embedding_spec, head_spec
    from sonicboom_amd.parts.norm import rmsnorm_spec
    rt = runtime(dtype)
    spec = rmsnorm_spec("n.weight", 200, 3e-4)
    dev, ref = tensors_for(spec, dtype)
    x = rand(6, 200, scale=2.0)
    got = build_part(spec, dev, rt).forward(x.to(DEV), dtype)
    close(got, P.rms_norm(x.numpy(), ref["n.weight"], 3e-4), dtype, "norm")
    espec, hspec = embedding_spec("e.weight", 90, 40), head_spec("e.weight", 90, 40)     # a tied pair
    dev, ref = tensors_for(espec, dtype, scale=1.0)
    ids = torch.tensor([0, 89, 3, 3], dtype=torch.int32, device=DEV)
    emb = build_part(espec, dev, rt).forward(ids)
    assert emb.dtype == F32 and np.array_equal(emb.cpu().numpy(), P.embedding(ref["e.weight"], [0, 89, 3, 3]))
    h = rand(5, 40).to(dtype)
    logits = build_part(hspec, dev, rt).forward(h.to(DEV))
    assert logits.dtype == F32
    close(logits, P.linear(h.float().numpy(), ref["e.weight"]), dtype, "head")


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_feed_forward_alone(dtype):
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.ffn import gated_ffn_spec
    spec = gated_ffn_spec("m.", 72, 200)
    dev, ref = tensors_for(spec, dtype)
    ffn = build_part(spec, dev, runtime(dtype))
    for rows in (3, 70):                        # the weight-streaming and the tiled kernels
        h, x = rand(rows, 72).to(dtype), rand(rows, 72, seed=5)
        xd = x.to(DEV)
        ffn.forward(h.to(DEV), xd, None)
        want = P.swiglu(h.float().numpy(), ref["m.gate_proj.weight"], ref["m.up_proj.weight"],
                        ref["m.down_proj.weight"]) + x.numpy()
        close(xd, want, dtype, f"ffn rows={rows}")


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_feed_forward_with_a_gelu_gate(dtype):
    """The gate's activation is a constant of the part: the same feed-forward with the tanh form
    of GELU, in 32-bit (product, then the activation kernel) and bfloat16 (fused epilogues)."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.ffn import gated_ffn_spec
    spec = gated_ffn_spec("m.", 72, 200, activation="gelu_tanh")
    dev, ref = tensors_for(spec, dtype)
    ffn = build_part(spec, dev, runtime(dtype))
    for rows in (3, 70):
        h, x = rand(rows, 72).to(dtype), rand(rows, 72, seed=5)
        xd = x.to(DEV)
        ffn.forward(h.to(DEV), xd, None)
        f = h.float().numpy()
        g, u = P.linear(f, ref["m.gate_proj.weight"]), P.linear(f, ref["m.up_proj.weight"])
        gelu = 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * g * (1.0 + 0.044715 * g * g)))
        want = P.linear((gelu * u).astype(np.float32), ref["m.down_proj.weight"]) + x.numpy()
        close(xd, want, dtype, f"gelu ffn rows={rows}")
        silu = P.swiglu(f, ref["m.gate_proj.weight"], ref["m.up_proj.weight"], ref["m.down_proj.weight"]) + x.numpy()
        assert np.abs(silu - want).max() > 1e-3          # not the SiLU result
    with pytest.raises(ValueError, match="unknown activation"):
        build_part(gated_ffn_spec("m.", 72, 200, activation="relu"), dev, runtime(dtype))


def run_mixer(mixer, rt, h_rows, cuts, width):
    """Feed rows of one sequence to a mixer in the given cuts; returns what it added to a zero stream."""
    from sonicboom_amd.cache import PagedCache, group_entries
    from sonicboom_amd.engine.model import LayerBinding
    from sonicboom_amd.engine.step import StepContext, StepEntry
    cs = mixer.cache_spec()
    cache = PagedCache(group_entries({0: (cs.kv_heads, cs.head_dim, cs.window)}), 64 * 8, rt.cache_dtype, rt.device)
    k, v, g = cache.entry_views(0)
    binding = LayerBinding(0, g, k, v, True, None)
    slot = cache.alloc_slot()
    outs, start = [], 0
    for n in cuts:
        entries = [StepEntry(slot, [0] * n, ())]
        cache.reserve([slot], [n])
        ctx = StepContext(cache, entries, rt.device, mixer.row_tile)
        x = torch.zeros((n, width), dtype=F32, device=DEV)
        mixer.forward(h_rows[start:start + n].to(DEV).contiguous(), x, ctx, binding)
        cache.advance([slot], [n])
        outs.append(x)
        start += n
    return torch.cat(outs)


@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("hq, hkv, hd, window, rot", [(5, 1, 16, 0, 0), (6, 3, 48, 40, 0), (4, 4, 32, 0, 16)])
def test_attention_mixer_alone(dtype, hq, hkv, hd, window, rot):
    """Whole, and cut into steps: prompt, more rows on top of the cache, single rows."""
    from sonicboom_amd.parts import build_part
    from sonicboom_amd.parts.attention import attention_spec
    from sonicboom_amd.parts.position import rope_spec
    width, n = 88, 100
    ff = [1.0 + 0.1 * i for i in range((rot or hd) // 2)]
    spec = attention_spec("a.", width, hq, hkv, hd, rope_spec(hd, 5e4, rot, ff, 1.3), window=window, out_bias=True)
    dev, ref = tensors_for(spec, dtype)
    rt = runtime(dtype)
    mixer = build_part(spec, dev, rt)
    h = rand(n, width).to(dtype)
    hn = h.float().numpy()
    pos = np.arange(n)
    q = P.rope_neox(P.linear(hn, ref["a.q_proj.weight"], ref["a.q_proj.bias"]), pos, hd, 5e4, rot, ff)
    k = P.rope_neox(P.linear(hn, ref["a.k_proj.weight"], ref["a.k_proj.bias"]), pos, hd, 5e4, rot, ff)
    v = P.linear(hn, ref["a.v_proj.weight"], ref["a.v_proj.bias"])
    scale = float(np.float32(1 / math.sqrt(hd)) * np.float32(1.3))
    a = P.attention(q, k, v, pos, pos, hq, hkv, hd, scale, True, window)
    want = P.linear(a, ref["a.o_proj.weight"], ref["a.o_proj.bias"])
    for cuts in ([n], [70, 20] + [1] * 10):
        close(run_mixer(mixer, rt, h, cuts, width), want, dtype, f"cuts {cuts[:3]}")


# ----------------------------------------------------------------------------------------------
# architectures that live in this file only
# ----------------------------------------------------------------------------------------------
def register_toys():
    from sonicboom_amd import ops
    from sonicboom_amd.config import register_architecture
    from sonicboom_amd.parts import Mixer, StateSpec, register_part
    from sonicboom_amd.parts.position import Position

    @register_part("mixer", "toy_decay")
    class DecayMixer(Mixer):
        """s <- a * s + W_in h_t;  x_t += W_out s.  State of its own: one vector per sequence."""

        def __init__(self, spec, tensors, parts, rt):
            super().__init__(spec, tensors, parts, rt)
            self.a = float(spec.params["decay"])
            self.inner = int(spec.params["inner"])
            self.w_in, self.w_out = tensors["w_in"].float(), tensors["w_out"].float()

        def state_spec(self):
            return StateSpec((self.inner,), torch.float32)

        def forward(self, h, x, ctx, binding):
            u = h.float() @ self.w_in.T                    # a toy may use torch; it is no product path
            row = 0
            for slot, n in zip(ctx.slot_list, ctx.n_new):  # rows of a sequence in order
                s = binding.state[slot]
                for r in range(row, row + n):
                    s.mul_(self.a).add_(u[r])
                    x[r] += self.w_out @ s
                row += n

    from sonicboom_amd.cache import PAGE
    from sonicboom_amd.parts import RowsSpec

    @register_part("mixer", "toy_latent")
    class LatentMixer(Mixer):
        """Keeps one compressed row c_t = W_c h_t per token in the cache (no heads, no values) and
        adds W_o times the mean of the rows of the last ``window`` tokens (of all, if 0)."""

        def __init__(self, spec, tensors, parts, rt):
            super().__init__(spec, tensors, parts, rt)
            self.rank, self.window = int(spec.params["rank"]), int(spec.params["window"])
            self.w_c, self.w_o = tensors["w_c"].float(), tensors["w_o"].float()

        def cache_spec(self):
            return RowsSpec((self.rank,), self.window)

        def forward(self, h, x, ctx, binding):
            rows, table = binding.k_cache, ctx.page_table(binding.group).long()      # [pages, PAGE, rank]
            assert binding.v_cache is None and tuple(rows.shape[1:]) == (PAGE, self.rank)
            pos = ctx.row_pos.long()
            if binding.writes_cache:
                c = (h.float() @ self.w_c.T).to(rows.dtype)
                rows[table[ctx.row_seq.long(), pos // PAGE], pos % PAGE] = c
            row = 0
            for i, n in enumerate(ctx.n_new):
                for r in range(row, row + n):
                    last = int(ctx.host_row_pos[r])
                    idx = torch.arange(max(0, last - self.window + 1) if self.window else 0, last + 1, device=x.device)
                    x[r] += self.w_o @ rows[table[i, idx // PAGE], idx % PAGE].float().mean(0)
                row += n

    @register_part("position", "toy_alibi_free_shift")
    class ShiftPosition(Position):
        """Not rotary: adds position * slope to the first element of every query and key head."""

        def __init__(self, spec, tensors, parts, rt):
            super().__init__(spec, tensors, parts, rt)
            self.slope = float(spec.params["slope"])

        def rotary_tables(self):
            return None

        def apply(self, qkv, ctx, heads_q, heads_kv, head_dim):
            pos = ctx.row_pos.float() * self.slope
            view = qkv.view(qkv.shape[0], -1, head_dim)
            view[:, :heads_q + heads_kv, 0] += pos[:, None]

    from sonicboom_amd.parts import Part

    @register_part("ffn", "toy_routed")
    class RoutedFFN(Part):
        """Every row goes to the ``top`` experts whose router logits are largest, and gets their
        outputs weighted by the softmax over those logits (float32).  The experts are nested
        parts of the framework's own dense kind; the routing is torch on the host's terms."""
        category = "ffn"

        def __init__(self, spec, tensors, parts, rt):
            super().__init__(spec, tensors, parts, rt)
            self.top = int(spec.params["top"])
            self.router = tensors["router"].float()
            self.experts = [parts[f"expert{i}"] for i in range(int(spec.params["n_experts"]))]

        def forward(self, h, x, ctx):
            logits = h.float() @ self.router.T
            best, which = torch.topk(logits, self.top, dim=-1)
            share = torch.softmax(best, dim=-1)
            for e, expert in enumerate(self.experts):
                rows, slot = torch.nonzero(which == e, as_tuple=True)
                if rows.numel() == 0:
                    continue
                out = torch.zeros((rows.numel(), x.shape[1]), dtype=torch.float32, device=x.device)
                expert.forward(h[rows].contiguous(), out, ctx)
                x[rows] += out * share[rows, slot][:, None]

    @register_part("embedding", "toy_learned_positions")
    class PositionedEmbedding(Part):
        """x_t = E[token_t] + P[position_t]: an embedding that reads the step's context."""
        category = "embedding"

        def __init__(self, spec, tensors, parts, rt):
            super().__init__(spec, tensors, parts, rt)
            self.table, self.places = tensors["table"], tensors["places"].float()

        def forward(self, ids, ctx):
            return ops.embed(self.table, ids) + self.places[ctx.row_pos.long()]

    return ops, register_architecture


class ToyConfig:
    def __init__(self, d):
        self.d = dict(d)

    @classmethod
    def from_dict(cls, d):
        for key in ("vocab_size", "width", "layers"):
            if key not in d:
                raise ValueError(f"missing/invalid config key: {key}")
        return cls(d)

    def to_dict(self):
        return dict(self.d)


def toy_spec(cfg):
    from sonicboom_amd.parts import ModelSpec, OrderEntry, PartSpec, TensorSpec
    from sonicboom_amd.parts.attention import attention_spec
    from sonicboom_amd.parts.block import prenorm_block_spec
    from sonicboom_amd.parts.embedding import embedding_spec, head_spec
    from sonicboom_amd.parts.ffn import gated_ffn_spec
    from sonicboom_amd.parts.norm import rmsnorm_spec
    from sonicboom_amd.parts.position import rope_spec
    d, w, v = cfg.d, cfg.d["width"], cfg.d["vocab_size"]
    blocks, order, cache = [], [], 0
    for i, layer in enumerate(d["layers"]):
        p = f"l{i}."
        kind = layer["mixer"]
        if kind == "decay":
            mixer = PartSpec("mixer", "toy_decay", {"decay": layer["decay"], "inner": layer["inner"]}, {
                "w_in": TensorSpec(p + "w_in", (layer["inner"], w)), "w_out": TensorSpec(p + "w_out", (w, layer["inner"]))})
        elif kind == "latent":
            mixer = PartSpec("mixer", "toy_latent", {"rank": layer["rank"], "window": layer.get("window", 0)}, {
                "w_c": TensorSpec(p + "w_c", (layer["rank"], w)), "w_o": TensorSpec(p + "w_o", (w, layer["rank"]))})
        else:
            if layer.get("position") == "shift":
                pos = PartSpec("position", "toy_alibi_free_shift", {"slope": layer["slope"]})
            else:
                pos = rope_spec(layer["head_dim"], layer.get("base", 1e4))
            mixer = attention_spec(p + "attn.", w, layer["heads"], layer["kv_heads"], layer["head_dim"], pos,
                                   window=layer.get("window", 0), qkv_bias=layer.get("bias", True))
        if "experts" in layer:
            ffn = PartSpec("ffn", "toy_routed", {"top": layer["top"], "n_experts": layer["experts"]},
                           {"router": TensorSpec(p + "router", (layer["experts"], w), init=(0.0, 1.0))},
                           {f"expert{e}": gated_ffn_spec(p + f"e{e}.", w, layer["ff"]) for e in range(layer["experts"])})
        else:
            ffn = gated_ffn_spec(p + "mlp.", w, layer["ff"])
        blocks.append(prenorm_block_spec(rmsnorm_spec(p + "n1", w, d["eps"]), mixer,
                                         rmsnorm_spec(p + "n2", w, d["eps"]), ffn))
    for e in d["order"]:
        order.append(OrderEntry(e["block"], e.get("cache"), e.get("writes", True)))
    embedding = embedding_spec("emb", v, w)
    if d.get("learned_positions"):
        embedding = PartSpec("embedding", "toy_learned_positions", {"vocab": v, "width": w}, {
            "table": TensorSpec("emb", (v, w)), "places": TensorSpec("places", (d["learned_positions"], w))})
    return ModelSpec("ToyForCausalLM", w, v, embedding, blocks, order,
                     rmsnorm_spec("norm", w, d["eps"]), head_spec("head", v, w))


def plain_toy(cfg, w, tokens, margins=None):
    """The toy architecture written out with the plain parts: whole sequence, no cache.
    ``margins``: a list that receives, per routed layer, every row's gap between the last chosen
    and the first rejected router logit."""
    d = cfg.d
    n = len(tokens)
    pos = np.arange(n)
    x = P.embedding(w["emb"], tokens)
    if d.get("learned_positions"):
        x = (x + w["places"][pos]).astype(np.float32)
    kv = {}
    for e in d["order"]:
        i = e["block"]
        layer, p = d["layers"][i], f"l{i}."
        h = P.rms_norm(x, w[p + "n1"], d["eps"])
        if layer["mixer"] == "decay":
            s = np.zeros(layer["inner"], np.float32)
            out = np.zeros_like(x)
            u = P.linear(h, w[p + "w_in"])
            for t in range(n):
                s = np.float32(layer["decay"]) * s + u[t]
                out[t] = w[p + "w_out"] @ s
        elif layer["mixer"] == "latent":
            if e.get("writes", True):
                kv[e["cache"]] = P.linear(h, w[p + "w_c"])
            c, win = kv[e["cache"]].astype(np.float64), layer.get("window", 0)
            out = np.stack([w[p + "w_o"].astype(np.float64) @ c[max(0, t - win + 1) if win else 0:t + 1].mean(0)
                            for t in range(n)]).astype(np.float32)
        else:
            hq, hkv, hd = layer["heads"], layer["kv_heads"], layer["head_dim"]
            bias = (lambda nm: w[p + f"attn.{nm}_proj.bias"]) if layer.get("bias", True) else (lambda nm: None)

            def place(a):
                if layer.get("position") == "shift":
                    a = a.copy().reshape(n, -1, hd)
                    a[:, :, 0] += (pos * np.float32(layer["slope"])).astype(np.float32)[:, None]
                    return a.reshape(n, -1)
                return P.rope_neox(a, pos, hd, layer.get("base", 1e4))
            q = place(P.linear(h, w[p + "attn.q_proj.weight"], bias("q")))
            if e.get("writes", True):
                kv[e["cache"]] = (place(P.linear(h, w[p + "attn.k_proj.weight"], bias("k"))),
                                  P.linear(h, w[p + "attn.v_proj.weight"], bias("v")))
            k, v = kv[e["cache"]]
            a = P.attention(q, k, v, pos, pos, hq, hkv, hd, float(np.float32(1 / math.sqrt(hd))), True,
                            layer.get("window", 0))
            out = P.linear(a, w[p + "attn.o_proj.weight"])
        x = (out + x).astype(np.float32)
        f = P.rms_norm(x, w[p + "n2"], d["eps"])
        if "experts" in layer:
            logits = P.linear(f, w[p + "router"]).astype(np.float64)
            order_ = np.argsort(-logits, axis=1, kind="stable")
            top = layer["top"]
            if margins is not None:
                rows = np.arange(n)
                margins.append(logits[rows, order_[:, top - 1]] - logits[rows, order_[:, top]])
            y = np.zeros_like(x, dtype=np.float64)
            for t in range(n):
                chosen = order_[t, :top]
                z = np.exp(logits[t, chosen] - logits[t, chosen].max())
                z /= z.sum()
                for share, e in zip(z, chosen):
                    q = p + f"e{e}."
                    y[t] += share * P.swiglu(f[t:t + 1], w[q + "gate_proj.weight"], w[q + "up_proj.weight"],
                                             w[q + "down_proj.weight"])[0]
            x = (y + x).astype(np.float32)
        else:
            x = (P.swiglu(f, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"],
                          w[p + "mlp.down_proj.weight"]) + x).astype(np.float32)
    return P.linear(P.rms_norm(x, w["norm"], d["eps"]), w["head"])


TOY_STATE = {
    "architectures": ["ToyForCausalLM"], "vocab_size": 120, "width": 48, "eps": 1e-5,
    "layers": [{"mixer": "decay", "decay": 0.9, "inner": 24, "ff": 64},
               {"mixer": "attention", "heads": 3, "kv_heads": 1, "head_dim": 16, "ff": 40, "position": "shift",
                "slope": 0.01, "bias": False}],
    # the decay layer runs twice (each run has its own state), around an attention layer
    "order": [{"block": 0}, {"block": 1, "cache": 0}, {"block": 0}],
}
TOY_WINDOWS = {
    "architectures": ["ToyForCausalLM"], "vocab_size": 150, "width": 64, "eps": 1e-6,
    "layers": [{"mixer": "attention", "heads": 4, "kv_heads": 2, "head_dim": 16, "ff": 96},
               {"mixer": "attention", "heads": 4, "kv_heads": 2, "head_dim": 16, "ff": 80, "window": 50},
               {"mixer": "attention", "heads": 2, "kv_heads": 1, "head_dim": 32, "ff": 72, "window": 70, "base": 5e5}],
    # entry 1 reads entry 0's keys (same heads); block 0 runs a second time with a cache of its own;
    # the two windowed layers have different needs, so three cache groups exist
    "order": [{"block": 0, "cache": 0}, {"block": 0, "cache": 0, "writes": False}, {"block": 1, "cache": 1},
              {"block": 2, "cache": 2}, {"block": 0, "cache": 3}],
}


TOY_LATENT = {
    "architectures": ["ToyForCausalLM"], "vocab_size": 110, "width": 40, "eps": 1e-5,
    "layers": [{"mixer": "latent", "rank": 12, "ff": 48},
               {"mixer": "attention", "heads": 2, "kv_heads": 1, "head_dim": 16, "ff": 56},
               {"mixer": "latent", "rank": 20, "window": 70, "ff": 40}],
    # the first latent layer runs a second time reading the rows of its first run
    "order": [{"block": 0, "cache": 0}, {"block": 1, "cache": 1}, {"block": 2, "cache": 2},
              {"block": 0, "cache": 0, "writes": False}],
}


TOY_ROUTED = {
    "architectures": ["ToyForCausalLM"], "vocab_size": 130, "width": 56, "eps": 1e-5,
    "layers": [{"mixer": "attention", "heads": 2, "kv_heads": 2, "head_dim": 16, "ff": 72},
               # routing sits in the last layer: a row that another rounding would route elsewhere
               # then changes its own logits only, and the test can leave such rows out
               {"mixer": "attention", "heads": 4, "kv_heads": 1, "head_dim": 16, "ff": 24, "experts": 5, "top": 2}],
    "order": [{"block": 0, "cache": 0}, {"block": 1, "cache": 1}],
}


TOY_PLACES = {
    "architectures": ["ToyForCausalLM"], "vocab_size": 140, "width": 48, "eps": 1e-5, "learned_positions": 200,
    # no rotation anywhere: the shift "encoding" with slope 0 leaves queries and keys as they are,
    # so the order of the tokens reaches the model through the embedding alone
    "layers": [{"mixer": "attention", "heads": 3, "kv_heads": 3, "head_dim": 16, "ff": 64, "position": "shift",
                "slope": 0.0}],
    "order": [{"block": 0, "cache": 0}],
}


def build_toy(cfg_dict, dtype, **engine_options):
    from sonicboom_amd.config import architecture_of
    from sonicboom_amd.engine import DecoderModel, Engine
    _, register_architecture = register_toys()
    register_architecture("ToyForCausalLM", ToyConfig, toy_spec)
    arch = architecture_of(cfg_dict)                       # found through the one registry
    cfg = arch.config_class.from_dict(cfg_dict)
    spec = arch.build_spec(cfg)
    dev, ref = tensors_for(spec, dtype, seed=3, scale=0.1)
    model = DecoderModel(spec, dev, runtime(dtype), cfg)
    return cfg, ref, model, Engine(model, max_tokens=64 * 12, **engine_options)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_toy_mixer_with_state_of_its_own(dtype):
    from sonicboom_amd.engine import StepEntry, generate
    from sonicboom_amd.sampling import SamplingParams
    cfg, ref, model, eng = build_toy(TOY_STATE, dtype)
    assert sorted(model.state_specs) == [0, 2] and len(model.groups) == 1
    rng = np.random.default_rng(0)
    a, b = ([int(t) for t in rng.integers(0, 120, size=n)] for n in (30, 75))
    want_a, want_b = plain_toy(cfg, ref, a), plain_toy(cfg, ref, b)
    # prompts of unequal lengths in one step, then token by token; b's slot is reused afterwards
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    out = eng.step([StepEntry(sa, a[:10], range(10)), StepEntry(sb, b[:40], range(40))])
    close(out[:10], want_a[:10], dtype, "toy a prompt")
    close(out[10:], want_b[:40], dtype, "toy b prompt")
    for i in range(20):
        out = eng.step([StepEntry(sa, [a[10 + i]], [0]), StepEntry(sb, [b[40 + i]], [0])])
        close(out[:1], want_a[10 + i:11 + i], dtype, f"toy a token {i}")
        close(out[1:], want_b[40 + i:41 + i], dtype, f"toy b token {i}")
    eng.free_slot(sa)
    eng.free_slot(sb)
    # a slot used again starts from a zero state
    s = eng.alloc_slot()
    assert s in (sa, sb)
    close(eng.step([StepEntry(s, b, range(len(b)))]), want_b, dtype, "toy b whole, on a used slot")
    eng.free_slot(s)
    # the generation loop drives it too (kernel by kernel: the toy is not replayable)
    toks = generate(eng, [a[:5], b[:9]], SamplingParams(max_tokens=6), stop_tokens=())
    assert not eng.decode_loop().use_graph and [len(t) for t in toks] == [6, 6]
    if dtype == F32:
        for prompt, out_t in zip((a[:5], b[:9]), toks):
            logits = plain_toy(cfg, ref, prompt + out_t)
            assert out_t == [int(np.argmax(logits[len(prompt) - 1 + i])) for i in range(6)]


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_windows_shared_cache_and_a_layer_that_runs_twice(dtype):
    from sonicboom_amd.engine import StepEntry
    cfg, ref, model, eng = build_toy(TOY_WINDOWS, dtype)
    needs = sorted((g.kv_heads, g.head_dim, g.window, g.entries) for g in model.groups)
    assert needs == [(1, 32, 70, (2,)), (2, 16, 0, (0, 3)), (2, 16, 50, (1,))]
    rng = np.random.default_rng(1)
    tokens = [int(t) for t in rng.integers(0, 150, size=300)]
    want = plain_toy(cfg, ref, tokens)
    s = eng.alloc_slot()
    got = [eng.step([StepEntry(s, tokens[:130], range(130))])]
    got.append(eng.step([StepEntry(s, tokens[130:200], range(70))]))       # more rows on top of the cache
    for t in tokens[200:]:
        got.append(eng.step([StepEntry(s, [t], [0])]))
    close(torch.cat(got), want, dtype, "windows and shared cache")
    # the windowed groups have given back the pages their windows left
    held = {g.window: eng.cache.held_pages(i) for i, g in enumerate(eng.cache.groups)}
    assert held[0] == 5 and held[50] <= 2 and held[70] <= 3
    eng.free_slot(s)
    assert all(eng.cache.held_pages(i) == 0 for i in range(3))


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_toy_mixer_that_caches_rows_of_its_own_shape(dtype):
    """A mixer that keeps a compressed row per token instead of keys and values of heads, defined
    above in this file: its `cache_spec` names the row's shape and a window, the cache gives it
    pages of such rows in groups of their own beside the attention layer's keys and values, a
    second run of the layer reads the first run's rows, and the windowed group gives pages back."""
    from sonicboom_amd.engine import StepEntry
    cfg, ref, model, eng = build_toy(TOY_LATENT, dtype)
    needs = sorted((g.row_shape, g.kv_heads, g.head_dim, g.window, g.entries) for g in model.groups)
    assert needs == [((), 1, 16, 0, (1,)), ((12,), 0, 0, 0, (0,)), ((20,), 0, 0, 70, (2,))]
    rng = np.random.default_rng(5)
    a, b = ([int(t) for t in rng.integers(0, 110, size=n)] for n in (230, 90))
    want_a, want_b = plain_toy(cfg, ref, a), plain_toy(cfg, ref, b)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    out = eng.step([StepEntry(sa, a[:130], range(130)), StepEntry(sb, b[:50], range(50))])
    close(out[:130], want_a[:130], dtype, "latent a prompt")
    close(out[130:], want_b[:50], dtype, "latent b prompt")
    out = eng.step([StepEntry(sa, a[130:200], range(70))])                  # more rows on top of the cache
    close(out, want_a[130:200], dtype, "latent a, second piece")
    for i in range(30):
        out = eng.step([StepEntry(sa, [a[200 + i]], [0]), StepEntry(sb, [b[50 + i]], [0])])
        close(out[:1], want_a[200 + i:201 + i], dtype, f"latent a token {i}")
        close(out[1:], want_b[50 + i:51 + i], dtype, f"latent b token {i}")
    held = {g.row_shape: eng.cache.held_pages(i) for i, g in enumerate(eng.cache.groups)}
    assert held[(12,)] == 4 + 2 and held[(20,)] <= 3 + 2          # a: 230 tokens, b: 80
    eng.free_slot(sa)
    eng.free_slot(sb)
    assert all(eng.cache.held_pages(i) == 0 for i in range(3))
    s = eng.alloc_slot()                                          # used pages, used slot
    close(eng.step([StepEntry(s, b, range(len(b)))]), want_b, dtype, "latent b whole, on a used slot")
    eng.free_slot(s)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_toy_feed_forward_with_routing(dtype):
    """A feed-forward that routes every row to two of five experts, defined above in this file
    from a router tensor and five nested parts of the framework's dense kind: registered, built
    from its spec, loaded by tensor name and stepped (whole, cut, and two sequences at once)
    without a change to the framework."""
    from sonicboom_amd.engine import StepEntry
    cfg, ref, model, eng = build_toy(TOY_ROUTED, dtype)
    assert not eng.decode_loop().use_graph              # the toy routes with host control flow
    rng = np.random.default_rng(4)
    a, b = ([int(t) for t in rng.integers(0, 130, size=n)] for n in (90, 41))
    gaps_a, gaps_b = [], []
    want_a, want_b = plain_toy(cfg, ref, a, gaps_a), plain_toy(cfg, ref, b, gaps_b)
    # rows whose routing hangs on less than the rounding of the path are left out
    least = 1e-4 if dtype == F32 else 0.05
    ok_a, ok_b = gaps_a[0] > least, gaps_b[0] > least
    assert ok_a.sum() > 60 and ok_b.sum() > 25
    s = eng.alloc_slot()
    got = eng.step([StepEntry(s, a, range(len(a)))])
    close(got[ok_a], want_a[ok_a], dtype, "routed, whole")
    eng.free_slot(s)
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    out = eng.step([StepEntry(sa, a[:50], range(50)), StepEntry(sb, b[:20], range(20))])
    close(out[:50][ok_a[:50]], want_a[:50][ok_a[:50]], dtype, "routed, a's prompt")
    close(out[50:][ok_b[:20]], want_b[:20][ok_b[:20]], dtype, "routed, b's prompt")
    for i in range(21):
        out = eng.step([StepEntry(sa, [a[50 + i]], [0]), StepEntry(sb, [b[20 + i]], [0])])
        if ok_a[50 + i]:
            close(out[:1], want_a[50 + i:51 + i], dtype, f"routed, a token {i}")
        if ok_b[20 + i]:
            close(out[1:], want_b[20 + i:21 + i], dtype, f"routed, b token {i}")
    eng.free_slot(sa)
    eng.free_slot(sb)
    assert eng.cache.held_pages() == 0


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_toy_embedding_that_adds_a_row_per_position(dtype):
    """Learned absolute positions: an embedding part defined above in this file that adds a row
    of a table by each row's position, which it reads from the step's context.  Whole, cut, two
    sequences at once, and through the generation loop (where the step's context is the decode
    loop's fixed buffers)."""
    from sonicboom_amd.engine import StepEntry, generate
    from sonicboom_amd.sampling import SamplingParams
    cfg, ref, model, eng = build_toy(TOY_PLACES, dtype)
    rng = np.random.default_rng(8)
    a, b = ([int(t) for t in rng.integers(0, 140, size=n)] for n in (90, 33))
    want_a, want_b = plain_toy(cfg, ref, a), plain_toy(cfg, ref, b)
    moved = plain_toy(cfg, dict(ref, places=np.roll(ref["places"], 1, axis=0)), a)
    assert np.abs(moved - want_a).max() > 0.05            # the positions' rows do matter
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    out = eng.step([StepEntry(sa, a[:60], range(60)), StepEntry(sb, b[:10], range(10))])
    close(out[:60], want_a[:60], dtype, "places, a's prompt")
    close(out[60:], want_b[:10], dtype, "places, b's prompt")
    for i in range(23):
        out = eng.step([StepEntry(sa, [a[60 + i]], [0]), StepEntry(sb, [b[10 + i]], [0])])
        close(out[:1], want_a[60 + i:61 + i], dtype, f"places, a token {i}")
        close(out[1:], want_b[10 + i:11 + i], dtype, f"places, b token {i}")
    eng.free_slot(sa)
    eng.free_slot(sb)
    toks = generate(eng, [a[:7], b[:12]], SamplingParams(max_tokens=8), stop_tokens=())
    if dtype == F32:
        for prompt, out_t in zip((a[:7], b[:12]), toks):
            logits = plain_toy(cfg, ref, prompt + out_t)
            assert out_t == [int(np.argmax(logits[len(prompt) - 1 + i])) for i in range(8)]


def test_windowed_groups_get_pools_of_their_own_size():
    """With a bound on the sequences and on a step's rows, a windowed group's pool holds a window
    and a step's rows a sequence instead of the whole cache, and a prompt longer than that pool
    runs through it portion by portion."""
    from sonicboom_amd.engine import StepEntry
    cfg, ref, model, eng = build_toy(TOY_WINDOWS, F32, max_slots=2, max_step_rows=64)
    pools = {g.window: eng.cache.pools[i].n_pages for i, g in enumerate(eng.cache.groups)}
    assert pools == {0: 12, 50: 2 * 3 + 1, 70: 2 * 4 + 1}
    assert eng.cache.k[[g.window for g in eng.cache.groups].index(50)].shape[1] == 7
    rng = np.random.default_rng(2)
    a, b = ([int(t) for t in rng.integers(0, 150, size=n)] for n in (400, 300))      # 7 + 5 pages of all keys
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    out = eng.step([StepEntry(sa, a, range(len(a))), StepEntry(sb, b, range(len(b)))])      # eleven portions
    close(out[:400], plain_toy(cfg, ref, a), F32, "a through small pools")
    close(out[400:], plain_toy(cfg, ref, b), F32, "b through small pools")
    held = {g.window: eng.cache.held_pages(i) for i, g in enumerate(eng.cache.groups)}
    assert held[0] == 12 and held[50] <= 4 and held[70] <= 6
    eng.free_slot(sa)
    eng.free_slot(sb)
    assert all(eng.cache.held_pages(i) == 0 for i in range(3))

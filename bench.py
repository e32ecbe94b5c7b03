"""Decode and prefill throughput of the Qwen2.5-7B layer sizes with random bf16 weights
on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
                    [--sizes 7b|14b|72b] [--prompt T] [--context C]

A "step" is one decode step: every sequence of the batch goes on by one token
(step function, greedy choice on the device, the token fed back).  The default
run has the sizes of the benchmark configuration (28 layers, width 3584, 28
heads, 4 kv heads, head size 128, inner width 18944, vocabulary 152064), a
batch of 8 and a cache for 4096 tokens per sequence, each holding a
2,048-token prompt of seeded random ids.  One JSON line is printed:
decoded tokens a second, the prefill of one 2,048-token prompt, the decode
step against the HBM roofline, and decode at batch 1 and 64.
"""
import argparse
import json
import statistics
import sys
import time

PEAK_HBM_GBS = 8000.0            # MI355X, published
PEAK_FLOPS = {"bf16": 2.5e15, "fp32": 157.3e12}

CONFIG_7B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2",
    "num_hidden_layers": 28, "hidden_size": 3584, "num_attention_heads": 28, "num_key_value_heads": 4,
    "intermediate_size": 18944, "vocab_size": 152064, "rope_theta": 1000000.0, "rms_norm_eps": 1e-6,
    "max_position_embeddings": 32768, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu",
}
# the other sizes the baseline names, for runs beyond the default one (--sizes)
CONFIG_14B = dict(CONFIG_7B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
                  num_key_value_heads=8, intermediate_size=13824)
CONFIG_72B = dict(CONFIG_7B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                  num_key_value_heads=8, intermediate_size=29568)
SIZES = {"7b": ("Qwen2.5-7B", CONFIG_7B), "14b": ("Qwen2.5-14B", CONFIG_14B), "72b": ("Qwen2.5-72B", CONFIG_72B)}
CONTEXT = 4096
PROMPT = 2048


def model_numbers(cfg, n_layers):
    d, ff, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    hq, hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = d // hq
    qw, kvw = hq * hd, hkv * hd
    layer_params = d * (qw + 2 * kvw) + (qw + 2 * kvw) + qw * d + 3 * d * ff + 2 * d
    return dict(d=d, ff=ff, v=v, hq=hq, hkv=hkv, hd=hd, qw=qw, kvw=kvw, layer_params=layer_params,
                layers=n_layers)


def prefill_flops(m, t):
    per_layer = 2 * t * (m["d"] * (m["qw"] + 2 * m["kvw"]) + m["qw"] * m["d"] + 3 * m["d"] * m["ff"])
    attn = 4 * (t * (t + 1) // 2) * m["hq"] * m["hd"]          # scores and mix over the causal pairs
    return m["layers"] * (per_layer + attn) + 2 * m["v"] * m["d"]   # the head runs for the last row only


def decode_bytes(m, batch, lengths):
    """Bytes a decode step has to read: every weight it uses once (bf16), the embedding rows of
    the batch, and the cached keys and values of the live requests."""
    weights = m["layers"] * m["layer_params"] * 2 + (m["v"] * m["d"] + m["d"]) * 2 + batch * m["d"] * 2
    kv = sum(lengths) * 2 * m["kvw"] * 2 * m["layers"]
    return weights + kv


def main() -> int:
    global PROMPT, CONTEXT
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--layers", type=int, default=0, help="run fewer layers than the configuration has")
    ap.add_argument("--sizes", choices=sorted(SIZES), default="7b", help="layer sizes (default: the benchmark's)")
    ap.add_argument("--prompt", type=int, default=PROMPT, help="cached prompt tokens per sequence")
    ap.add_argument("--context", type=int, default=CONTEXT, help="cache size per sequence")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--no-graph", action="store_true", help="launch decode steps kernel by kernel")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2

    import numpy as np
    import torch

    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry
    from sonicboom_amd.engine.decode import DecodeLoop

    PROMPT, CONTEXT = a.prompt, max(a.context, a.prompt + a.steps + a.warmup + 64)
    model_name, base_cfg = SIZES[a.sizes]
    cfg = dict(base_cfg)
    full_layers = cfg["num_hidden_layers"]
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    m = model_numbers(cfg, cfg["num_hidden_layers"])
    t0 = time.time()
    model = DecoderModel.from_random(cfg, seed=0, dtype="bfloat16", device="cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] model of {cfg['num_hidden_layers']} layers ready in {time.time() - t0:.1f} s",
          file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)

    def prompts(n):
        return [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=PROMPT)] for _ in range(n)]

    def sync_time(fn):
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t

    # ---- prefill of one prompt (2,048 tokens unless --prompt says otherwise) ----------------
    engine = Engine(model, max_tokens=CONTEXT)
    times = []
    for i in range(5):
        p = prompts(1)[0]
        slot = engine.alloc_slot()
        times.append(sync_time(lambda: engine.step([StepEntry(slot, p, (PROMPT - 1,))])))
        engine.free_slot(slot)
    prefill_s = statistics.median(times[1:])
    pf = prefill_flops(m, PROMPT)
    prefill = {"value": round(PROMPT / prefill_s, 1), "tokens": PROMPT, "ms": round(prefill_s * 1e3, 3),
               "frac": round(pf / prefill_s / PEAK_FLOPS["bf16"], 4)}
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    del engine

    # ---- decode -----------------------------------------------------------------------------
    def decode_run(batch, steps, warmup):
        eng = Engine(model, max_tokens=CONTEXT * batch)
        loop = DecodeLoop(eng, use_graph=not a.no_graph)
        slots = [eng.alloc_slot() for _ in range(batch)]
        ps = prompts(batch)
        first = []
        for i in range(0, batch, 8):            # prompts in steps of 8 sequences
            logits = eng.step([StepEntry(s, p, (PROMPT - 1,)) for s, p in zip(slots[i:i + 8], ps[i:i + 8])])
            first += torch.argmax(logits, dim=-1).tolist()
        loop.start(slots, first)
        for _ in range(warmup):
            loop.step()
        torch.cuda.synchronize()
        t = time.perf_counter()
        for _ in range(steps):
            loop.step()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t) / steps
        lengths = [eng.length(s) for s in slots]
        loop.close()
        for s in slots:
            eng.free_slot(s)
        del eng
        return dt, lengths

    step_s, lengths = decode_run(a.batch, a.steps, a.warmup)
    value = a.batch / step_s
    nbytes = decode_bytes(m, a.batch, lengths)
    roofline = {"bound": "hbm", "achieved": round(nbytes / step_s / 1e9, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s", "frac": round(nbytes / step_s / 1e9 / PEAK_HBM_GBS, 4)}
    print(f"[bench] decode b{a.batch}: {value:.1f} tok/s, {step_s * 1e3:.3f} ms/step, {roofline}",
          file=sys.stderr, flush=True)
    points = {}
    if not a.no_points:
        for b in (1, 64):
            dt, _ = decode_run(b, max(8, a.steps // 2), max(2, a.warmup // 2))
            points[f"decode_b{b}"] = round(b / dt, 1)
            print(f"[bench] decode b{b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)

    line = {
        "metric": f"decode tokens/s, {model_name} sizes, batch {a.batch}, {PROMPT}-token cached prompts",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "model": f"{model_name} sizes, random bf16 weights", "layers": cfg["num_hidden_layers"],
            "layers_of_configuration": full_layers, "hidden_size": m["d"], "num_attention_heads": m["hq"],
            "num_key_value_heads": m["hkv"], "head_dim": m["hd"], "intermediate_size": m["ff"],
            "vocab_size": m["v"], "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "tie_word_embeddings": False, "global_batch": a.batch, "seq_len": CONTEXT,
            "cached_prompt_tokens": PROMPT, "parallelism": "single GPU", "decode_graph": not a.no_graph,
        },
        "prefill": prefill, "roofline": roofline, "points": points,
    }
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

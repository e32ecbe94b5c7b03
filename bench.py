"""Decode and prefill throughput of the Qwen2.5 layer sizes with random bf16 weights on one
MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch B] [--layers L]
                    [--sizes 0.5b|1.5b|3b|7b|14b|32b|72b] [--prompt T] [--context C] [--workload steady|mixed|forms]

A "step" is one decode step: every sequence of the batch goes on by one token (step function,
greedy choice on the device, the token fed back).

``--workload steady`` (the default) has the sizes of the benchmark configuration (28 layers,
width 3584, 28 heads, 4 kv heads, head size 128, inner width 18944, vocabulary 152064), a batch
of 8 and a cache for 4096 tokens per sequence, each holding a 2,048-token prompt of seeded random
ids.  One JSON line is printed: decoded tokens a second (from the median step), the prefill of one
2,048-token prompt, the decode step against the HBM roofline with the rates of its kernels, and
decode at batch 1 and 64.

The same line carries the context-length curve as further ``points`` (and with bytes, flops and
fractions under ``curve``): for cached depths of 512, 4,096, 8,192, 16,384 and 32,768 tokens the
decode rate at batch 1 and batch 8 (``decode_b1_d8192`` ...) and the prefill rate of one prompt of
that length (``prefill_8192`` ...); ``--no-curve`` leaves it out, ``--curve 512,4096`` picks depths.
``--runs R`` (R > 1) starts R fresh processes of the same command one after the other, before
anything touches the GPU here, and prints the run whose ``value`` is the median, with all values.
Beside the JSON line on standard output, every metric goes to standard error as a
``RESULT key=value ...`` line; the engine clock sampled during the timed decode steps is in both.

``--workload mixed`` runs what the baseline names for the larger sizes through the generation
loop itself: ``--sizes 14b``: 16 prompts of seeded lengths uniform in [256, 4096] in a cache of
8192 tokens a sequence, prompts in one step, then 256 greedy steps; ``--sizes 72b``: 8 prompts of
512 to 2048 tokens, 128 steps, 4096 tokens a sequence.  Prefill and decode are timed apart.

``--workload forms`` prints a table instead of the line: the decode step (``--batches 1,8``) with
the qkv, output and down product forced, one at a time, to every form (waves a block x K slices)
of the kernel that streams the weights, against the launchers' own choices.
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
    "max_position_embeddings": 131072, "tie_word_embeddings": False, "use_sliding_window": False,
    "hidden_act": "silu",
}
# the other sizes the baseline names, for runs beyond the default one (--sizes)
CONFIG_14B = dict(CONFIG_7B, num_hidden_layers=48, hidden_size=5120, num_attention_heads=40,
                  num_key_value_heads=8, intermediate_size=13824)
CONFIG_72B = dict(CONFIG_7B, num_hidden_layers=80, hidden_size=8192, num_attention_heads=64,
                  num_key_value_heads=8, intermediate_size=29568)
CONFIG_32B = dict(CONFIG_14B, num_hidden_layers=64, intermediate_size=27648)
# the family's small members: tied head, a vocabulary of 151,936
CONFIG_05B = dict(CONFIG_7B, num_hidden_layers=24, hidden_size=896, num_attention_heads=14, num_key_value_heads=2,
                  intermediate_size=4864, vocab_size=151936, tie_word_embeddings=True)
CONFIG_15B = dict(CONFIG_05B, num_hidden_layers=28, hidden_size=1536, num_attention_heads=12, intermediate_size=8960)
CONFIG_3B = dict(CONFIG_05B, num_hidden_layers=36, hidden_size=2048, num_attention_heads=16, intermediate_size=11008)
SIZES = {"7b": ("Qwen2.5-7B", CONFIG_7B), "14b": ("Qwen2.5-14B", CONFIG_14B), "72b": ("Qwen2.5-72B", CONFIG_72B),
         "32b": ("Qwen2.5-32B", CONFIG_32B), "0.5b": ("Qwen2.5-0.5B", CONFIG_05B), "1.5b": ("Qwen2.5-1.5B", CONFIG_15B),
         "3b": ("Qwen2.5-3B", CONFIG_3B)}
# the mixed workloads: prompts, shortest, longest, greedy steps, cache tokens a sequence
MIXED = {"72b": (8, 512, 2048, 128, 4096), "32b": (8, 512, 2048, 128, 4096)}
MIXED_DEFAULT = (16, 256, 4096, 256, 8192)
CONTEXT = 4096
PROMPT = 2048
CURVE_DEPTHS = (512, 4096, 8192, 16384, 32768)
CURVE_BATCHES = (1, 8)


def model_numbers(cfg, n_layers):
    d, ff, v = cfg["hidden_size"], cfg["intermediate_size"], cfg["vocab_size"]
    hq, hkv = cfg["num_attention_heads"], cfg["num_key_value_heads"]
    hd = d // hq
    qw, kvw = hq * hd, hkv * hd
    layer_params = d * (qw + 2 * kvw) + (qw + 2 * kvw) + qw * d + 3 * d * ff + 2 * d
    return dict(d=d, ff=ff, v=v, hq=hq, hkv=hkv, hd=hd, qw=qw, kvw=kvw, layer_params=layer_params,
                layers=n_layers)


def prefill_flops(m, lengths):
    """Flops of a prompt step of sequences of these lengths whose last rows go through the head."""
    t = sum(lengths)
    per_layer = 2 * t * (m["d"] * (m["qw"] + 2 * m["kvw"]) + m["qw"] * m["d"] + 3 * m["d"] * m["ff"])
    attn = sum(4 * (n * (n + 1) // 2) * m["hq"] * m["hd"] for n in lengths)   # scores and mix, causal pairs
    return m["layers"] * (per_layer + attn) + len(lengths) * 2 * m["v"] * m["d"]


def decode_bytes(m, batch, lengths):
    """Bytes a decode step has to read: every weight it uses once (bf16), the embedding rows of
    the batch, and the cached keys and values of the live requests."""
    weights = m["layers"] * m["layer_params"] * 2 + (m["v"] * m["d"] + m["d"]) * 2 + batch * m["d"] * 2
    kv = sum(lengths) * 2 * m["kvw"] * 2 * m["layers"]
    return weights + kv


class ClockSampler:
    """Samples the GPU's engine clock in a thread while work runs (the driver's ``pp_dpm_sclk``
    file, else ``rocm-smi --showclocks``): what the matrix pipes' peak has to be scaled by under
    load, and what a run's figures have to be read against."""

    def __init__(self, period=0.4):
        import threading
        self.period, self.mhz, self._stop = period, [], threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    @staticmethod
    def read():
        import glob
        import re
        import subprocess
        # the driver's own file first (microseconds to read): the level marked with a star
        for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
            try:
                with open(path) as f:
                    m = re.search(r"(\d+)\s*Mhz\s*\*", f.read(), re.IGNORECASE)
            except OSError:
                continue
            if m:
                return int(m.group(1))
        try:
            out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
        except (OSError, subprocess.SubprocessError):
            return None
        m = re.search(r"sclk clock level: \S+ \((\d+)Mhz\)", out)
        return int(m.group(1)) if m else None

    def _run(self):
        while not self._stop.is_set():
            v = self.read()
            if v is not None:
                self.mhz.append(v)
            self._stop.wait(self.period)

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join()

    def summary(self):
        if not self.mhz:
            return None
        return {"samples": len(self.mhz), "min_mhz": min(self.mhz), "max_mhz": max(self.mhz),
                "median_mhz": int(statistics.median(self.mhz))}


class OpTimer:
    """Times the kernel calls of one step that runs kernel by kernel: every function of
    ``sonicboom_amd.ops`` that launches is wrapped between two events on the stream, and the
    times are summed by (function, what it worked on)."""

    NAMES = ("embed", "rmsnorm", "gemm_bf16", "gemm_bf16_partial", "reduce_resid_norm", "rope_kv_store",
             "attention", "attention_decode_rope", "argmax", "gemm_plain", "silu_mul", "add_into", "cast")

    def __init__(self, m):
        self.m, self.records, self._saved = m, [], {}

    def _label(self, name, args, kw):
        m = self.m
        if name in ("gemm_bf16", "gemm_bf16_partial"):
            n, k = kw.get("packed_shape") or (args[1].shape[0], args[1].shape[-1])
            if kw.get("gated"):
                return "gate_up"
            return {(m["qw"] + 2 * m["kvw"], m["d"]): "qkv", (m["d"], m["qw"]): "out", (m["d"], m["ff"]): "down",
                    (m["v"], m["d"]): "head"}.get((n, k), f"product_{n}x{k}")
        # (a decode step's attention rotates and stores the new key and value itself)
        return {"reduce_resid_norm": "add_slices_norm", "rope_kv_store": "rotate_store",
                "attention_decode_rope": "attention"}.get(name, name)

    def __enter__(self):
        import torch
        from sonicboom_amd import ops
        for name in self.NAMES:
            fn = getattr(ops, name)
            self._saved[name] = fn

            def timed(*args, _fn=fn, _name=name, **kw):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                out = _fn(*args, **kw)
                e1.record()
                if out is not None or _name not in ("gemm_bf16", "gemm_bf16_partial"):   # None: not taken
                    self.records.append((self._label(_name, args, kw), e0, e1))
                return out
            setattr(ops, name, timed)
        return self

    def __exit__(self, *exc):
        from sonicboom_amd import ops
        for name, fn in self._saved.items():
            setattr(ops, name, fn)

    def totals(self):
        """label -> (microseconds, calls)"""
        import torch
        torch.cuda.synchronize()
        out = {}
        for label, e0, e1 in self.records:
            us, n = out.get(label, (0.0, 0))
            out[label] = (us + e0.elapsed_time(e1) * 1e3, n + 1)
        return out


def kernel_rates(m, totals, rows, kv_tokens, prefill_lengths=None):
    """Achieved rates of the step's kernels from an OpTimer's totals: GB/s of the bytes each must
    read for a decode step, TFLOP/s for a prompt step."""
    L = m["layers"]
    weights = {"qkv": m["d"] * (m["qw"] + 2 * m["kvw"]), "out": m["qw"] * m["d"], "gate_up": 2 * m["d"] * m["ff"],
               "down": m["d"] * m["ff"]}
    out = {}
    for label, (us, calls) in sorted(totals.items()):
        item = {"us": round(us, 1), "calls": calls}
        if prefill_lengths is None:
            if label in weights:
                item["GB/s"] = round(weights[label] * 2 * calls / us / 1e3, 1)
            elif label == "head":
                item["GB/s"] = round(m["v"] * m["d"] * 2 * calls / us / 1e3, 1)
            elif label == "attention":
                item["GB/s"] = round(kv_tokens * 2 * m["kvw"] * 2 * calls / us / 1e3, 1)
            if "GB/s" in item:
                item["frac"] = round(item["GB/s"] / PEAK_HBM_GBS, 3)
        else:
            if label in weights:
                # per layer, not per call: a long prompt runs in portions, several calls a layer
                item["TFLOP/s"] = round(2 * rows * weights[label] * L / us / 1e6, 1)
            elif label == "attention":
                flops = sum(4 * (n * (n + 1) // 2) * m["hq"] * m["hd"] for n in prefill_lengths)
                item["TFLOP/s"] = round(flops * L / us / 1e6, 1)
            if "TFLOP/s" in item:
                item["frac"] = round(item["TFLOP/s"] * 1e12 / PEAK_FLOPS["bf16"], 3)
        out[label] = item
    return out


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
    ap.add_argument("--workload", choices=("steady", "mixed", "forms"), default="steady")
    ap.add_argument("--batches", default="1,8", help="--workload forms: the batch sizes, comma separated")
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 and batch 64 points")
    ap.add_argument("--no-graph", action="store_true", help="launch decode steps kernel by kernel")
    ap.add_argument("--no-kernels", action="store_true", help="skip the per-kernel rates")
    ap.add_argument("--clocks", action="store_true",
                    help="also run prompt steps back to back for a few seconds and sample the engine clock meanwhile")
    ap.add_argument("--curve", default=",".join(str(d) for d in CURVE_DEPTHS),
                    help="cached depths of the context-length curve (decode at batch 1 and 8, prefill of one prompt)")
    ap.add_argument("--no-curve", action="store_true", help="skip the context-length curve")
    ap.add_argument("--runs", type=int, default=1,
                    help="fresh processes to run one after the other; the median run is printed")
    a = ap.parse_args()
    if a.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {a.gpus} is not supported")
        return 2
    if a.runs > 1:
        argv, skip = [], False
        for arg in sys.argv[1:]:
            if skip:
                skip = False
            elif arg == "--runs":
                skip = True
            elif not arg.startswith("--runs="):
                argv.append(arg)
        return median_of_runs(argv, a.runs)

    import numpy as np
    import torch

    from sonicboom_amd import ops
    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry, generate
    from sonicboom_amd.engine.decode import DecodeLoop
    from sonicboom_amd.sampling import SamplingParams

    PROMPT, CONTEXT = a.prompt, max(a.context, a.prompt + a.steps + a.warmup + 64)
    if a.prompt != 2048 and "--curve" not in " ".join(sys.argv[1:]):
        a.no_curve = True           # a run at a depth of its own is one point, not the curve
    model_name, base_cfg = SIZES[a.sizes]
    cfg = dict(base_cfg)
    full_layers = cfg["num_hidden_layers"]
    if a.layers:
        cfg["num_hidden_layers"] = a.layers
    cfg["max_position_embeddings"] = max(cfg["max_position_embeddings"], CONTEXT)
    m = model_numbers(cfg, cfg["num_hidden_layers"])
    t0 = time.time()
    model = DecoderModel.from_random(cfg, seed=0, dtype="bfloat16", device="cuda:0")
    torch.cuda.synchronize()
    print(f"[bench] model of {cfg['num_hidden_layers']} layers ready in {time.time() - t0:.1f} s, "
          f"{torch.cuda.max_memory_allocated() / 2**30:.1f} GiB at most on the device",
          file=sys.stderr, flush=True)
    rng = np.random.default_rng(0)
    peak_measured = None if a.no_kernels else round(ops.read_bandwidth() / 1e9, 1)

    def config(**more):
        c = {
            "model": f"{model_name} sizes, random bf16 weights", "layers": cfg["num_hidden_layers"],
            "layers_of_configuration": full_layers, "hidden_size": m["d"], "num_attention_heads": m["hq"],
            "num_key_value_heads": m["hkv"], "head_dim": m["hd"], "intermediate_size": m["ff"],
            "vocab_size": m["v"], "rope_theta": cfg["rope_theta"], "rms_norm_eps": cfg["rms_norm_eps"],
            "tie_word_embeddings": bool(cfg["tie_word_embeddings"]), "parallelism": "single GPU", "decode_graph": not a.no_graph,
        }
        c.update(more)
        return c

    def random_prompts(lengths):
        return [[int(t) for t in rng.integers(0, cfg["vocab_size"], size=n)] for n in lengths]

    def sync_time(fn):
        torch.cuda.synchronize()
        t = time.perf_counter()
        fn()
        torch.cuda.synchronize()
        return time.perf_counter() - t

    # ------------------------------------------------------------------------------------------
    if a.workload == "forms":
        # The decode step with one product at a time forced to every form of the weight-streaming
        # kernel (waves a block x K slices), everything else as the launchers choose: a table on
        # standard output, no JSON line.  The products are told apart by their packed shapes.
        d, ff = m["d"], m["ff"]
        targets = {"qkv": ((m["hq"] + 2 * m["hkv"]) * m["hd"], d), "out": (d, m["hq"] * m["hd"]), "down": (d, ff)}
        forced = {"shape": None, "form": (0, 0)}
        launcher_partial = ops.gemm_bf16_partial

        def partial(x, w, packed_shape=None):
            if packed_shape is not None and tuple(packed_shape) == forced["shape"]:
                with ops.gemm_few_rows_kernel(None, *forced["form"]):
                    return launcher_partial(x, w, packed_shape=packed_shape)
            return launcher_partial(x, w, packed_shape=packed_shape)
        ops.gemm_bf16_partial = partial
        layers = cfg["num_hidden_layers"]
        slice_counts = (1, 2, 3, 4, 5, 6, 8)
        for batch in (int(b) for b in a.batches.split(",")):
            eng = Engine(model, ((PROMPT + 511) // 64) * 64 * batch, max_slots=batch)
            slots = [eng.alloc_slot() for _ in range(batch)]
            eng.step([StepEntry(s, p, (PROMPT - 1,)) for s, p in zip(slots, random_prompts([PROMPT] * batch))])

            def step_ms(shape, form):
                forced["shape"], forced["form"] = shape, form
                loop = DecodeLoop(eng, use_graph=not a.no_graph)
                loop.start(slots, [1] * batch)
                for _ in range(4):
                    loop.step()
                times = [sync_time(loop.step) for _ in range(24)]
                loop.close()
                for s in slots:
                    eng.cache.truncate(s, PROMPT)
                return statistics.median(times) * 1e3
            own = statistics.median(step_ms(None, (0, 0)) for _ in range(3))
            print(f"{model_name} sizes, batch {batch}, {PROMPT} cached tokens: the launchers' own choices {own:.4f} ms a step")
            for name, shape in targets.items():
                print(f"  {name} {shape[0]} x {shape[1]} ({shape[0] * shape[1] * 2 / 1e6:.1f} MB); step in ms (difference a layer "
                      f"in us) by waves; columns: {', '.join(str(c) for c in slice_counts)} slices", flush=True)
                for waves in (4, 5, 6, 7, 8):
                    cells = []
                    for slices in slice_counts:
                        t = step_ms(shape, (waves, slices))
                        cells.append(f"{t:.3f} ({(t - own) * 1e3 / layers:+.2f})")
                    print(f"    {waves} waves: " + "  ".join(cells), flush=True)
            for s in slots:
                eng.free_slot(s)
            del eng
        ops.gemm_bf16_partial = launcher_partial
        return 0

    if a.workload == "mixed":
        n_prompts, shortest, longest, n_steps, per_seq = MIXED.get(a.sizes, MIXED_DEFAULT)
        lengths = [int(n) for n in rng.integers(shortest, longest + 1, size=n_prompts)]
        prompts = random_prompts(lengths)
        engine = Engine(model, max_tokens=per_seq * n_prompts)
        engine.use_graphs = not a.no_graph
        params = SamplingParams(max_tokens=n_steps)
        marks = []

        def run():
            marks.clear()
            t_start = time.perf_counter()

            def first_token(i, t):
                if not marks:
                    marks.append(time.perf_counter())      # the prompt step and the first choice are done
                return False
            outs = generate(engine, prompts, params, stop_tokens=(), max_batch=n_prompts, callback=first_token)
            torch.cuda.synchronize()
            t_end = time.perf_counter()
            assert all(len(o) == n_steps for o in outs)
            return marks[0] - t_start, t_end - marks[0]

        warm = generate(engine, [p[:64] for p in prompts], SamplingParams(max_tokens=4), stop_tokens=(),
                        max_batch=n_prompts)          # compiles nothing, but pages in the kernels
        del warm
        runs = [run() for _ in range(3)]
        prefill_s = statistics.median(r[0] for r in runs)
        decode_s = statistics.median(r[1] for r in runs)
        decoded = n_prompts * (n_steps - 1)           # the first token of each comes from the prompt step
        step_s = decode_s / (n_steps - 1)
        mean_lengths = [n + n_steps / 2 for n in lengths]
        nbytes = decode_bytes(m, n_prompts, mean_lengths)
        pf = prefill_flops(m, lengths)
        line = {
            "metric": f"decode tokens/s, {model_name} sizes, {n_prompts} prompts of {shortest}-{longest} tokens "
                      f"in one batch, {n_steps} greedy steps through the generation loop",
            "value": round(decoded / decode_s, 1), "unit": "tokens/s", "n_gpus": 1, "steps": n_steps - 1,
            "warmup": 1, "ms_per_step": round(step_s * 1e3, 4), "higher_is_better": True, "scaling": "weak",
            "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
            "config": config(global_batch=n_prompts, seq_len=per_seq, prompt_tokens=sum(lengths),
                             shortest_prompt=min(lengths), longest_prompt=max(lengths)),
            "prefill": {"value": round(sum(lengths) / prefill_s, 1), "tokens": sum(lengths),
                        "ms": round(prefill_s * 1e3, 3), "frac": round(pf / prefill_s / PEAK_FLOPS["bf16"], 4)},
            "roofline": {"bound": "hbm", "achieved": round(nbytes / step_s / 1e9, 1), "peak": PEAK_HBM_GBS,
                         "unit": "GB/s", "frac": round(nbytes / step_s / 1e9 / PEAK_HBM_GBS, 4),
                         "peak_measured": peak_measured, "bytes_per_step": int(nbytes)},
            "runs": [{"prefill_ms": round(p * 1e3, 2), "decode_ms": round(d * 1e3, 2)} for p, d in runs],
        }
        print(json.dumps(line), flush=True)
        return 0

    # ---- prefill of one prompt (2,048 tokens unless --prompt says otherwise) ----------------
    def prefill_run(engine, n_tokens, timed, kernels):
        """Median seconds of ``timed`` prompt steps of one prompt of ``n_tokens`` in an empty slot
        (after one untimed step), as the bench line's ``prefill`` entry."""
        times = []
        for i in range(timed + 1):
            p = random_prompts([n_tokens])[0]
            slot = engine.alloc_slot()
            times.append(sync_time(lambda: engine.step([StepEntry(slot, p, (n_tokens - 1,))])))
            engine.free_slot(slot)
        secs = statistics.median(times[1:])
        pf = prefill_flops(m, [n_tokens])
        out = {"value": round(n_tokens / secs, 1), "tokens": n_tokens, "ms": round(secs * 1e3, 3),
               "frac": round(pf / secs / PEAK_FLOPS["bf16"], 4), "flops": int(pf)}
        if kernels:
            slot = engine.alloc_slot()
            with OpTimer(m) as timer:
                engine.step([StepEntry(slot, random_prompts([n_tokens])[0], (n_tokens - 1,))])
            engine.free_slot(slot)
            out["kernels"] = kernel_rates(m, timer.totals(), n_tokens, 0, prefill_lengths=[n_tokens])
        return out, pf

    engine = Engine(model, max_tokens=CONTEXT)
    prefill, pf = prefill_run(engine, PROMPT, 4, not a.no_kernels)
    if a.clocks:
        idle = ClockSampler.read()
        p = random_prompts([PROMPT])[0]
        with ClockSampler() as sampler:
            t_end = time.time() + 6.0
            n_runs, t_run = 0, 0.0
            while time.time() < t_end:
                slot = engine.alloc_slot()
                t_run += sync_time(lambda: engine.step([StepEntry(slot, p, (PROMPT - 1,))]))
                engine.free_slot(slot)
                n_runs += 1
        clocks = sampler.summary()
        if clocks is not None:
            clocks.update(idle_mhz=idle, prompt_steps=n_runs, ms_per_prompt_step=round(t_run / n_runs * 1e3, 3),
                          frac_at_median_clock=round(pf / (t_run / n_runs) / (PEAK_FLOPS["bf16"] * clocks["median_mhz"] / 2400.0), 4))
        prefill["clocks"] = clocks
    print(f"[bench] prefill {prefill}", file=sys.stderr, flush=True)
    del engine

    # ---- decode -----------------------------------------------------------------------------
    def decode_steps(eng, slots, first, steps, warmup, kernels=False, clock=None):
        """Time ``steps`` decode steps of the sequences in ``slots`` (fed ``first``) after
        ``warmup`` untimed ones: median and mean seconds a step, the lengths after the run, the
        kernels' rates, and the tokens the next step would feed."""
        loop = DecodeLoop(eng, use_graph=not a.no_graph)
        batch = len(slots)
        loop.start(slots, first)
        for _ in range(warmup):
            loop.step()
        torch.cuda.synchronize()
        per_step = []
        if clock is not None:
            clock.__enter__()
        t_all = time.perf_counter()
        for _ in range(steps):
            t = time.perf_counter()
            loop.step()                         # ends with the chosen tokens on the host
            per_step.append(time.perf_counter() - t)
        torch.cuda.synchronize()
        mean = (time.perf_counter() - t_all) / steps
        if clock is not None:
            clock.__exit__()
        lengths = [eng.length(s) for s in slots]
        rates = None
        if kernels:
            plain = DecodeLoop(eng, use_graph=False)
            plain.start(slots, loop.pending)
            plain.step()
            with OpTimer(m) as timer:
                plain.step()
            rates = kernel_rates(m, timer.totals(), batch, sum(lengths) + batch, None)
            loop.pending = plain.pending
        pending = list(loop.pending)
        loop.close()
        return statistics.median(per_step), mean, lengths, rates, pending

    def fill(eng, batch, prompt):
        """``batch`` slots, each with a cached prompt of ``prompt`` random tokens, and the first
        token of each; the prompts run in one step (in portions of the engine's row limit)."""
        slots = [eng.alloc_slot() for _ in range(batch)]
        ps = random_prompts([prompt] * batch)
        logits = eng.step([StepEntry(s, p, (prompt - 1,)) for s, p in zip(slots, ps)])
        return slots, torch.argmax(logits, dim=-1).tolist()

    def per_sequence(prompt, steps, warmup):
        """Cache tokens a sequence needs for these runs (whole pages, with room to spare)."""
        return ((prompt + 2 * (steps + warmup) + 8 + 127) // 64) * 64

    def decode_run(batch, steps, warmup, kernels=False, clock=None):
        eng = Engine(model, max_tokens=max(CONTEXT, per_sequence(PROMPT, steps, warmup)) * batch)
        slots, first = fill(eng, batch, PROMPT)
        out = decode_steps(eng, slots, first, steps, warmup, kernels, clock)
        for s in slots:
            eng.free_slot(s)
        del eng
        return out[:4]

    def hbm(nbytes, secs):
        return {"bound": "hbm", "achieved": round(nbytes / secs / 1e9, 1), "peak": PEAK_HBM_GBS,
                "unit": "GB/s", "frac": round(nbytes / secs / 1e9 / PEAK_HBM_GBS, 4),
                "peak_measured": peak_measured, "bytes_per_step": int(nbytes)}

    sampler = ClockSampler(period=0.2)
    idle_mhz = ClockSampler.read()
    step_s, mean_s, lengths, rates = decode_run(a.batch, a.steps, a.warmup, kernels=not a.no_kernels, clock=sampler)
    clock = sampler.summary()
    if clock is not None:
        clock["idle_mhz"] = idle_mhz
    value = a.batch / step_s
    roofline = hbm(decode_bytes(m, a.batch, lengths), step_s)
    if rates is not None:
        roofline["kernels"] = rates
    print(f"[bench] decode b{a.batch}: {value:.1f} tok/s, median {step_s * 1e3:.3f} ms/step "
          f"(mean {mean_s * 1e3:.3f}), {roofline}, engine clock {clock}", file=sys.stderr, flush=True)
    points = {}
    if not a.no_points:
        for b in (1, 64):
            dt, _, _, _ = decode_run(b, max(16, a.steps // 2), max(4, a.warmup // 2))
            points[f"decode_b{b}"] = round(b / dt, 1)
            print(f"[bench] decode b{b}: {points[f'decode_b{b}']} tok/s", file=sys.stderr, flush=True)

    # ---- the context-length curve --------------------------------------------------------------
    curve = {}
    depths = [] if (a.no_curve or a.no_points) else [int(d) for d in a.curve.split(",") if d.strip()]
    steps_c, warm_c = max(8, min(a.steps, 32)), max(3, min(a.warmup, 8))
    for depth in depths:
        per_seq = per_sequence(depth, steps_c, warm_c)
        eng = Engine(model, max_tokens=per_seq * max(CURVE_BATCHES))
        item, _ = prefill_run(eng, depth, 2, not a.no_kernels)
        if "kernels" in item:          # the curve keeps the rate of the kernel that grows with the depth
            item["attention_TFLOPs"] = item["kernels"].get("attention", {}).get("TFLOP/s")
            item["attention_frac"] = item["kernels"].get("attention", {}).get("frac")
            del item["kernels"]
        entry = {"prefill": item}
        points[f"prefill_{depth}"] = item["value"]
        slots, first = fill(eng, max(CURVE_BATCHES), depth)
        for b in sorted(CURVE_BATCHES, reverse=True):        # the larger batch first, then its first sequences
            for s in slots[b:]:
                eng.free_slot(s)
            slots, first = slots[:b], first[:b]
            dt, _, lens, rates_c, first = decode_steps(eng, slots, first, steps_c, warm_c, kernels=not a.no_kernels)
            d_item = {"value": round(b / dt, 1), "ms": round(dt * 1e3, 4)}
            d_item.update({k: v for k, v in hbm(decode_bytes(m, b, lens), dt).items()
                           if k in ("achieved", "frac", "bytes_per_step")})
            if rates_c is not None and "attention" in rates_c:
                d_item["attention_us"] = rates_c["attention"]["us"]
                d_item["attention_GBs"] = rates_c["attention"].get("GB/s")
            entry[f"decode_b{b}"] = d_item
            points[f"decode_b{b}_d{depth}"] = d_item["value"]
        for s in slots:
            eng.free_slot(s)
        del eng
        curve[f"d{depth}"] = entry
        print(f"[bench] depth {depth}: {entry}", file=sys.stderr, flush=True)

    # ---- prefix reuse: a 512-token prefix is in the cache, 64 new tokens come, time to the first token ----
    prefix_reuse = None
    if depths:
        from sonicboom_amd.api import Model
        session = Model(model).session(max_tokens=64 * 32)
        base = random_prompts([512])[0]
        session.generate([base], max_tokens=1, stop_tokens=[], keep=True)
        with_reuse, whole = [], []
        for i in range(6):
            new = base + random_prompts([64])[0]
            with_reuse.append(sync_time(lambda: session.generate([new], max_tokens=1, stop_tokens=[], keep=True)))
            assert session.reused == [512]
        session.forget()
        for i in range(4):
            new = base + random_prompts([64])[0]
            whole.append(sync_time(lambda: session.generate([new], max_tokens=1, stop_tokens=[])))
        prefix_reuse = {"prefix": 512, "new": 64, "ttft_ms": round(statistics.median(with_reuse[1:]) * 1e3, 3),
                        "ttft_ms_without_reuse": round(statistics.median(whole[1:]) * 1e3, 3)}
        print(f"[bench] prefix reuse {prefix_reuse}", file=sys.stderr, flush=True)
        del session

    line = {
        "metric": f"decode tokens/s, {model_name} sizes, batch {a.batch}, {PROMPT}-token cached prompts",
        "value": round(value, 1), "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(step_s * 1e3, 4), "ms_per_step_mean": round(mean_s * 1e3, 4),
        "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": config(global_batch=a.batch, seq_len=CONTEXT, cached_prompt_tokens=PROMPT),
        "prefill": prefill, "roofline": roofline, "points": points, "clock": clock,
    }
    if curve:
        line["curve"] = curve
    if prefix_reuse:
        line["prefix_reuse"] = prefix_reuse
    result_lines(line)
    print(json.dumps(line), flush=True)
    return 0


def result_lines(line, out=sys.stderr):
    """The run's metrics as ``RESULT key=value ...`` lines, one a metric, for tools that parse
    such lines rather than JSON; the engine clock the timed steps ran at is on every line."""
    clock = line.get("clock") or {}
    mhz = clock.get("median_mhz")
    tail = f" sclk_mhz={mhz if mhz is not None else 'unknown'}"
    print(f"RESULT metric=decode_tok_s batch={line['config']['global_batch']} value={line['value']} "
          f"ms_per_step={line['ms_per_step']} hbm_frac={line['roofline']['frac']}{tail}", file=out)
    pre = line.get("prefill")
    if pre:
        print(f"RESULT metric=prefill_tok_s tokens={pre['tokens']} value={pre['value']} ms={pre['ms']} "
              f"flops_frac={pre['frac']}{tail}", file=out)
    for name, v in (line.get("points") or {}).items():
        print(f"RESULT metric={name} value={v}{tail}", file=out)
    reuse = line.get("prefix_reuse")
    if reuse:
        print(f"RESULT metric=prefix_reuse_ttft_ms prefix={reuse['prefix']} new={reuse['new']} value={reuse['ttft_ms']} "
              f"without_reuse={reuse['ttft_ms_without_reuse']}{tail}", file=out)
    out.flush()


def median_of_runs(argv, runs):
    """``runs`` fresh processes of this program, one after the other (nothing here has touched
    the GPU); the line of the run whose value is the median, with every run's value."""
    import os
    import subprocess
    lines = []
    for i in range(runs):
        cmd = [sys.executable, os.path.abspath(__file__)] + argv + ["--runs", "1"]
        p = subprocess.run(cmd, stdout=subprocess.PIPE, text=True)
        if p.returncode != 0:
            print(f"bench.py: run {i + 1} of {runs} ended with {p.returncode}", file=sys.stderr)
            return p.returncode or 1
        found = [ln for ln in p.stdout.splitlines() if ln.startswith("{")]
        lines.append(json.loads(found[-1]))
        print(f"[bench] run {i + 1} of {runs}: {lines[-1]['value']} {lines[-1]['unit']}", file=sys.stderr, flush=True)
    order = sorted(range(runs), key=lambda i: lines[i]["value"])
    line = lines[order[(runs - 1) // 2]]
    line["process_runs"] = runs
    line["values_of_runs"] = [ln["value"] for ln in lines]
    if all("points" in ln for ln in lines):
        line["points"] = {k: statistics.median(ln["points"][k] for ln in lines) for k in line["points"]
                          if all(k in ln["points"] for ln in lines)}
    result_lines(line)
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

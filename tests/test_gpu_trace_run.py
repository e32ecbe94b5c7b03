"""bin/trace_run as a user runs it: a model folder, steps on standard input, logits in files.
The same requests are replayed whole, with their last 32 tokens one by one, and in batches of
unequal lengths on a cache that forces slots and pages to be used again; float32 and bfloat16."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT, TINY, random_prompt
from helpers import assert_logits_close, plain_logits

pytestmark = pytest.mark.gpu


def run_trace(folder, dtype, steps, out_dir, max_tokens):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
           "--out", str(out_dir), "--max-tokens", str(max_tokens)]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run(cmd, input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    done = [int(line.split()[1]) for line in p.stdout.splitlines() if line.startswith("done ")]
    assert done == [s["step"] for s in steps]
    return p


def read_logits(out_dir, step, vocab):
    return np.fromfile(os.path.join(out_dir, f"{step}.f32"), dtype="<f4").reshape(-1, vocab)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B"])
def test_replay_three_ways(model_folders, tmp_path, name, dtype):
    folder, vocab = model_folders[name], TINY[name]["vocab_size"]
    rng = np.random.default_rng(11)
    reqs = {rid: random_prompt(rng, vocab, n) for rid, n in (("a", 70), ("b", 33), ("c", 129), ("d", 40))}
    steps, expect = [], {}            # expect[step] = list of (request, first position, count)
    n = 0

    def add(entries, end=()):
        nonlocal n
        steps.append({"step": n, "entries": entries, "end": list(end)})
        n += 1
        return n - 1

    # 1. each request alone and whole
    for rid, toks in reqs.items():
        s = add([{"id": rid + "1", "tokens": toks, "want": list(range(len(toks)))}], end=[rid + "1"])
        expect[s] = [(rid, 0, len(toks))]
    # 2. the last 32 tokens one by one
    for rid, toks in reqs.items():
        head = len(toks) - 32
        s = add([{"id": rid + "2", "tokens": toks[:head], "want": list(range(head))}])
        expect[s] = [(rid, 0, head)]
        for i in range(head, len(toks)):
            s = add([{"id": rid + "2", "tokens": [toks[i]], "want": [0]}], end=[rid + "2"] if i == len(toks) - 1 else ())
            expect[s] = [(rid, i, 1)]
    # 3. batches of unequal lengths; the shorter requests end earlier; one batch after another
    for batch, prompt_lens in ((("a", "b"), (50, 20)), (("c", "d"), (100, 33)), (("b", "a", "d"), (1, 64, 17))):
        tag = "3" + "".join(batch)
        s = add([{"id": r + tag, "tokens": reqs[r][:pl], "want": [pl - 1]} for r, pl in zip(batch, prompt_lens)])
        expect[s] = [(r, pl - 1, 1) for r, pl in zip(batch, prompt_lens)]
        pos = dict(zip(batch, prompt_lens))
        live = [r for r in batch if pos[r] < len(reqs[r])]
        while live:
            ending = [r for r in live if pos[r] + 1 == len(reqs[r])]
            s = add([{"id": r + tag, "tokens": [reqs[r][pos[r]]], "want": [0]} for r in live],
                    end=[r + tag for r in ending])
            expect[s] = [(r, pos[r], 1) for r in live]
            for r in live:
                pos[r] += 1
            live = [r for r in live if r not in ending]
    # a step that wants nothing writes no file
    quiet = add([{"id": "q", "tokens": reqs["b"][:5], "want": []}], end=["q"])

    out_dir = tmp_path / "out"
    # the cache holds the largest batch (129 + 40 tokens, each rounded up to 64) and no more
    run_trace(folder, dtype, steps, out_dir, max_tokens=192 + 64)
    assert not os.path.exists(out_dir / f"{quiet}.f32")
    for s, parts in expect.items():
        got = read_logits(out_dir, s, vocab)
        want = np.concatenate([plain_logits(folder, reqs[r])[p0:p0 + cnt] for r, p0, cnt in parts])
        assert_logits_close(got, want, dtype, f"{name} step {s}")


def plain_dump(folder, tokens, path, want):
    """The plain implementation's intermediates for one whole request, in the dump format."""
    from plain import qwen2_plain as P
    cfg, w = P.load_model(folder)
    pos = np.arange(len(tokens))
    lines = ["# plain implementation"]

    def emit(name, a):
        a = np.asarray(a, np.float32).reshape(-1)
        lines.append(f"@ {name} f32 {a.size} 1 1 1")
        lines.extend("%.9g" % v for v in a.tolist())
    x = P.embedding(w["model.embed_tokens.weight"], tokens)
    emit("embedding", x)
    for layer in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{layer}."
        h = P.rms_norm(x, w[p + "input_layernorm.weight"], cfg["rms_norm_eps"])
        x1 = (P.self_attention(h, pos, w, p + "self_attn.", cfg) + x).astype(np.float32)
        emit(f"entry{layer}.after_mixer", x1)
        x = P.block(x, pos, w, layer, cfg)
        emit(f"entry{layer}.after_ffn", x)
    emit("logits", P.lm_head(x, w, cfg)[want])
    with open(path, "w") as f:
        f.write("\n".join(lines) + "\n")


def test_dumps_of_intermediates_and_their_comparison(model_folders, tmp_path):
    """--trace writes every step's residual stream after each mixer and feed-forward; the
    comparison tool finds them equal to the plain implementation's in 32-bit, and names the first
    entry that differs when one layer's weights do."""
    import shutil

    import torch
    from safetensors import safe_open
    from safetensors.torch import save_file
    folder, vocab = model_folders["B"], TINY["B"]["vocab_size"]
    tokens = random_prompt(np.random.default_rng(3), vocab, 21)
    want = [0, 20]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens, "want": want}], "end": ["a"]}]
    cmd = lambda model, out: [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", model,  # noqa: E731
                              "--dtype", "float32", "--out", str(out), "--max-tokens", "64", "--trace", str(out)]
    text = "".join(json.dumps(s) + "\n" for s in steps)
    p = subprocess.run(cmd(folder, tmp_path / "good"), input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    plain_dump(folder, tokens, tmp_path / "plain.dump", want)
    compare = [sys.executable, os.path.join(ROOT, "bin", "compare_dumps")]
    r = subprocess.run(compare + [str(tmp_path / "plain.dump"), str(tmp_path / "good" / "0.dump"), "1e-4"],
                       capture_output=True, text=True)
    assert r.returncode == 0 and "dumps agree" in r.stdout, r.stdout + r.stderr
    names = [line.split()[0] for line in r.stdout.splitlines() if line.startswith(("embedding", "entry", "logits"))]
    assert names == ["embedding"] + [f"entry{i}.after_{w}" for i in range(3) for w in ("mixer", "ffn")] + ["logits"]
    # the same model with layer 1's down projection changed: the first difference is after that feed-forward
    bad = tmp_path / "bad_model"
    os.makedirs(bad)
    shutil.copy(os.path.join(folder, "config.json"), bad / "config.json")
    tensors = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            t = f.get_tensor(name)
            tensors[name] = (t * 1.5).to(t.dtype) if name == "model.layers.1.mlp.down_proj.weight" else t
    save_file(tensors, str(bad / "model.safetensors"), metadata={"format": "pt"})
    p = subprocess.run(cmd(str(bad), tmp_path / "bad"), input=text, capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    r = subprocess.run(compare + [str(tmp_path / "plain.dump"), str(tmp_path / "bad" / "0.dump")],
                       capture_output=True, text=True)
    assert r.returncode == 1 and "first tensor out of tolerance: entry1.after_ffn" in r.stdout, r.stdout
    assert subprocess.run(compare, capture_output=True, text=True).returncode == 2
    del torch


def test_trace_run_reports_bad_input(model_folders, tmp_path):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", "float32",
           "--out", str(tmp_path / "o"), "--max-tokens", "64"]
    p = subprocess.run(cmd, input="", capture_output=True, text=True, timeout=120)
    assert p.returncode != 0 and "config.json" in p.stderr

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


def test_trace_run_reports_bad_input(model_folders, tmp_path):
    cmd = [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(tmp_path), "--dtype", "float32",
           "--out", str(tmp_path / "o"), "--max-tokens", "64"]
    p = subprocess.run(cmd, input="", capture_output=True, text=True, timeout=120)
    assert p.returncode != 0 and "config.json" in p.stderr

"""Command line: token ids in, token ids out.

Options follow the reference's token tool
(/root/reference/tools/baseline/gen_from_tokens.cpp:34-50: ``-m``, ``--tokens``,
``-n``, ``--ctx``; usage on stderr, exit status 2) and its sampling struct's
field names (/root/reference/capi/include/sonicboom/capi.h:663-676).  The
tokens file holds one prompt per line, ids separated by blanks; the output is
one line of produced ids per prompt (gen_from_tokens.cpp:92-96).
"""
from __future__ import annotations

import argparse
import json
import sys

USAGE = ("sb-gen (-m MODEL_DIR | --random CONFIG.json [--seed S]) --tokens FILE [-n N] [--ctx N]\n"
         "              [--dtype bfloat16|float32] [--batch B] [--temperature T] [--top-k K] [--top-p P]\n"
         "              [--min-p P] [--sample-seed S] [--repeat-penalty R] [--repeat-last-n N]\n"
         "              [--presence-penalty X] [--frequency-penalty X] [--stop ID,ID,...]\n")


class _Parser(argparse.ArgumentParser):
    def error(self, message):
        sys.stderr.write(f"sb-gen: {message}\nusage: {USAGE}")
        raise SystemExit(2)


def parse(argv):
    p = _Parser(prog="sb-gen", add_help=True, usage=USAGE)
    p.add_argument("-m", "--model", help="folder with config.json and model.safetensors")
    p.add_argument("--random", metavar="CONFIG.json", help="random weights for this configuration")
    p.add_argument("--seed", type=int, default=0, help="seed of the random weights")
    p.add_argument("--dtype", choices=("bfloat16", "float32", "bf16", "fp32"), default="bfloat16")
    p.add_argument("--tokens", required=True, help="file with one prompt of token ids per line")
    p.add_argument("-n", type=int, default=16, dest="n", help="tokens to produce per prompt (max_tokens)")
    p.add_argument("--ctx", type=int, default=0, help="cache size in tokens (default: what the prompts need)")
    p.add_argument("--batch", type=int, default=64, help="most prompts that run together")
    p.add_argument("--temperature", type=float, default=0.0)
    p.add_argument("--top-k", type=int, default=0)
    p.add_argument("--top-p", type=float, default=1.0)
    p.add_argument("--min-p", type=float, default=0.0)
    p.add_argument("--sample-seed", type=int, default=0, help="seed of the sampling draws")
    p.add_argument("--repeat-penalty", type=float, default=1.0)
    p.add_argument("--repeat-last-n", type=int, default=64)
    p.add_argument("--presence-penalty", type=float, default=0.0)
    p.add_argument("--frequency-penalty", type=float, default=0.0)
    p.add_argument("--stop", default=None, help="comma separated stop token ids (default: the model's eos ids)")
    a = p.parse_args(argv)
    if bool(a.model) == bool(a.random):
        p.error("give exactly one of -m and --random")
    a.dtype = {"bf16": "bfloat16", "fp32": "float32"}.get(a.dtype, a.dtype)
    return a


def read_prompts(path):
    try:
        with open(path) as f:
            prompts = [[int(t) for t in line.split()] for line in f if line.strip()]
    except FileNotFoundError:
        sys.stderr.write(f"tokens file not found: {path}\n")
        raise SystemExit(2)
    except ValueError as e:
        sys.stderr.write(f"tokens file {path}: {e}\n")
        raise SystemExit(2)
    if not prompts:
        sys.stderr.write(f"tokens file empty: {path}\n")
        raise SystemExit(2)
    return prompts


def main(argv=None) -> int:
    a = parse(sys.argv[1:] if argv is None else argv)
    prompts = read_prompts(a.tokens)
    from .api import Model
    from .cache import PAGE, pages_for
    try:
        if a.model:
            model = Model.load(a.model, a.dtype)
        else:
            with open(a.random) as f:
                model = Model.random(json.load(f), a.seed, a.dtype)
        ctx = a.ctx
        if ctx <= 0:
            group = sorted(len(p) for p in prompts)[-a.batch:]
            ctx = sum(pages_for(n + a.n) for n in group) * PAGE
        session = model.session(ctx)
        stop = None if a.stop is None else [int(t) for t in a.stop.split(",") if t.strip()]
        outs = session.generate(
            prompts, temperature=a.temperature, top_p=a.top_p, top_k=a.top_k, seed=a.sample_seed,
            max_tokens=a.n, min_p=a.min_p, repeat_penalty=a.repeat_penalty, repeat_last_n=a.repeat_last_n,
            presence_penalty=a.presence_penalty, frequency_penalty=a.frequency_penalty, stop_tokens=stop,
            max_batch=a.batch)
    except (ValueError, RuntimeError, OSError) as e:
        sys.stderr.write(f"sb-gen: {e}\n")
        return 1
    for out in outs:
        print(" ".join(str(t) for t in out))
    return 0


if __name__ == "__main__":
    raise SystemExit(main())

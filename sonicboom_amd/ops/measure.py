"""Timings of single kernels on the GPU at hand, for choosing between their forms.

    python -m sonicboom_amd.ops.measure attention-decode --heads 28 --kv-heads 4 --head-dim 128 \\
        --batch 64 --keys 2060 [--pages-per-wave 0,1,2,4,8,16]
    python -m sonicboom_amd.ops.measure product --rows 64 --out 18944 --in 3584 --gated \\
        [--kernels stream,skinny,tiled]

Every timed call reads memory that the calls before it did not leave in the caches (the
operands rotate through about 1.5 GB), as a decode step finds it.  Times are means of back-to-back
launches between two events; a kernel of a few microseconds is then bound by the launches
themselves, so read those against each other only.
"""
from __future__ import annotations

import argparse
import sys

import torch

from . import kernels as K
from . import library

DEV = "cuda:0"


def _time(fn, n_sets: int, rounds: int = 4) -> float:
    """Mean microseconds of fn(i) over rounds * n_sets calls, after one pass to warm up."""
    for i in range(n_sets):
        fn(i)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for i in range(rounds * n_sets):
        fn(i)
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) * 1e3 / (rounds * n_sets)


def attention_decode(a) -> None:
    hq, hkv, hd, batch, keys = a.heads, a.kv_heads, a.head_dim, a.batch, a.keys
    used = keys // K.PAGE + 1
    width = (used + 15) // 16 * 16                      # as the decode loop rounds the table
    bytes_read = batch * used * hkv * K.PAGE * hd * 2 * 2
    n_sets = max(2, min(8, int(1.5e9 // bytes_read)))
    per_set = batch * width
    kc = torch.randn(per_set * n_sets, hkv, K.PAGE, hd, device=DEV, dtype=torch.bfloat16)
    vc = torch.randn(per_set * n_sets, hkv, hd, K.PAGE, device=DEV, dtype=torch.bfloat16)
    q = torch.randn(batch, hq * hd, device=DEV, dtype=torch.bfloat16)
    tables = [(torch.arange(per_set, device=DEV, dtype=torch.int32) + s * per_set).reshape(batch, width).contiguous()
              for s in range(n_sets)]
    pos = torch.full((batch,), keys, device=DEV, dtype=torch.int32)
    print(f"decode attention: {batch} sequences of {keys + 1} keys, {hq} heads on {hkv} kv heads of {hd}; "
          f"page table {width} wide; {bytes_read / 1e6:.1f} MB of keys and values a call")
    for pages in a.pages_per_wave:
        with K.attention_decode_pages_per_wave(hd, pages):
            us = _time(lambda i: K.attention_decode_mfma(q, kc, vc, tables[i % n_sets], pos, hq, hkv, hd, hd ** -0.5, 0),
                       n_sets)
        label = "chosen by the launcher" if pages == 0 else f"{pages} pages per wave"
        print(f"  {label:24s} {us:8.1f} us  {bytes_read / us / 1e6:5.2f} TB/s", flush=True)


def product(a) -> None:
    rows, n, k, gated = a.rows, a.out, getattr(a, "in"), a.gated
    w_rows = n * (2 if gated else 1)
    n_sets = max(2, int(1.2e9 // (w_rows * k * 2)))
    ws = [K.pack_weight(torch.randn(w_rows, k, device=DEV, dtype=torch.bfloat16) * 0.02, gated) for _ in range(n_sets)]
    x = torch.randn(rows, k, device=DEV, dtype=torch.bfloat16)
    print(f"product: {rows} rows, {n} outputs{' (gated)' if gated else ''}, inner size {k}; "
          f"{w_rows * k * 2 / 1e6:.1f} MB of weights a call")
    for which in a.kernels:
        with K.gemm_few_rows_kernel(None if which == "chosen" else which):
            try:
                us = _time(lambda i: K.gemm_bf16(x, ws[i % n_sets], None, None, torch.bfloat16, gated=gated,
                                                 packed_shape=(w_rows, k)), n_sets, rounds=3)
            except library.KernelLibraryError as e:
                print(f"  {which:8s} refused: {e}")
                continue
        print(f"  {which:8s} {us:8.1f} us  {w_rows * k * 2 / us / 1e6:5.2f} TB/s", flush=True)


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="python -m sonicboom_amd.ops.measure", description=__doc__.split("\n")[0])
    sub = ap.add_subparsers(dest="what", required=True)
    ad = sub.add_parser("attention-decode")
    ad.add_argument("--heads", type=int, default=28)
    ad.add_argument("--kv-heads", type=int, default=4)
    ad.add_argument("--head-dim", type=int, default=128)
    ad.add_argument("--batch", type=int, default=64)
    ad.add_argument("--keys", type=int, default=2060, help="cached keys per sequence")
    ad.add_argument("--pages-per-wave", type=lambda s: [int(v) for v in s.split(",")], default=[0, 1, 2, 4, 8, 16])
    pr = sub.add_parser("product")
    pr.add_argument("--rows", type=int, default=64)
    pr.add_argument("--out", type=int, default=18944)
    pr.add_argument("--in", type=int, default=3584)
    pr.add_argument("--gated", action="store_true")
    pr.add_argument("--kernels", type=lambda s: s.split(","), default=["chosen", "stream", "skinny", "tiled"])
    a = ap.parse_args(argv)
    if not torch.cuda.is_available():
        print("no GPU: these measurements need an MI355X", file=sys.stderr)
        return 2
    (attention_decode if a.what == "attention-decode" else product)(a)
    return 0


if __name__ == "__main__":
    sys.exit(main())

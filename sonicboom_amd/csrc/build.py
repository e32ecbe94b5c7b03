"""Compiles the HIP sources of this folder for gfx950 into shared libraries.

Two kinds of library come out of it:

* ``libsbhip.so`` — every kernel whose code does not depend on the model;
* ``libsbattn_hd<N>.so`` — the MFMA attention kernels for one head size N,
  compiled when a model of that head size is first built (or ahead of time by
  :func:`build_all`).

A library lives in ``_build/`` beside the sources together with a stamp that
holds the hash of the sources and flags it was made from.  :func:`ensure`
loads nothing; it returns the path of an up-to-date library and compiles it
first when the stamp does not match, printing a line per file and a line every
few seconds while the compiler runs.  When the source folder cannot be written
the libraries go to a per-user folder under the system's temporary directory.
"""
from __future__ import annotations

import hashlib
import os
import shutil
import subprocess
import sys
import tempfile
import threading
import time
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
ARCH = "gfx950"

# Packed FP32 instructions are switched off for every kernel of the library.
FLAGS = [
    "-O3", "-std=c++17", f"--offload-arch={ARCH}", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-format-security", "-Wno-unused-result",
]

CORE_SOURCES = [
    "status.hip", "embed_norm.hip", "elementwise.hip", "gemm_plain.hip", "rope_kv.hip",
    "attention_plain.hip", "sampling.hip", "gemm_skinny.hip", "gemm_stream.hip", "gemm_mfma.hip",
    "random_fill.hip",
]
HEADERS = ["common.h", "sb_hip.h", "mfma.h"]
ATTN_SOURCES = ["attention_mfma.hip"]

# Head sizes compiled ahead of time by build_all(): every size the kernels take.
PREBUILT_HEAD_DIMS = tuple(range(16, 257, 16))
MAX_HEAD_DIM = 256


class BuildError(RuntimeError):
    pass


def _log(msg: str) -> None:
    print(f"[sonicboom_amd build] {msg}", file=sys.stderr, flush=True)


def hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise BuildError("hipcc not found (looked at $HIPCC, PATH and /opt/rocm/bin/hipcc)")


_BUILD_DIR = None


def build_dir() -> str:
    """``_build/`` beside the sources, or a per-user folder when that cannot be written."""
    global _BUILD_DIR
    if _BUILD_DIR is None:
        d = os.path.join(HERE, "_build")
        try:
            os.makedirs(d, exist_ok=True)
            fd, probe = tempfile.mkstemp(dir=d)
            os.close(fd)
            os.remove(probe)
        except OSError:
            d = os.path.join(tempfile.gettempdir(), f"sonicboom_amd_build_{os.getuid()}")
            os.makedirs(d, exist_ok=True)
        _BUILD_DIR = d
    return _BUILD_DIR


def _existing(names):
    return [n for n in names if os.path.exists(os.path.join(HERE, n))]


def _hash(sources, defines) -> str:
    h = hashlib.sha256()
    h.update(" ".join(FLAGS + sorted(defines)).encode())
    for name in sorted(sources) + sorted(_existing(HEADERS)):
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()


def _run(cmd, what):
    env = dict(os.environ)
    env.setdefault("HOME", tempfile.gettempdir())   # the compiler wants some HOME
    p = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, env=env)
    if p.returncode != 0:
        raise BuildError(f"{what} failed ({p.returncode}):\n{' '.join(cmd)}\n{p.stdout}")
    return p.stdout


def _compile_library(lib_name, sources, defines, jobs) -> str:
    out_dir = build_dir()
    lib = os.path.join(out_dir, lib_name)
    stamp = lib + ".stamp"
    want = _hash(sources, defines)
    cc = hipcc()
    obj_dir = os.path.join(out_dir, "obj_" + lib_name.replace(".so", ""))
    os.makedirs(obj_dir, exist_ok=True)
    flags = FLAGS + [f"-D{d}" for d in defines] + [f'-DSB_BUILD_FLAGS="{ARCH} -O3 no-packed-fp32"', f"-I{HERE}"]
    _log(f"compiling {lib_name} for {ARCH}: {len(sources)} file(s), {jobs} at a time")
    t0 = time.time()
    done = threading.Event()

    def heartbeat():
        while not done.wait(15.0):
            _log(f"  ... still compiling {lib_name} ({time.time() - t0:.0f} s)")

    hb = threading.Thread(target=heartbeat, daemon=True)
    hb.start()
    try:
        def one(src):
            obj = os.path.join(obj_dir, src.replace(".hip", ".o"))
            _run([cc, *flags, "-c", os.path.join(HERE, src), "-o", obj], f"compiling {src}")
            _log(f"  compiled {src} ({time.time() - t0:.0f} s)")
            return obj
        with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
            objs = list(ex.map(one, sources))
        tmp = lib + f".tmp{os.getpid()}"
        _run([cc, "-shared", "-fPIC", f"--offload-arch={ARCH}", *objs, "-o", tmp], f"linking {lib_name}")
        os.replace(tmp, lib)
        with open(stamp, "w") as f:
            f.write(want)
    finally:
        done.set()
    _log(f"built {lib} in {time.time() - t0:.0f} s")
    return lib


def _jobs() -> int:
    try:
        n = int(os.environ.get("MAX_JOBS", "0"))
    except ValueError:
        n = 0
    return n if n > 0 else min(8, os.cpu_count() or 1)


def _ensure(lib_name, sources, defines, force) -> str:
    sources = _existing(sources)
    if not sources:
        raise BuildError(f"no sources for {lib_name} in {HERE}")
    out_dir = build_dir()
    lib = os.path.join(out_dir, lib_name)
    stamp = lib + ".stamp"
    want = _hash(sources, defines)
    if not force and os.path.exists(lib) and os.path.exists(stamp):
        with open(stamp) as f:
            if f.read().strip() == want:
                return lib
        _log(f"{lib_name} is older than its sources")
    return _compile_library(lib_name, sources, defines, _jobs())


def ensure_core(force: bool = False) -> str:
    """Path of an up-to-date ``libsbhip.so`` (compiled now if need be)."""
    return _ensure("libsbhip.so", CORE_SOURCES, [], force)


def ensure_attention(head_dim: int, force: bool = False) -> str:
    """Path of the MFMA attention library for one head size."""
    if head_dim % 16 or not 16 <= head_dim <= MAX_HEAD_DIM:
        raise BuildError(f"the MFMA attention kernels take head sizes 16..{MAX_HEAD_DIM} in steps of 16, not {head_dim}")
    return _ensure(f"libsbattn_hd{head_dim}.so", ATTN_SOURCES, [f"SB_HEAD_DIM={head_dim}"], force)


def ensure_plain_host(force: bool = False) -> str:
    """Path of ``libsbplain.so``: the kernels' plain C++ twins on host memory (plain_host.cpp),
    compiled with the host compiler.  The tests compare the kernels with them."""
    out_dir = build_dir()
    lib, stamp = os.path.join(out_dir, "libsbplain.so"), os.path.join(out_dir, "libsbplain.so.stamp")
    src, header = os.path.join(HERE, "plain_host.cpp"), os.path.join(HERE, "plain_host.h")
    h = hashlib.sha256()
    for path in (src, header, os.path.join(HERE, "sb_hip.h")):
        with open(path, "rb") as f:
            h.update(f.read())
    want = h.hexdigest()
    if not force and os.path.exists(lib) and os.path.exists(stamp):
        with open(stamp) as f:
            if f.read().strip() == want:
                return lib
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("amdclang++")
    if not cxx:
        raise BuildError("no host C++ compiler (g++) for the plain twins")
    tmp = lib + f".tmp{os.getpid()}"
    # no contraction into fused multiply-adds: the arithmetic is what the source says
    _run([cxx, "-O2", "-std=c++17", "-shared", "-fPIC", "-ffp-contract=off", "-Wall", src, "-o", tmp],
         "compiling plain_host.cpp")
    os.replace(tmp, lib)
    with open(stamp, "w") as f:
        f.write(want)
    _log(f"built {lib}")
    return lib


def build_all(force: bool = True) -> None:
    """Compile the core library, the plain host twins and the attention libraries of the usual
    head sizes."""
    ensure_core(force=force)
    ensure_plain_host(force=force)
    if _existing(ATTN_SOURCES):
        with ThreadPoolExecutor(max_workers=_jobs()) as ex:
            list(ex.map(lambda hd: ensure_attention(hd, force=force), PREBUILT_HEAD_DIMS))


if __name__ == "__main__":
    build_all(force="--force" in sys.argv or True)

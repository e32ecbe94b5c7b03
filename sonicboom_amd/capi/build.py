"""Builds the C interface library and the C++ command line next to it (``_build/``), with the
host compiler and the running interpreter's headers and library."""
from __future__ import annotations

import os
import shutil
import subprocess
import sysconfig

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "_build")
LIBRARY = os.path.join(OUT, "libsonicboom_amd.so")
COMMAND = os.path.join(OUT, "sb-gen")


class CapiBuildError(RuntimeError):
    pass


def _run(cmd):
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise CapiBuildError(f"{' '.join(cmd)}\n{r.stdout}{r.stderr}")


def _stale(target, sources):
    if not os.path.exists(target):
        return True
    t = os.path.getmtime(target)
    return any(os.path.getmtime(s) > t for s in sources)


def build_sanitized():
    """The library and the command line once more under ``_build/sanitize/`` with the host
    compiler's address and undefined-behaviour sanitizers, for runs of the host code on a machine
    without a GPU (the GPU boxes run no sanitizer).  Returns (library, command, environment a
    program linked against it needs)."""
    cxx = shutil.which("g++") or shutil.which("c++")
    if not cxx:
        raise CapiBuildError("no C++ compiler (g++) on PATH")
    out = os.path.join(OUT, "sanitize")
    os.makedirs(out, exist_ok=True)
    include = sysconfig.get_paths()["include"]
    libdir = sysconfig.get_config_var("LIBDIR") or "/usr/lib"
    version = sysconfig.get_config_var("LDVERSION") or sysconfig.get_config_var("VERSION")
    soname = sysconfig.get_config_var("INSTSONAME") or f"libpython{version}.so"
    san = ["-fsanitize=address,undefined", "-fno-omit-frame-pointer", "-g", "-O1"]
    lib, cmd = os.path.join(out, "libsonicboom_amd.so"), os.path.join(out, "sb-gen")
    _run([cxx, *san, "-std=c++17", "-shared", "-fPIC", "-Wall", f'-DSB_LIBPYTHON="{soname}"',
          os.path.join(HERE, "capi.cpp"), f"-I{HERE}", f"-I{include}", f"-L{libdir}", f"-lpython{version}", "-ldl",
          "-o", lib])
    _run([cxx, *san, "-std=c++17", "-Wall", os.path.join(HERE, "sb_gen.cpp"), f"-I{HERE}", f"-L{out}",
          "-lsonicboom_amd", "-Wl,-rpath,$ORIGIN", "-o", cmd])
    # the interpreter's own allocations at exit are not this library's leaks
    env = {"ASAN_OPTIONS": "detect_leaks=0:abort_on_error=1", "UBSAN_OPTIONS": "halt_on_error=1:print_stacktrace=1"}
    return lib, cmd, env


def build(force: bool = False):
    """Compile what is missing or older than its sources; returns (library, command)."""
    cxx = shutil.which("g++") or shutil.which("c++") or shutil.which("amdclang++")
    if not cxx:
        raise CapiBuildError("no C++ compiler (g++) on PATH")
    os.makedirs(OUT, exist_ok=True)
    include = sysconfig.get_paths()["include"]
    libdir = sysconfig.get_config_var("LIBDIR") or "/usr/lib"
    version = sysconfig.get_config_var("LDVERSION") or sysconfig.get_config_var("VERSION")
    soname = sysconfig.get_config_var("INSTSONAME") or f"libpython{version}.so"
    header = os.path.join(HERE, "sonicboom_amd.h")
    src = os.path.join(HERE, "capi.cpp")
    if force or _stale(LIBRARY, [src, header]):
        _run([cxx, "-O2", "-std=c++17", "-shared", "-fPIC", "-Wall", f'-DSB_LIBPYTHON="{soname}"', src, f"-I{HERE}",
              f"-I{include}", f"-L{libdir}", f"-lpython{version}", "-ldl", "-o", LIBRARY])
    main = os.path.join(HERE, "sb_gen.cpp")
    if force or _stale(COMMAND, [main, header, LIBRARY]):
        _run([cxx, "-O2", "-std=c++17", "-Wall", main, f"-I{HERE}", f"-L{OUT}", "-lsonicboom_amd",
              "-Wl,-rpath,$ORIGIN", "-o", COMMAND])
    return LIBRARY, COMMAND


if __name__ == "__main__":
    import sys
    if "--sanitize" in sys.argv:
        print(*build_sanitized()[:2], sep="\n")
    else:
        print(*build(force=True), sep="\n")

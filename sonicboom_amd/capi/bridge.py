"""What the C interface calls.  Every entry goes through :func:`call`, which turns any
exception into ``(status, message)`` so that none reaches C; results are plain Python objects,
and bulk data is copied straight to the caller's buffers by address."""
from __future__ import annotations

import ctypes
import json

# the values of boom_status in sonicboom_amd.h
OK, ERR_CONFIG, ERR_WEIGHT, ERR_BINDING, ERR_RUNTIME, ERR_INTERNAL, ERR_UNSUPPORTED = 0, 1, 2, 4, 5, 6, 7


def _status_of(exc: BaseException) -> int:
    from ..cache.paged import CacheError
    from ..config.base import ConfigError
    from ..csrc.build import BuildError
    from ..engine.step import StepError
    from ..ops.library import KernelLibraryError
    from ..weights.loader import WeightError
    from ..weights.safetensors_io import SafetensorsError
    if isinstance(exc, (WeightError, SafetensorsError)):
        return ERR_WEIGHT
    if isinstance(exc, ConfigError):
        return ERR_CONFIG
    if isinstance(exc, (StepError, CacheError)):
        return ERR_BINDING
    if isinstance(exc, (KernelLibraryError, BuildError)):
        return ERR_UNSUPPORTED if "unsupported" in str(exc).lower() else ERR_RUNTIME
    if isinstance(exc, FileNotFoundError):
        return ERR_CONFIG
    if isinstance(exc, (ValueError, KeyError, IndexError, TypeError)):
        return ERR_BINDING
    if isinstance(exc, (RuntimeError, OSError)):
        return ERR_RUNTIME
    return ERR_INTERNAL


def call(name: str, *args):
    """Run entry ``name``; (0, result) or (status, "kind: message")."""
    try:
        return OK, _ENTRIES[name](*args)
    except BaseException as exc:      # nothing may escape into C
        return _status_of(exc), f"{type(exc).__name__}: {exc}"


def _model_load(folder, dtype, device):
    from ..api import Model
    return Model.load(folder, dtype=dtype or "bfloat16", device=f"cuda:{device}")


def _model_random(config_path, seed, dtype, device):
    from ..api import Model
    with open(config_path) as f:
        cfg = json.load(f)
    return Model.random(cfg, seed=seed, dtype=dtype or "bfloat16", device=f"cuda:{device}")


def _session_new(model, max_tokens):
    return model.session(int(max_tokens))


def _step(session, entries, out_addr):
    """entries: [(slot, [tokens], [want])]; float32 logits copied to out_addr; returns the count."""
    logits = session.step([(int(s), list(t), list(w)) for s, t, w in entries])
    host = logits.detach().float().cpu().contiguous()
    n = host.numel()
    if n:
        ctypes.memmove(out_addr, host.data_ptr(), n * 4)
    return n


def _generate(session, prompts, sampling, stop, cb_addr, user_addr, out_addr, n_out_addr):
    max_tokens = int(sampling["max_tokens"])
    callback = None
    if cb_addr:
        proto = ctypes.CFUNCTYPE(ctypes.c_int, ctypes.c_void_p, ctypes.c_uint32, ctypes.c_int32)
        fn = proto(cb_addr)
        callback = lambda i, t: bool(fn(user_addr, i, t))      # noqa: E731
    outs = session.generate(prompts, stop_tokens=stop, callback=callback, **sampling)
    out = (ctypes.c_int32 * (max_tokens * len(prompts))).from_address(out_addr) if prompts and max_tokens else None
    counts = (ctypes.c_uint32 * len(prompts)).from_address(n_out_addr) if prompts else None
    for i, toks in enumerate(outs):
        counts[i] = len(toks)
        for j, t in enumerate(toks[:max_tokens]):
            out[i * max_tokens + j] = t
    return len(outs)


def _session_keep(session, on):
    session.keep = bool(on)
    if not session.keep:
        session.forget()


def _session_reused(session, out_addr, cap):
    """Counts of the last generate's reused tokens, copied to out_addr when cap holds them."""
    counts = session.reused
    if counts and cap >= len(counts):
        buf = (ctypes.c_uint64 * len(counts)).from_address(out_addr)
        for i, n in enumerate(counts):
            buf[i] = n
    return len(counts)


def _build_info():
    from .. import __version__
    from ..ops import library
    info = {"package": "sonicboom_amd", "version": __version__}
    try:
        info["kernels"] = library.core().sb_build_info().decode()
        info["kernel_libraries"] = library.loaded_paths()
    except Exception as exc:          # no GPU or no compiler: say so instead of failing
        info["kernels"] = f"unavailable: {exc}"
    return json.dumps(info)


_ENTRIES = {
    "model_load": _model_load,
    "model_random": _model_random,
    "model_arch": lambda m: m.arch,
    "model_eos": lambda m: [int(t) for t in m.eos],
    "model_vocab": lambda m: int(m.vocab_size),
    "session_new": _session_new,
    "session_vocab": lambda s: int(s.model.vocab_size),
    "slot_alloc": lambda s: int(s.alloc_slot()),
    "slot_free": lambda s, slot: s.free_slot(int(slot)),
    "step": _step,
    "generate": _generate,
    "session_keep": _session_keep,
    "session_reused": _session_reused,
    "build_info": _build_info,
}

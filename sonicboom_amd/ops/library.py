"""Loads the HIP kernel libraries through ctypes and declares their entry points.

There is no fallback: when a library cannot be built or loaded, or the GPU is
missing, the call that needs it raises :class:`KernelLibraryError`.
"""
from __future__ import annotations

import ctypes
import threading
from ctypes import c_char_p, c_double, c_float, c_int, c_size_t, c_uint64, c_void_p

from ..csrc import build


class KernelLibraryError(RuntimeError):
    """The HIP kernel library is missing, or a kernel refused its arguments."""


_P, _I, _F, _Z = c_void_p, c_int, c_float, c_size_t

_CORE_SIGNATURES = {
    "sb_embed": [_P, _P, _I, _P, _I, _I, _I, _P],
    "sb_rmsnorm": [_P, _I, _P, _P, _I, _P, _I, _I, _F, _P],
    "sb_gemm": [_P, _I, _P, _I, _P, _I, _P, _I, _P, _I, _I, _I, _P],
    "sb_silu_mul": [_P, _I, _P, _I, _I, _I, _P],
    "sb_gate_mul": [_P, _I, _P, _I, _I, _I, _I, _P],
    "sb_add_into": [_P, _P, _I, _Z, _P],
    "sb_cast": [_P, _I, _P, _I, _Z, _P],
    "sb_rope_kv_store": [_P, _I, _P, _I, _I, _I, _P, _P, _P, _I, _P, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
    "sb_reduce_resid_norm": [_P, _I, _P, _P, _I, _P, _I, _P, _I, _I, _I, _F, _I, _P],
    "sb_reduce_resid_norm_max_width": [],
    "sb_attention": [_P, _P, _I, _I, _P, _P, _I, _P, _I, _I, _P, _P, _I, _I, _I, _I, _F, _I, _P],
    "sb_argmax": [_P, _P, _I, _I, _P, _P, _P],
    "sb_argmax_parts": [_I],
    "sb_penalize": [_P, _I, _P, _P, _P, _I, _F, _F, _F, _I, _P],
    "sb_top_candidates": [_P, _P, _P, _I, _I, _I, _F, _P, _P],
    "sb_mask_logits": [_P, _I, _I, _P, _I, _P],
    "sb_draw": [_P, _P, _P, _P, _I, _I, _I, _I, _F, _I, c_double, c_uint64, _P],
    "sb_draw_after": [_P, _P, _P, _P, _I, _I, _I, _I, _F, _I, c_double, c_uint64, _P],
    "sb_random_normal": [_P, _I, c_uint64, c_uint64, c_uint64, _I, c_double, c_double, _P],
}
# Entry points of later kernels; declared when the library has them.
_OPTIONAL_SIGNATURES = {
    "sb_gemm_skinny_partial_bf16": [_P, _P, _P, _I, _I, _I, _I, _P],
    "sb_gemm_skinny_slices": [_I, _I, _I],
    "sb_gemm_skinny_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _P, _Z, _P],
    "sb_gemm_mfma_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _I, _P],
    "sb_gemm_stream_bf16": [_P, _I, _P, _P, _P, _I, _P, _I, _I, _I, _I, _I, _P],
    "sb_gemm_stream_slices": [_I, _I, _I, _I],
    "sb_gemm_stream_partial_bf16": [_P, _P, _P, _I, _I, _I, _I, _P],
    "sb_gemm_mfma_slices": [_I, _I, _I, _I],
    "sb_gemm_mfma_partial_bf16": [_P, _P, _P, _I, _I, _I, _I, _P],
}
_ATTN_SIGNATURES = {
    # out, q, k_cache, v_cache, page_table, max_pages, n_pages, row_pos, part_o, part_ml, n_seqs,
    # heads_q, heads_kv, scale, window, pages per wave (0: chosen), stream
    "sb_attn_decode_bf16": [_P, _P, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _F, _I, _I, _P],
    # out, q, k_cache, v_cache, page_table, max_pages, n_pages, row_pos, tiles, n_tiles, heads_q,
    # heads_kv, scale, window, stream
    "sb_attn_prefill_bf16": [_P, _P, _P, _P, _P, _I, _I, _P, _P, _I, _I, _I, _F, _I, _I, _P],
    "sb_attn_prefill_tile_rows": [_I, _I],
    "sb_attn_prefill_tall_ok": [_I, _I],
    # out, qkv, row_stride, n_slices, bias, inv_freq, freq_factors, rot_dims, store_kv, k_cache, v_cache,
    # page_table, max_pages, n_pages, row_pos, part_o, part_ml, n_seqs, heads_q, heads_kv, scale, window,
    # pages per wave, stream
    "sb_attn_decode_rope_bf16": [_P, _P, _I, _I, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _P, _P, _P, _I, _I, _I, _F,
                                 _I, _I, _P],
    "sb_attn_decode_rope_ok": [_I, _I, _I, _I],
    "sb_attn_decode_chunks": [_I],
    "sb_attn_head_dim": [],
}

_lock = threading.Lock()
_core = None
_attn = {}


def _declare(lib, table, optional=False):
    for name, argtypes in table.items():
        try:
            fn = getattr(lib, name)
        except AttributeError:
            if optional:
                continue
            raise KernelLibraryError(f"the kernel library has no entry point {name}") from None
        fn.argtypes = argtypes
        fn.restype = c_int


def core():
    """The core library, built on first use."""
    global _core
    if _core is None:
        with _lock:
            if _core is None:
                try:
                    path = build.ensure_core()
                    lib = ctypes.CDLL(path)
                except (build.BuildError, OSError) as e:
                    raise KernelLibraryError(f"cannot load the HIP kernel library: {e}") from e
                lib.sb_last_error.restype = c_char_p
                lib.sb_build_info.restype = c_char_p
                _declare(lib, _CORE_SIGNATURES)
                _declare(lib, _OPTIONAL_SIGNATURES, optional=True)
                lib.sb_gemm_skinny_scratch.argtypes = [_I, _I, _I, _I]
                lib.sb_gemm_skinny_scratch.restype = c_size_t
                lib.sb_top_candidates_scratch.argtypes = [_I, _I]
                lib.sb_top_candidates_scratch.restype = c_size_t
                lib.sb_read_probe.argtypes = [_P, _P, _Z, _I, _P]
                lib.sb_read_probe.restype = c_int
                lib._sb_path = path
                _core = lib
    return _core


def attention_library(head_dim: int):
    """The MFMA attention library of one head size, built on first use."""
    lib = _attn.get(head_dim)
    if lib is None:
        with _lock:
            lib = _attn.get(head_dim)
            if lib is None:
                try:
                    path = build.ensure_attention(head_dim)
                    lib = ctypes.CDLL(path)
                except (build.BuildError, OSError) as e:
                    raise KernelLibraryError(f"cannot load the attention kernels for head size {head_dim}: {e}") from e
                lib.sb_attn_last_error.restype = c_char_p
                _declare(lib, _ATTN_SIGNATURES)
                for fn in (lib.sb_attn_decode_part_o, lib.sb_attn_decode_part_ml):
                    fn.argtypes = [_I, _I, _I, _I]
                    fn.restype = c_size_t
                lib._sb_path = path
                _attn[head_dim] = lib
    return lib


def loaded_paths():
    """Paths of the shared libraries this process has loaded."""
    out = []
    if _core is not None:
        out.append(_core._sb_path)
    out += [lib._sb_path for lib in _attn.values()]
    return out


def check(status: int, lib=None, error_fn="sb_last_error") -> None:
    if status != 0:
        lib = lib or core()
        msg = getattr(lib, error_fn)().decode(errors="replace")
        raise KernelLibraryError(msg or f"kernel call failed with status {status}")

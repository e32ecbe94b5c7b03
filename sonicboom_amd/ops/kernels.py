"""Python faces of the HIP kernels.

Each function checks on the host that the operands have the shapes, types and
placement its kernel and grid assume, then launches on torch's current stream.
Tensors are torch tensors on a HIP device; torch is used for memory and
streams only.  Nothing here falls back to the CPU or to a library routine:
a missing library or a refused size raises
:class:`~sonicboom_amd.ops.library.KernelLibraryError`.
"""
from __future__ import annotations

import contextlib
import math
import threading

from typing import Optional

import torch

from . import library
from .library import KernelLibraryError, check

class _Hints(threading.local):
    """Choices a test or a measurement imposes on the launchers, for the calls of its own thread
    inside a ``with`` block; every kernel call passes them as arguments (the library keeps no
    such state)."""
    few_rows_kernel = None      # "stream", "skinny", "tiled" or None
    stream = 0                  # waves | slices << 8 of the weight-streaming product
    tile_shape = -1             # of the tiled product
    decode_pages = 0            # pages per wave of decode attention


_hints = _Hints()

from ..csrc.header import PAGE          # tokens per cache page: SB_PAGE of csrc/sb_hip.h
MAX_CANDIDATES = 256

_DT = {torch.float32: 0, torch.bfloat16: 1}


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise KernelLibraryError(f"kernels take float32 and bfloat16 tensors, not {t.dtype}") from None


def _dev(*ts) -> None:
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise KernelLibraryError("kernel operands must live on the GPU (there is no CPU path)")
        if not t.is_contiguous():
            raise KernelLibraryError("kernel operands must be contiguous")


def _i32(t: torch.Tensor, n: int, what: str) -> None:
    if t.dtype != torch.int32 or t.numel() < n:
        raise KernelLibraryError(f"{what} must be int32 with at least {n} elements")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The current HIP stream's handle.  (torch's own accessor for the raw handle where it has one:
    building a Stream object for every launch cost 8 us of a launch's 14 on the host.)"""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _p(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


# --------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rows of ``table`` [vocab, width] named by int32 ``ids`` [n], as float32."""
    _dev(table, ids, out)
    if table.dim() != 2:
        raise KernelLibraryError("embedding table must be [vocab, width]")
    n = ids.numel()
    _i32(ids, n, "token ids")
    vocab, width = table.shape
    if out is None:
        out = torch.empty((n, width), dtype=torch.float32, device=table.device)
    elif out.dtype != torch.float32 or out.numel() != n * width:
        raise KernelLibraryError("embedding output must be float32 [n, width]")
    lib = library.core()
    check(lib.sb_embed(_p(out), _p(table), _dt(table), _p(ids), n, width, vocab, _stream()))
    return out


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out_dtype: torch.dtype,
            rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMS norm of float32 rows ``x`` [n, width]; ``rows`` (int32) picks and orders source rows."""
    _dev(x, weight, rows)
    if x.dtype != torch.float32 or x.dim() != 2:
        raise KernelLibraryError("rmsnorm input must be float32 [rows, width]")
    width = x.shape[1]
    if weight is not None and weight.numel() != width:
        raise KernelLibraryError(f"rmsnorm weight has {weight.numel()} elements, the rows have {width}")
    n = x.shape[0] if rows is None else rows.numel()
    if rows is not None:
        _i32(rows, n, "row index")
    y = torch.empty((n, width), dtype=out_dtype, device=x.device)
    lib = library.core()
    check(lib.sb_rmsnorm(_p(y), _dt(y), _p(x), _p(weight), _dt(weight) if weight is not None else 0,
                         _p(rows), n, width, float(eps), _stream()))
    return y


def gemm_plain(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], resid: Optional[torch.Tensor],
               out_dtype: torch.dtype, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y = x w^T (+bias) (+resid) by the plain tiled kernel; any sizes, f32 or bf16 operands."""
    _dev(x, w, bias, resid, out)
    if x.dim() != 2 or w.dim() != 2 or x.shape[1] != w.shape[1]:
        raise KernelLibraryError(f"gemm shapes do not match: x {tuple(x.shape)}, w {tuple(w.shape)}")
    t, k = x.shape
    n = w.shape[0]
    if bias is not None and bias.numel() != n:
        raise KernelLibraryError(f"bias has {bias.numel()} elements, the product has {n} columns")
    if resid is not None and (resid.dtype != torch.float32 or tuple(resid.shape) != (t, n)):
        raise KernelLibraryError("the residual must be float32 and shaped like the product")
    if out is None:
        out = torch.empty((t, n), dtype=out_dtype, device=x.device)
    elif out.dtype != out_dtype or tuple(out.shape) != (t, n):
        raise KernelLibraryError("gemm output buffer has the wrong shape or type")
    lib = library.core()
    check(lib.sb_gemm(_p(out), _dt(out), _p(x), _dt(x), _p(w), _dt(w), _p(bias),
                      _dt(bias) if bias is not None else 0, _p(resid), t, n, k, _stream()))
    return out


GATES = {"silu": 1, "gelu_tanh": 2}      # sb_gate of csrc/sb_hip.h


def gate_code(activation) -> int:
    """The kernels' number of a gate activation given by name (or already by number)."""
    if isinstance(activation, bool):
        return 1 if activation else 0
    if isinstance(activation, int):
        return activation
    try:
        return GATES[activation]
    except KeyError:
        raise KernelLibraryError(f"unknown gate activation {activation!r}; known: {sorted(GATES)}") from None


def gate_mul(gu: torch.Tensor, out_dtype: torch.dtype, activation="silu") -> torch.Tensor:
    """act(gu[:, :w]) * gu[:, w:] for gu [n, 2w]; ``activation``: "silu" or "gelu_tanh"."""
    _dev(gu)
    if gu.dim() != 2 or gu.shape[1] % 2:
        raise KernelLibraryError("gate_mul input must be [rows, 2*width]")
    n, w2 = gu.shape
    out = torch.empty((n, w2 // 2), dtype=out_dtype, device=gu.device)
    lib = library.core()
    check(lib.sb_gate_mul(_p(out), _dt(out), _p(gu), _dt(gu), n, w2 // 2, gate_code(activation), _stream()))
    return out


def silu_mul(gu: torch.Tensor, out_dtype: torch.dtype) -> torch.Tensor:
    """silu(gu[:, :w]) * gu[:, w:] for gu [n, 2w]."""
    return gate_mul(gu, out_dtype, "silu")


def add_into(resid: torch.Tensor, y: torch.Tensor) -> None:
    """resid += y (resid float32)."""
    _dev(resid, y)
    if resid.dtype != torch.float32 or resid.numel() != y.numel():
        raise KernelLibraryError("add_into needs a float32 residual and an addend of the same size")
    lib = library.core()
    check(lib.sb_add_into(_p(resid), _p(y), _dt(y), resid.numel(), _stream()))


def cast(x: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    _dev(x)
    if x.dtype == dtype:
        return x
    out = torch.empty(x.shape, dtype=dtype, device=x.device)
    lib = library.core()
    check(lib.sb_cast(_p(out), _dt(out), _p(x), _dt(x), x.numel(), _stream()))
    return out


def _check_cache(k_cache, v_cache, heads_kv, head_dim):
    if k_cache.dim() != 4 or v_cache.dim() != 4 or tuple(k_cache.shape[1:]) != (heads_kv, PAGE, head_dim) \
            or tuple(v_cache.shape[1:]) != (heads_kv, head_dim, PAGE) or k_cache.shape[0] != v_cache.shape[0] \
            or k_cache.dtype != v_cache.dtype:
        raise KernelLibraryError(
            f"cache must be keys [pages, {heads_kv}, {PAGE}, {head_dim}] and values "
            f"[pages, {heads_kv}, {head_dim}, {PAGE}], found {tuple(k_cache.shape)} and {tuple(v_cache.shape)}")


def _check_rows(row_pos, row_seq, page_table, n_rows):
    _i32(row_pos, n_rows, "row positions")
    _i32(row_seq, n_rows, "row sequence index")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")


def rope_kv_store(qkv: torch.Tensor, q_dtype: torch.dtype, inv_freq: Optional[torch.Tensor],
                  freq_factors: Optional[torch.Tensor], rot_dims: int, row_pos: torch.Tensor,
                  row_seq: torch.Tensor, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  page_table: Optional[torch.Tensor], heads_q: int, heads_kv: int, head_dim: int,
                  bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Rotate queries and keys of ``qkv`` [n, (hq+2hkv)*hd], return the queries
    [n, hq*hd] in ``q_dtype`` and store keys and values in the paged cache.
    ``heads_kv`` = 0 (and no cache) for a layer that stores nothing.  ``qkv`` may be
    [slices, n, width]: partial sums of the projection, added here in ascending order;
    ``bias`` (float32 [width]) is added after them."""
    _dev(qkv, inv_freq, freq_factors, row_pos, row_seq, k_cache, v_cache, page_table, bias)
    n_slices = 1
    if qkv.dim() == 3:
        n_slices = qkv.shape[0]
        qkv = qkv.view(-1, qkv.shape[2])
    n = qkv.shape[0] // n_slices
    need = (heads_q + 2 * heads_kv) * head_dim
    if qkv.dim() != 2 or qkv.shape[1] < need:
        raise KernelLibraryError(f"qkv rows have {qkv.shape[1]} elements, {need} are needed")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() < need):
        raise KernelLibraryError("the qkv bias must be float32 and cover a whole row")
    if inv_freq is not None:
        if inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2:
            raise KernelLibraryError("inv_freq must be float32 [rot_dims/2]")
        if freq_factors is not None and (freq_factors.dtype != torch.float32 or freq_factors.numel() < rot_dims // 2):
            raise KernelLibraryError("freq_factors must be float32 [rot_dims/2]")
    _i32(row_pos, n, "row positions")
    max_pages = n_pages = 0
    if heads_kv > 0:
        _check_cache(k_cache, v_cache, heads_kv, head_dim)
        _check_rows(row_pos, row_seq, page_table, n)
        max_pages, n_pages = page_table.shape[1], k_cache.shape[0]
    q = torch.empty((n, heads_q * head_dim), dtype=q_dtype, device=qkv.device)
    lib = library.core()
    check(lib.sb_rope_kv_store(
        _p(q), _dt(q), _p(qkv), _dt(qkv), qkv.shape[1], n_slices, _p(bias), _p(inv_freq), _p(freq_factors), rot_dims,
        _p(row_pos), _p(row_seq), _p(k_cache), _p(v_cache), _dt(k_cache) if k_cache is not None else 0,
        _p(page_table), max_pages, n_pages, n, heads_q, heads_kv, head_dim, _stream()))
    return q


def attention_plain(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                    row_pos: torch.Tensor, row_seq: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int,
                    scale: float, window: int) -> torch.Tensor:
    """Attention of rows ``q`` [n, hq*hd] over the cache, by the plain kernel."""
    _dev(q, k_cache, v_cache, page_table, row_pos, row_seq)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim:
        raise KernelLibraryError(f"queries must be [rows, {heads_q * head_dim}]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    _check_rows(row_pos, row_seq, page_table, n)
    out = torch.empty((n, heads_q * head_dim), dtype=q.dtype, device=q.device)
    lib = library.core()
    check(lib.sb_attention(_p(out), _p(q), _dt(q), q.shape[1], _p(k_cache), _p(v_cache), _dt(k_cache),
                           _p(page_table), page_table.shape[1], k_cache.shape[0], _p(row_pos), _p(row_seq),
                           n, heads_q, heads_kv, head_dim, float(scale), int(window), _stream()))
    return out


def argmax(logits: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """First maximum of every row of float32 ``logits`` [n, vocab], int32 [n]."""
    _dev(logits, out)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelLibraryError("logits must be float32 [rows, vocab]")
    n, vocab = logits.shape
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    else:
        _i32(out, n, "argmax output")
    lib = library.core()
    parts = lib.sb_argmax_parts(vocab)
    pv = pi = None
    if parts > 1:
        pv = torch.empty((n * parts,), dtype=torch.float32, device=logits.device)
        pi = torch.empty((n * parts,), dtype=torch.int32, device=logits.device)
    check(lib.sb_argmax(_p(out), _p(logits), n, vocab, _p(pv), _p(pi), _stream()))
    return out


def penalize(logits: torch.Tensor, item_row: torch.Tensor, item_token: torch.Tensor, item_count: torch.Tensor,
             repeat_penalty: float, presence_penalty: float, frequency_penalty: float, exact: bool) -> None:
    """Apply sampling penalties in place for (row, token, count) triples."""
    _dev(logits, item_row, item_token, item_count)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelLibraryError("logits must be float32 [rows, vocab]")
    n = item_row.numel()
    for t, what in ((item_row, "item rows"), (item_token, "item tokens"), (item_count, "item counts")):
        _i32(t, n, what)
    lib = library.core()
    check(lib.sb_penalize(_p(logits), logits.shape[1], _p(item_row), _p(item_token), _p(item_count), n,
                          float(repeat_penalty), float(presence_penalty), float(frequency_penalty),
                          1 if exact else 0, _stream()))


def top_candidates(logits: torch.Tensor, temperature: float, k: int = MAX_CANDIDATES):
    """The ``k`` best candidates of every row by z = logit / temperature:
    (ids int32 [n,k], z float32 [n,k]) ordered by (z descending, id ascending)."""
    _dev(logits)
    if logits.dtype != torch.float32 or logits.dim() != 2:
        raise KernelLibraryError("logits must be float32 [rows, vocab]")
    n, vocab = logits.shape
    ids = torch.empty((n, k), dtype=torch.int32, device=logits.device)
    z = torch.empty((n, k), dtype=torch.float32, device=logits.device)
    lib = library.core()
    words = lib.sb_top_candidates_scratch(n, vocab)
    scratch = torch.empty((words,), dtype=torch.int64, device=logits.device) if words else None
    check(lib.sb_top_candidates(_p(ids), _p(z), _p(logits), n, vocab, k, float(temperature), _p(scratch), _stream()))
    return ids, z


def mask_logits(logits: torch.Tensor, bitmaps: torch.Tensor) -> None:
    """The mask of constrained decoding, in place: float32 ``logits`` [rows, vocab] become -inf
    wherever the row's bitmap (uint8 [rows, bytes]: bit i & 7 of byte i >> 3 for id i; ids past the
    bitmap are not allowed) does not allow the id."""
    _dev(logits, bitmaps)
    if logits.dtype != torch.float32 or logits.dim() != 2 or not logits.is_contiguous():
        raise KernelLibraryError("logits must be contiguous float32 [rows, vocab]")
    if bitmaps.dtype != torch.uint8 or bitmaps.dim() != 2 or bitmaps.shape[0] != logits.shape[0] \
            or bitmaps.shape[1] == 0 or not bitmaps.is_contiguous():
        raise KernelLibraryError("bitmaps must be contiguous uint8 [rows, bytes], a row for every row of logits")
    check(library.core().sb_mask_logits(_p(logits), logits.shape[0], logits.shape[1], _p(bitmaps),
                                        bitmaps.shape[1], _stream()))


def draw(cand_ids: torch.Tensor, cand_z: torch.Tensor, positions, top_k: int, log_min_p: Optional[float],
         top_p: Optional[float], seed: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One token per row (int32 [n]; -1 where no candidate is kept) from the candidates that
    :func:`top_candidates` wrote: the window of 30 below the best z, top-k (0: off), min-p
    (``log_min_p`` = ln(min_p) rounded to float32, None: off), top-p (a float64, None: off) and
    the Gumbel-max draw under (seed, position of the row's new token, candidate id).
    ``positions``: one absolute position per row, a sequence or an int64 tensor on the device; or
    an int32 tensor on the device of each row's cached length before the step, whose new token then
    takes position length + 1 (a decode step's own bookkeeping: nothing comes from the host)."""
    _dev(cand_ids, cand_z)
    if cand_ids.dtype != torch.int32 or cand_z.dtype != torch.float32 or cand_ids.dim() != 2 \
            or tuple(cand_ids.shape) != tuple(cand_z.shape):
        raise KernelLibraryError("candidates must be int32 ids and float32 z of one shape [rows, k]")
    n, k = cand_ids.shape
    if not torch.is_tensor(positions):
        positions = torch.tensor([int(q) for q in positions], dtype=torch.int64).to(cand_ids.device)
    _dev(positions, out)
    if positions.dtype not in (torch.int64, torch.int32) or positions.numel() != n or not positions.is_contiguous():
        raise KernelLibraryError("positions must be int64 (or int32 lengths), contiguous, one per row")
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=cand_ids.device)
    elif out.dtype != torch.int32 or out.numel() != n or not out.is_contiguous():
        raise KernelLibraryError("the tokens' buffer must be contiguous int32, one per row")
    lib = library.core()
    entry = lib.sb_draw if positions.dtype == torch.int64 else lib.sb_draw_after
    check(entry(_p(out), _p(cand_ids.contiguous()), _p(cand_z.contiguous()), _p(positions),
                n, k, int(top_k), 0 if log_min_p is None else 1,
                0.0 if log_min_p is None else float(log_min_p), 0 if top_p is None else 1,
                0.0 if top_p is None else float(top_p), int(seed) & 0xFFFFFFFFFFFFFFFF, _stream()))
    return out


def read_bandwidth(n_bytes: int = 1 << 30, blocks: int = 512, repeats: int = 5, device="cuda:0") -> float:
    """Bytes a second that a plain streaming read of ``n_bytes`` reaches on this GPU (the best of
    ``repeats`` passes over a buffer that the caches do not hold): what "achievable" means beside
    the published peak in a bandwidth report."""
    n_bytes = max(16, n_bytes // 16 * 16)
    src = torch.zeros((n_bytes // 4,), dtype=torch.int32, device=device)
    sink = torch.zeros((4,), dtype=torch.int32, device=device)
    lib = library.core()
    best = 0.0
    for _ in range(repeats + 1):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        check(lib.sb_read_probe(_p(sink), _p(src), n_bytes, int(blocks), _stream()))
        e1.record()
        e1.synchronize()
        best = max(best, n_bytes / (e0.elapsed_time(e1) * 1e-3))
    return best


_RANDOM_KINDS = {torch.float32: 0, torch.bfloat16: 1, torch.float64: 2}


def random_normal(shape, seed: int, tensor_index: int, mean: float = 0.0, std: float = 1.0,
                  dtype: torch.dtype = torch.float32, device="cuda:0", first: int = 0) -> torch.Tensor:
    """Seeded normal values of ``shape`` drawn on the device: float32(mean + std z) as float32 or
    rounded to bfloat16, or (``dtype`` float64) the standard normals z themselves.  Element e of
    the tensor (counted from ``first``, a multiple of four) is a function of (seed, tensor_index,
    e) alone, the one the host computes in :mod:`sonicboom_amd.weights.random_stream`."""
    try:
        kind = _RANDOM_KINDS[dtype]
    except KeyError:
        raise KernelLibraryError(f"random values come as float32, bfloat16 or float64, not {dtype}") from None
    out = torch.empty(tuple(shape), dtype=dtype, device=device)
    if not out.is_cuda:
        raise KernelLibraryError("random values are drawn on the GPU (the host has its own function for them)")
    lib = library.core()
    with torch.cuda.device(out.device):
        check(lib.sb_random_normal(_p(out), kind, out.numel(), int(first), int(seed) & (2 ** 64 - 1),
                                   int(tensor_index), float(mean), float(std), _stream()))
    return out


# --------------------------------------------------------------------------
# dispatch between the plain kernels and the MFMA kernels
# --------------------------------------------------------------------------
SKINNY_MAX_ROWS = 64


def gemm_bf16_partial(x: torch.Tensor, w: torch.Tensor, packed_shape=None) -> Optional[torch.Tensor]:
    """The raw product x w^T of bfloat16 rows in K slices, float32 [slices, rows, out], for a
    consumer that adds the slices itself (:func:`reduce_resid_norm`, :func:`rope_kv_store`).
    Packed weights, up to 64 rows: the kernel whose waves split the output features and share
    the rows through LDS, with K cut over the grid so that the blocks fill the GPU.
    Packed weights, more rows: the tiled kernel with K cut over the grid, as long as the cut gives
    more than one slice (a narrow matrix and up to a few hundred rows, where one slice would leave
    most of the GPU without a tile; or a thousand or two, where tiles of 256 x 256 with K cut in
    two to four beat the whole product in smaller tiles).  Row-major weights, up to 64 rows: the kernel whose waves split K.  None when
    none applies: the caller then takes the whole product."""
    _dev(x, w)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16 or x.dim() != 2:
        return None
    n, k = packed_shape if packed_shape is not None else (w.shape[0], w.shape[-1])
    t = x.shape[0]
    if x.shape[1] != k:
        raise KernelLibraryError(f"gemm shapes do not match: x {tuple(x.shape)}, w {(n, k)}")
    if t == 0 or k % 8 or x.data_ptr() % 16 or w.data_ptr() % 16:
        return None
    lib = library.core()
    which = _hints.few_rows_kernel
    if packed_shape is not None and t <= SKINNY_MAX_ROWS and which in (None, "stream"):
        slices = lib.sb_gemm_stream_slices(t, n, k, _hints.stream)
        partial = torch.empty((slices, t, n), dtype=torch.float32, device=x.device)
        check(lib.sb_gemm_stream_partial_bf16(_p(partial), _p(x), _p(w), t, n, k, _hints.stream, _stream()))
        return partial
    if packed_shape is not None and (t > SKINNY_MAX_ROWS or which == "tiled"):
        slices = lib.sb_gemm_mfma_slices(t, n, k, 1)
        if slices > 1 or t <= SKINNY_MAX_ROWS:
            partial = torch.empty((slices, t, n), dtype=torch.float32, device=x.device)
            check(lib.sb_gemm_mfma_partial_bf16(_p(partial), _p(x), _p(w), t, n, k, 1, _stream()))
            return partial
        return None
    if t > SKINNY_MAX_ROWS:
        return None
    slices = lib.sb_gemm_skinny_slices(t, n, k)
    partial = torch.empty((slices, t, n), dtype=torch.float32, device=x.device)
    check(lib.sb_gemm_skinny_partial_bf16(_p(partial), _p(x), _p(w), t, n, k, 1 if packed_shape is not None else 0,
                                          _stream()))
    return partial


def reduce_resid_norm(partial: torch.Tensor, bias: Optional[torch.Tensor], x: torch.Tensor,
                      norm_weight: Optional[torch.Tensor], eps: float, out_dtype: Optional[torch.dtype]
                      ) -> Optional[torch.Tensor]:
    """x += sum of the slices of ``partial`` [slices, rows, width] (+ bias); when ``out_dtype`` is
    given also returns rmsnorm(x) * norm_weight in that type.  One pass over the row."""
    _dev(partial, bias, x, norm_weight)
    if partial.dim() != 3 or partial.dtype != torch.float32 or x.dtype != torch.float32 \
            or tuple(x.shape) != tuple(partial.shape[1:]):
        raise KernelLibraryError("reduce_resid_norm needs float32 slices [s, rows, width] and a residual [rows, width]")
    s_, t, width = partial.shape
    if bias is not None and bias.numel() != width:
        raise KernelLibraryError("bias does not match the row width")
    if norm_weight is not None and norm_weight.numel() != width:
        raise KernelLibraryError("norm weight does not match the row width")
    lib = library.core()
    if width % 4 or width > lib.sb_reduce_resid_norm_max_width():
        raise KernelLibraryError(f"reduce_resid_norm takes widths in steps of 4 up to "
                                 f"{lib.sb_reduce_resid_norm_max_width()}, not {width}")
    y = torch.empty((t, width), dtype=out_dtype, device=x.device) if out_dtype is not None else None
    check(lib.sb_reduce_resid_norm(_p(y), _dt(y) if y is not None else 0, _p(x), _p(partial), s_, _p(bias),
                                   _dt(bias) if bias is not None else 0, _p(norm_weight),
                                   _dt(norm_weight) if norm_weight is not None else 0, t, width, float(eps),
                                   1 if out_dtype is not None else 0, _stream()))
    return y


def reduce_resid_norm_ok(width: int) -> bool:
    return width % 4 == 0 and width <= library.core().sb_reduce_resid_norm_max_width()


def pack_weight(w: torch.Tensor, gated: bool = False) -> torch.Tensor:
    """A bf16 projection weight [out, in] in the matrix-core tile layout: rows padded to 16, k to
    32, and every 16 x 32 tile stored as one 1 KB block in fragment order — lane l = 16 g + r of a
    wave owns elements [row r][k = 8 g .. 8 g + 7] at offset 8 l — tiles of one row block being
    consecutive in k.  A wave then reads a whole fragment with one contiguous 1 KB load and walks
    K through consecutive memory.  With ``gated`` the two halves [gate; up] are packed one after
    the other.  Returns a flat bf16 tensor."""
    if w.dim() != 2 or w.dtype != torch.bfloat16:
        raise KernelLibraryError("pack_weight takes a bfloat16 matrix [out, in]")
    halves = w.chunk(2, dim=0) if gated else (w,)
    out = []
    for h in halves:
        n, k = h.shape
        n16, k32 = (n + 15) // 16 * 16, (k + 31) // 32 * 32
        if (n16, k32) != (n, k):
            h = torch.nn.functional.pad(h, (0, k32 - k, 0, n16 - n))
        out.append(h.reshape(n16 // 16, 16, k32 // 32, 4, 8).permute(0, 2, 3, 1, 4).reshape(-1))
    return torch.cat(out).contiguous() if len(out) > 1 else out[0].contiguous()


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], resid: Optional[torch.Tensor],
              out_dtype: torch.dtype, out: Optional[torch.Tensor] = None, gated: bool = False,
              packed_shape=None) -> Optional[torch.Tensor]:
    """bfloat16 product on the matrix cores: y = x w^T (+bias) (+resid), or with ``gated``
    (True or "silu", or "gelu_tanh") y = act(x wg^T) * (x wu^T) for w = [wg; wu].  Up to 64 rows go to one of the two
    weight-streaming kernels, more to the tiled one.  ``packed_shape`` = (rows of w, inner size) says that ``w`` is
    in the layout of :func:`pack_weight`.  Returns None when the sizes fit neither kernel (an
    inner size that is not a multiple of 8): the caller then takes the plain kernel."""
    _dev(x, w, bias, resid, out)
    if x.dtype != torch.bfloat16 or w.dtype != torch.bfloat16:
        return None
    w_rows, w_k = packed_shape if packed_shape is not None else (w.shape[0], w.shape[-1])
    if x.dim() != 2 or x.shape[1] != w_k or (packed_shape is None and w.dim() != 2):
        raise KernelLibraryError(f"gemm shapes do not match: x {tuple(x.shape)}, w {(w_rows, w_k)}")
    t, k = x.shape
    gate = gate_code(gated)
    n = w_rows // 2 if gated else w_rows
    if k % 8 or x.data_ptr() % 16 or w.data_ptr() % 16 or (gated and w_rows % 2):
        return None
    if bias is not None and bias.numel() != n:
        raise KernelLibraryError(f"bias has {bias.numel()} elements, the product has {n} columns")
    if resid is not None and (resid.dtype != torch.float32 or tuple(resid.shape) != (t, n)):
        raise KernelLibraryError("the residual must be float32 and shaped like the product")
    if out is None:
        out = torch.empty((t, n), dtype=out_dtype, device=x.device)
    elif out.dtype != out_dtype or tuple(out.shape) != (t, n):
        raise KernelLibraryError("gemm output buffer has the wrong shape or type")
    lib = library.core()
    bdt = _dt(bias) if bias is not None else 0
    packed = 1 if packed_shape is not None else 0
    # A wide packed matrix (enough 16-row tiles, or gate/up pairs of them, for STREAM_MIN_BLOCKS
    # blocks of four waves) and up to 128 rows: the kernel whose waves split the output features
    # and share the rows through LDS.  Other products of up to 64 rows: the kernel whose waves
    # split K and which can cut K over the grid as well.  The rest: the tiled kernel.
    which = _hints.few_rows_kernel
    if which is None:
        wave_units = -(-n // 16) if gated else -(-n // 32)
        which = "stream" if packed and wave_units >= 4 * STREAM_MIN_BLOCKS else "skinny"
        if t > SKINNY_MAX_ROWS and which == "stream":
            # 65 to 128 rows: the tiled kernel's 128 x 128 tiles do as well or better unless the
            # matrix is wide and their count leaves the last round over the 256 CUs nearly empty
            # (8,960 x 1,536 and 11,008 x 2,048 at 96 rows: 21 and 26 us tiled, 25 and 34 streamed)
            rounds = -(-n // (64 if gated else 128)) / 256.0
            if wave_units < 4 * STREAM_MIN_BLOCKS_MORE_ROWS or math.ceil(rounds) / rounds < 1.4:
                which = "tiled"
    if t <= STREAM_MAX_ROWS and which == "stream" and packed:
        check(lib.sb_gemm_stream_bf16(_p(out), _dt(out), _p(x), _p(w), _p(bias), bdt, _p(resid), t, n, k,
                                      gate, _hints.stream, _stream()))
    elif t <= SKINNY_MAX_ROWS and which != "tiled":
        need = lib.sb_gemm_skinny_scratch(t, n, k, gate)
        scratch = torch.empty((need,), dtype=torch.float32, device=x.device) if need else None
        check(lib.sb_gemm_skinny_bf16(_p(out), _dt(out), _p(x), _p(w), _p(bias), bdt, _p(resid), t, n, k,
                                      gate, packed, _p(scratch), need, _stream()))
    else:
        check(lib.sb_gemm_mfma_bf16(_p(out), _dt(out), _p(x), _p(w), _p(bias), bdt, _p(resid), t, n, k,
                                    gate, packed, _hints.tile_shape, _stream()))
    return out


@contextlib.contextmanager
def gemm_tile_shape(shape: Optional[int], path: Optional[str] = None):
    """For tests and measurements: inside the block the tiled products of this thread use tile
    shape ``shape`` (0: 128 x 128, 1: 256 x 128, 2: 256 x 256, 3: 128 x 256, 4: 192 x 256 outputs per
    block) instead of choosing one, and with ``path`` the kernel that stages tiles through
    "registers" or the one that loads them "direct" into LDS (packed weights, inner size in 64s;
    the only one with shapes 3 and 4)."""
    paths = {None: 0, "registers": 1, "direct": 2, "direct, a block a tile": 3}
    if path not in paths:
        raise ValueError(f"unknown path {path!r}")
    if shape is not None:
        shape = int(shape) + 16 * paths[path]
    before = _hints.tile_shape
    _hints.tile_shape = -1 if shape is None else int(shape)
    try:
        yield
    finally:
        _hints.tile_shape = before


@contextlib.contextmanager
def gemm_few_rows_kernel(which: Optional[str], waves: int = 0, slices: int = 0):
    """For tests and measurements: inside the block this thread's products of up to 64 rows,
    whole or in K slices, go to the kernel ``which`` ("stream", "skinny" or "tiled"; "stream"
    needs packed weights) whatever the sizes, and the stream kernel uses ``waves`` waves per block
    (4 to 8) and aims at ``slices`` K slices (1 to 8); 0: its own choice."""
    if which not in (None, "stream", "skinny", "tiled"):
        raise ValueError(f"unknown kernel {which!r}")
    before = (_hints.few_rows_kernel, _hints.stream)
    _hints.few_rows_kernel = which
    _hints.stream = (int(waves) & 0xff) | ((int(slices) & 0xff) << 8)
    try:
        yield
    finally:
        _hints.few_rows_kernel, _hints.stream = before


MFMA_MAX_HEAD_DIM = 256
# Blocks of four waves that a matrix must give the stream kernel.  A block streams its share of W at
# what one CU pulls, whatever the count of blocks, so fewer blocks than CUs only pay while the
# other kernel, which spreads K over the whole GPU, has more bytes to move than a block's share
# takes: gate/up pairs of 8,960 x 1,536 (140 blocks) 13 to 18 us against 18 to 29 at up to 64 rows,
# 11,008 x 2,048 (172 blocks) 19 to 25 against 25 to 34; 8,192 x 2,048 (128 blocks) 18 against 16,
# and 4,864 x 896 (76 blocks) 4 % slower in a whole decode step.
STREAM_MIN_BLOCKS = 136
STREAM_MIN_BLOCKS_MORE_ROWS = 192        # for 65 to 128 rows
STREAM_MAX_ROWS = 128


def attention_mfma_ok(q_dtype, cache_dtype, head_dim: int) -> bool:
    """Whether the matrix-core attention kernels take these types and this head size."""
    return (q_dtype == torch.bfloat16 and cache_dtype == torch.bfloat16 and head_dim % 16 == 0
            and 16 <= head_dim <= MFMA_MAX_HEAD_DIM)


def attention_decode_mfma(q, k_cache, v_cache, page_table, seq_pos, heads_q, heads_kv, head_dim, scale, window):
    """One bf16 query row per sequence (row i belongs to row i of ``page_table``) at position
    ``seq_pos[i]``, over the cache; keys are split over blocks and merged in ascending order."""
    _dev(q, k_cache, v_cache, page_table, seq_pos)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim or q.dtype != torch.bfloat16:
        raise KernelLibraryError(f"queries must be bfloat16 [sequences, {heads_q * head_dim}]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    _i32(seq_pos, n, "sequence positions")
    if page_table.dtype != torch.int32 or page_table.dim() != 2 or page_table.shape[0] < n:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    lib = library.attention_library(head_dim)
    max_pages = page_table.shape[1]
    chunks = lib.sb_attn_decode_chunks(max_pages)
    out = torch.empty_like(q)
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((lib.sb_attn_decode_part_o(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                             device=q.device)
        part_ml = torch.empty((lib.sb_attn_decode_part_ml(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                              device=q.device)
    check(lib.sb_attn_decode_bf16(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(page_table), max_pages,
                                  k_cache.shape[0], _p(seq_pos), _p(part_o), _p(part_ml), n, heads_q,
                                  heads_kv, float(scale), int(window), _hints.decode_pages, _stream()),
          lib, "sb_attn_last_error")
    return out


def attention_decode_rope_ok(qkv: torch.Tensor, q_dtype, cache_dtype, heads_q: int, heads_kv: int, head_dim: int,
                             rot_dims: int) -> bool:
    """Whether :func:`attention_decode_rope` takes these operands (else: :func:`rope_kv_store`, then
    :func:`attention`)."""
    if not attention_mfma_ok(q_dtype, cache_dtype, head_dim) or qkv.dtype != torch.float32:
        return False
    lib = library.attention_library(head_dim)
    return bool(lib.sb_attn_decode_rope_ok(heads_q, heads_kv, int(rot_dims), qkv.shape[-1]))


def attention_decode_rope(qkv: torch.Tensor, inv_freq: Optional[torch.Tensor], freq_factors: Optional[torch.Tensor],
                          rot_dims: int, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor,
                          seq_pos: torch.Tensor, heads_q: int, heads_kv: int, head_dim: int, scale: float, window: int,
                          bias: Optional[torch.Tensor] = None, store: bool = True) -> torch.Tensor:
    """A decode step's rotation, store and attention in one kernel: ``qkv`` float32 [n, width] or
    [slices, n, width] (partial sums of the projection, added in ascending order, then ``bias``),
    one row per sequence at position ``seq_pos[i]``.  Queries and keys are rotated as
    :func:`rope_kv_store` rotates them, the row's key and value go into the cache (``store``), and the
    row attends over its sequence's keys, its own among them.  Returns the attention output in
    bfloat16 [n, heads_q * head_dim]: the bits of the two kernels one after the other."""
    _dev(qkv, inv_freq, freq_factors, k_cache, v_cache, page_table, seq_pos, bias)
    n_slices = 1
    if qkv.dim() == 3:
        n_slices = qkv.shape[0]
        qkv = qkv.view(-1, qkv.shape[2])
    n = qkv.shape[0] // n_slices
    need = (heads_q + (2 * heads_kv if store else 0)) * head_dim
    if qkv.dtype != torch.float32 or qkv.shape[1] < need:
        raise KernelLibraryError(f"qkv rows must be float32 with at least {need} elements")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() < need):
        raise KernelLibraryError("the qkv bias must be float32 and cover a whole row")
    if inv_freq is not None:
        if inv_freq.dtype != torch.float32 or inv_freq.numel() != rot_dims // 2:
            raise KernelLibraryError("inv_freq must be float32 [rot_dims/2]")
        if freq_factors is not None and (freq_factors.dtype != torch.float32 or freq_factors.numel() < rot_dims // 2):
            raise KernelLibraryError("freq_factors must be float32 [rot_dims/2]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    if k_cache.dtype != torch.bfloat16:
        raise KernelLibraryError("the fused decode kernel takes a bfloat16 cache")
    _i32(seq_pos, n, "sequence positions")
    if page_table.dtype != torch.int32 or page_table.dim() != 2 or page_table.shape[0] < n:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    lib = library.attention_library(head_dim)
    max_pages = page_table.shape[1]
    chunks = lib.sb_attn_decode_chunks(max_pages)
    out = torch.empty((n, heads_q * head_dim), dtype=torch.bfloat16, device=qkv.device)
    part_o = part_ml = None
    if chunks > 1:
        part_o = torch.empty((lib.sb_attn_decode_part_o(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                             device=qkv.device)
        part_ml = torch.empty((lib.sb_attn_decode_part_ml(n, heads_q, heads_kv, max_pages),), dtype=torch.float32,
                              device=qkv.device)
    check(lib.sb_attn_decode_rope_bf16(_p(out), _p(qkv), qkv.shape[1], n_slices, _p(bias), _p(inv_freq),
                                       _p(freq_factors), int(rot_dims) if inv_freq is not None else 0,
                                       1 if store else 0, _p(k_cache), _p(v_cache), _p(page_table), max_pages,
                                       k_cache.shape[0], _p(seq_pos), _p(part_o), _p(part_ml), n, heads_q, heads_kv,
                                       float(scale), int(window), _hints.decode_pages, _stream()),
          lib, "sb_attn_last_error")
    return out


@contextlib.contextmanager
def attention_decode_pages_per_wave(head_dim: int, pages: int):
    """For tests and measurements: inside the block this thread's decode attention gives every
    wave ``pages`` pages (1, 2, 4 or 8; more than one only up to head size 128) instead of
    choosing from the sizes; 0: the launcher's choice."""
    before = _hints.decode_pages
    _hints.decode_pages = int(pages)
    try:
        yield
    finally:
        _hints.decode_pages = before


def attention_prefill_mfma(q, k_cache, v_cache, page_table, row_pos, tiles, heads_q, heads_kv, head_dim, scale,
                           window, tile_rows=16):
    """bf16 query rows over the cache; ``tiles`` int32 [n, 4] = (first row, rows <= tile_rows, sequence, 0)
    cuts the rows into runs of consecutive positions of one sequence.  ``tile_rows``: 16, or what
    :func:`attention_row_tile` gives for these heads."""
    _dev(q, k_cache, v_cache, page_table, row_pos, tiles)
    n = q.shape[0]
    if q.dim() != 2 or q.shape[1] != heads_q * head_dim or q.dtype != torch.bfloat16:
        raise KernelLibraryError(f"queries must be bfloat16 [rows, {heads_q * head_dim}]")
    _check_cache(k_cache, v_cache, heads_kv, head_dim)
    _i32(row_pos, n, "row positions")
    if tiles.dtype != torch.int32 or tiles.dim() != 2 or tiles.shape[1] != 4:
        raise KernelLibraryError("tiles must be int32 [n, 4]")
    if page_table.dtype != torch.int32 or page_table.dim() != 2:
        raise KernelLibraryError("page table must be int32 [sequences, pages]")
    lib = library.attention_library(head_dim)
    out = torch.empty_like(q)
    check(lib.sb_attn_prefill_bf16(_p(out), _p(q), _p(k_cache), _p(v_cache), _p(page_table), page_table.shape[1],
                                   k_cache.shape[0], _p(row_pos), _p(tiles), tiles.shape[0], heads_q, heads_kv,
                                   float(scale), int(window), int(tile_rows), _stream()), lib, "sb_attn_last_error")
    return out


# rows of one sequence that a block of the prefill attention kernels takes together; a mixer that
# calls attention() carries it as its row_tile attribute, so that a step describes its rows in
# runs of this height
ATTENTION_ROW_TILE = 16


def attention_row_tile(heads_q: int, heads_kv: int, head_dim: int, dtype=torch.bfloat16) -> int:
    """The height of row tiles that suits attention with these heads: 16, or 64 and 32 where the
    matrix-core kernel runs groups of one and two query heads per kv head (its blocks' waves
    that would have no head take further rows of the tile)."""
    if dtype != torch.bfloat16 or not attention_mfma_ok(dtype, dtype, head_dim) or not torch.cuda.is_available():
        return ATTENTION_ROW_TILE
    return int(library.attention_library(head_dim).sb_attn_prefill_tile_rows(int(heads_q), int(heads_kv)))


# the prefill kernel's second form, for long prompts: tiles of 32 rows (head sizes that 32 divides,
# up to 128, groups of three and more heads); taken when its blocks fill the GPU
TALL_ROW_TILE = 32
TALL_MIN_BLOCKS = 320


def attention_tall_ok(heads_q: int, heads_kv: int, head_dim: int, dtype=torch.bfloat16) -> bool:
    """Whether prefill attention with these heads also runs in tiles of 32 rows."""
    if dtype != torch.bfloat16 or not attention_mfma_ok(dtype, dtype, head_dim) or not torch.cuda.is_available():
        return False
    fn = getattr(library.attention_library(head_dim), "sb_attn_prefill_tall_ok", None)
    return bool(fn is not None and fn(int(heads_q), int(heads_kv)))


def attention_row_tiles(heads_q: int, heads_kv: int, head_dim: int, dtype=torch.bfloat16):
    """The heights of row tiles that a mixer calling :func:`attention` with these heads asks a
    step's context for (its ``row_tile`` attribute): the usual one first."""
    base = attention_row_tile(heads_q, heads_kv, head_dim, dtype)
    if base != TALL_ROW_TILE and attention_tall_ok(heads_q, heads_kv, head_dim, dtype):
        return (base, TALL_ROW_TILE)
    return (base,)


def attention(q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, page_table: torch.Tensor, ctx,
              heads_q: int, heads_kv: int, head_dim: int, scale: float, window: int,
              fast: bool = True, row_tile=ATTENTION_ROW_TILE) -> torch.Tensor:
    """Attention of a step's rows over the cache; ``ctx`` is the step's context.  bfloat16 with a
    head size in steps of 16 runs on the matrix cores (a decode kernel when every sequence brings
    one row, else the prefill kernel); everything else takes the plain kernel.  ``row_tile``: the
    height of the context's row tiles to use, or several (what :func:`attention_row_tiles` gives):
    tiles of 32 rows are then taken when their blocks fill the GPU."""
    if fast and attention_mfma_ok(q.dtype, k_cache.dtype, head_dim):
        if ctx.is_decode:
            return attention_decode_mfma(q, k_cache, v_cache, page_table, ctx.row_pos, heads_q, heads_kv,
                                         head_dim, scale, window)
        heights = (row_tile,) if isinstance(row_tile, int) else tuple(row_tile)
        height = heights[0]
        if TALL_ROW_TILE in heights[1:]:
            blocks = ctx.row_tiles(TALL_ROW_TILE).shape[0] * heads_kv * ((heads_q // heads_kv + 7) // 8)
            if blocks >= TALL_MIN_BLOCKS:
                height = TALL_ROW_TILE
        return attention_prefill_mfma(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_tiles(height),
                                      heads_q, heads_kv, head_dim, scale, window, tile_rows=height)
    return attention_plain(q, k_cache, v_cache, page_table, ctx.row_pos, ctx.row_seq, heads_q, heads_kv,
                           head_dim, scale, window)

"""Grouped-query self-attention over the paged cache.

Order of work, from /root/reference/core/src/model/emit.cpp:255-308: project
q, k and v, add their biases, rotate q and k (the bias precedes the rotation,
v is not rotated), store k and v, attend, project the result.  The scale is
1/sqrt(head_dim) unless the spec gives another, times the position encoding's
multiplier (/root/reference/core/src/model/recipe.cpp:65-70, :165-167).
Every size and switch is a parameter of the spec:

    heads_q, heads_kv, head_dim, window (0 = all keys), scale (None = 1/sqrt),
    qkv_bias, out_bias

and the position encoding is a nested part.  The three input projections are
packed into one matrix when the mixer is built, so a step runs one product
for q, k and v.  An order entry that only reads another entry's cache runs
the query rows of that matrix alone.
"""
from __future__ import annotations

from typing import Optional

import numpy as np
import torch

from .. import ops
from .base import KVSpec, Mixer, register_part
from .linear import Linear
from .spec import PartSpec, TensorSpec


def attention_spec(prefix: str, width: int, heads_q: int, heads_kv: int, head_dim: int,
                   position: PartSpec, window: int = 0, scale: Optional[float] = None,
                   qkv_bias: bool = True, out_bias: bool = False) -> PartSpec:
    qw, kvw = heads_q * head_dim, heads_kv * head_dim
    tensors = {
        "q_weight": TensorSpec(prefix + "q_proj.weight", (qw, width)),
        "k_weight": TensorSpec(prefix + "k_proj.weight", (kvw, width)),
        "v_weight": TensorSpec(prefix + "v_proj.weight", (kvw, width)),
        "o_weight": TensorSpec(prefix + "o_proj.weight", (width, qw)),
    }
    if qkv_bias:
        tensors["q_bias"] = TensorSpec(prefix + "q_proj.bias", (qw,))
        tensors["k_bias"] = TensorSpec(prefix + "k_proj.bias", (kvw,))
        tensors["v_bias"] = TensorSpec(prefix + "v_proj.bias", (kvw,))
    if out_bias:
        tensors["o_bias"] = TensorSpec(prefix + "o_proj.bias", (width,))
    return PartSpec("mixer", "attention", {
        "width": width, "heads_q": heads_q, "heads_kv": heads_kv, "head_dim": head_dim,
        "window": int(window), "scale": scale, "qkv_bias": qkv_bias, "out_bias": out_bias,
    }, tensors, {"position": position})


@register_part("mixer", "attention")
class Attention(Mixer):
    # a step's context lists its rows in runs of this many for the mixer's prefill kernel
    row_tile = ops.ATTENTION_ROW_TILE

    def __init__(self, spec, tensors, parts, rt):
        super().__init__(spec, tensors, parts, rt)
        p = spec.params
        self.width = int(p["width"])
        self.heads_q, self.heads_kv, self.head_dim = int(p["heads_q"]), int(p["heads_kv"]), int(p["head_dim"])
        if self.heads_q % self.heads_kv:
            raise ValueError(f"{self.heads_q} query heads are not a multiple of {self.heads_kv} kv heads")
        self.window = int(p.get("window") or 0)
        self.position = parts["position"]
        base_scale = p.get("scale")
        if base_scale is None:
            base_scale = float(np.float32(1.0) / np.sqrt(np.float32(self.head_dim)))
        self.scale = float(np.float32(base_scale) * np.float32(self.position.score_scale))
        self.q_width = self.heads_q * self.head_dim
        self.kv_width = self.heads_kv * self.head_dim
        if rt.fast_kernels:
            # (groups of one and two heads per kv head take higher tiles on the matrix cores)
            self.row_tile = ops.attention_row_tiles(self.heads_q, self.heads_kv, self.head_dim, rt.act_dtype)

        ws = [tensors["q_weight"], tensors["k_weight"], tensors["v_weight"]]
        w_qkv = torch.cat(ws, dim=0) if all(w.dtype == ws[0].dtype for w in ws) \
            else torch.cat([w.float() for w in ws], dim=0)
        b_qkv = None
        if p.get("qkv_bias", True):
            bs = [tensors["q_bias"], tensors["k_bias"], tensors["v_bias"]]
            b_qkv = torch.cat([b.float() for b in bs], dim=0)
        self.qkv = Linear(w_qkv, b_qkv, rt.fast_kernels)
        # an order entry that reads another entry's cache projects queries only: the model asks for
        # that projection (query_only) before finish_build() drops the separate query weight
        self._q_parts = (tensors["q_weight"], None if b_qkv is None else b_qkv[: self.q_width])
        self._q_only = None
        self.out = Linear(tensors["o_weight"], tensors.get("o_bias"), rt.fast_kernels)

    def query_only(self) -> None:
        """Build the queries-only projection (for run-order entries that read another entry's cache)."""
        if self._q_only is None:
            if self._q_parts is None:
                raise RuntimeError("the queries-only projection must be asked for while the model is built")
            self._q_only = Linear(self._q_parts[0], self._q_parts[1], self.rt.fast_kernels)

    def finish_build(self) -> None:
        self._q_parts = None

    def cache_spec(self) -> KVSpec:
        return KVSpec(self.heads_kv, self.head_dim, self.window)

    fuses_norm = True
    graph_safe = True     # its launches depend on device buffers only
    fold_rotation = True  # decode steps: rotate and store inside the attention kernel where it takes the sizes

    def forward(self, h, x, ctx, binding, then_norm=None):
        """x += attention(h).  Returns then_norm(x) when the output projection could apply the
        norm in its last pass, else None."""
        rt = self.rt
        writes = binding.writes_cache
        if not writes:
            self.query_only()
        proj = self.qkv if writes else self._q_only
        # q, k, v stay float32 until they have been rotated: one rounding on the way to the cache.
        tables = self.position.rotary_tables()
        bias = None
        qkv = proj.partial(h) if tables is not None else None
        if qkv is not None:
            bias = proj.bias          # the rotate-and-store kernel adds the K slices and the bias
        else:
            qkv = proj(h, torch.float32)
        if tables is None:
            self.position.apply(qkv, ctx, self.heads_q, self.heads_kv if writes else 0, self.head_dim)
            tables = (None, None, 0)
        inv_freq, freq_factors, rot_dims = tables
        page_table = ctx.page_table(binding.group)
        if ctx.is_decode and rt.fast_kernels and self.fold_rotation and ops.attention_decode_rope_ok(
                qkv, rt.act_dtype, binding.k_cache.dtype, self.heads_q, self.heads_kv, self.head_dim,
                rot_dims if inv_freq is not None else 0):
            # one token per sequence: rotation, store and attention in one kernel
            a = ops.attention_decode_rope(qkv, inv_freq, freq_factors, rot_dims, binding.k_cache, binding.v_cache,
                                          page_table, ctx.row_pos, self.heads_q, self.heads_kv, self.head_dim,
                                          self.scale, self.window, bias=bias, store=writes)
            return self.out.add_into(a, x, then_norm, rt.act_dtype)
        q = ops.rope_kv_store(
            qkv, rt.act_dtype, inv_freq, freq_factors, rot_dims, ctx.row_pos, ctx.row_seq,
            binding.k_cache if writes else None, binding.v_cache if writes else None,
            page_table if writes else None, self.heads_q, self.heads_kv if writes else 0, self.head_dim,
            bias=bias)
        a = ops.attention(q, binding.k_cache, binding.v_cache, page_table, ctx, self.heads_q, self.heads_kv,
                          self.head_dim, self.scale, self.window, fast=rt.fast_kernels, row_tile=self.row_tile)
        return self.out.add_into(a, x, then_norm, rt.act_dtype)

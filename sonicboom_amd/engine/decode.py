"""Repeated single-token steps of a set of sequences, with the step replayed as a HIP graph.

A decode step of B sequences launches a few hundred small kernels; launched one
by one from Python they cost more than the step's memory traffic.  The loop
therefore keeps the step's bookkeeping (token ids, positions, page tables) in
fixed device buffers, runs the step once or twice kernel by kernel, then
captures exactly the same launches into a HIP graph per (batch size, page
table width) and replays it, refreshing the buffers with one small copy per
step.  Graph and kernel-by-kernel steps run the same kernels on the same
shapes, so they give the same bits; the graph is only a way of launching.
Nothing in the graph clears memory with a memset node.

The reference captures its decode step the same way
(/root/reference/core/src/model/gemma4_plan.cpp:1650-1687, :1704-1797: set the
position, replay the captured step, read the token).
"""
from __future__ import annotations

import gc
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import ops
from ..cache.paged import CacheError, pages_for
from .step import ContextLayout, StepError, _Context, row_runs

WIDTH_STEP = 16      # page-table widths are rounded up to this many pages (1024 tokens)
CAPTURE_AFTER = 2    # kernel-by-kernel steps of a shape before its graph is captured
MAX_GRAPHS = 24      # recorded shapes kept; the one unused for longest goes first
EXACT_BATCHES = 8    # batches up to this size run as they are; larger ones are padded to a bucket


def batch_bucket(n: int) -> int:
    """The batch size a step of ``n`` sequences runs at: ``n`` itself up to 8, then the next of
    12, 16, 24, 32, 48, 64, ... (twice and three times the powers of two).  A batch whose
    sequences end one by one then passes through a handful of recorded shapes instead of one per
    size; the rows added are sequences without pages, which store nothing and see no key."""
    if n <= EXACT_BATCHES:
        return n
    p = 8
    while True:
        for b in (p + p // 2, 2 * p):
            if n <= b:
                return b
        p *= 2


class _StaticContext(_Context):
    """A decode step's bookkeeping in device buffers whose addresses never change: the tables of
    :class:`~sonicboom_amd.engine.step.ContextLayout` for ``batch`` sequences of one row each and
    page tables ``width`` wide, refilled every step."""

    def __init__(self, engine, batch: int, width: int):
        cache = engine.cache
        self.batch, self.width = batch, width
        self.n_rows = self.n_seqs = self.n_wanted = batch
        self.is_decode = True
        self.max_new = 1
        heights = engine.model.row_tiles
        self.layout = layout = ContextLayout(batch, batch, batch, {h: batch for h in heights},
                                             [(batch, width)] * len(cache.groups))
        dev = engine.device
        # two pinned staging buffers used in turn: a step never overwrites the one whose copy
        # may still be in flight
        self._hosts = [torch.zeros(layout.total, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._turn = 0
        self.dev = torch.zeros(layout.total, dtype=torch.int32, device=dev)
        self.next_ids = torch.zeros(batch, dtype=torch.int32, device=dev)
        layout.bind(self, self.dev)
        # the parts that never change for a decode step of this batch size: a row a sequence,
        # every row wanted, and whatever the height a run is that one row
        ar = np.arange(batch, dtype=np.int32)
        # the tables a step rewrites, as views of each staging buffer (made once)
        self._views = [{key: layout.view(h.numpy(), key) for key in ("ids", "row_pos", "len_before", "slots")
                        + tuple(("table", g) for g in range(layout.n_groups))} for h in self._hosts]
        for h in self._hosts:
            n = h.numpy()
            layout.view(n, "row_seq")[:] = ar
            layout.view(n, "cu_rows")[:] = np.arange(batch + 1, dtype=np.int32)
            layout.view(n, "want_rows")[:] = ar
            for height in layout.heights:
                layout.view(n, ("tiles", height))[:] = row_runs([1] * batch, np.arange(batch + 1), height)

    def refresh(self, cache, slots: Sequence[int], tokens: Sequence[int]) -> None:
        """This step's ids, positions and page tables, in one copy to the device.  Fewer
        sequences than the buffers' batch: the rest are rows of token 0 at position 0 with no
        page at all (they store nothing and attend to nothing; their logits are not read)."""
        host, views = self._hosts[self._turn], self._views[self._turn]
        self._turn ^= 1
        live = len(slots)
        lengths = np.zeros(self.batch, dtype=np.int32)
        lengths[:live] = [cache.length(s) for s in slots]
        ids = views["ids"]
        ids[:live] = np.asarray(tokens, dtype=np.int32)
        ids[live:] = 0
        views["row_pos"][:] = lengths
        views["len_before"][:] = lengths
        slot_row = views["slots"]
        slot_row[:live] = np.asarray(slots, dtype=np.int32)
        slot_row[live:] = slots[0]
        for g in range(self.layout.n_groups):
            table = views[("table", g)]
            table[:live] = cache.page_table(g, slots, min_width=self.width)
            table[live:] = -1
        self.max_len_after = int(lengths.max()) + 1
        # the host's view of the step, as StepContext has it
        self.slot_list = list(slots) + [slots[0]] * (self.batch - live)
        self.lengths_before = lengths.tolist()
        self.n_new = [1] * self.batch
        self.host_row_pos = lengths
        self.dev.copy_(host, non_blocking=True)


class DecodeLoop:
    """Single-token steps of a set of live sequences: ``step`` chooses greedily on the device,
    ``step_logits`` hands the logits to a sampler."""

    def __init__(self, engine, use_graph: bool = True):
        self.engine = engine
        # a part that steers its work from the host (Python control flow over the step's
        # sequences) cannot be replayed from a recording; parts say so with graph_safe
        parts = [p for b in engine.model.blocks for p in (getattr(b, "mixer", None), getattr(b, "ffn", None))]
        self.use_graph = use_graph and all(getattr(p, "graph_safe", False) for p in parts if p is not None)
        # added rows would run a mixer's per-sequence state of some live slot: no padding then
        self.pad_batches = not engine.cache.state
        self._ctx: Dict[Tuple[int, int], _StaticContext] = {}
        self._graphs: Dict[tuple, Tuple[torch.cuda.CUDAGraph, torch.Tensor]] = {}    # (batch, width, choice)
        self._uses: Dict[tuple, int] = {}
        self.slots: List[int] = []
        self.pending: List[int] = []

    def start(self, slots: Sequence[int], tokens: Sequence[int]) -> None:
        """The sequences to continue and the token each feeds next."""
        if len(slots) != len(tokens) or not slots:
            raise StepError("a decode loop needs one next token per sequence")
        self.slots = list(slots)
        self.pending = [int(t) for t in tokens]

    def close(self) -> None:
        self._graphs.clear()
        self._ctx.clear()
        self._uses.clear()

    def _key(self) -> Tuple[int, int]:
        cache = self.engine.cache
        need = max(pages_for(cache.length(s) + 1) for s in self.slots)
        batch = batch_bucket(len(self.slots)) if self.pad_batches else len(self.slots)
        return batch, ((need + WIDTH_STEP - 1) // WIDTH_STEP) * WIDTH_STEP

    def _choose(self, logits: torch.Tensor, ctx, choose) -> None:
        """The step's choice on the device, into ``ctx.next_ids``: the first maximum (``choose``
        is True) or a draw (``choose`` = (temperature, candidates, top_k, ln min_p or None, top_p
        or None, seed), what :meth:`Sampler.device_draw` gives) at the positions that follow from
        the step's own lengths."""
        if choose is True:
            ops.argmax(logits, out=ctx.next_ids)
        elif choose:
            temperature, k, top_k, log_min_p, top_p, seed = choose
            cand_ids, cand_z = ops.top_candidates(logits, temperature, k)
            ops.draw(cand_ids, cand_z, ctx.len_before, top_k, log_min_p, top_p, seed, out=ctx.next_ids)

    def _run(self, tokens: Sequence[int], choose):
        """One step of the live sequences feeding ``tokens``: the logits [B, vocab] and the
        buffer that holds the choice when ``choose`` asks for one (see :meth:`_choose`)."""
        eng = self.engine
        cache = eng.cache
        vocab = eng.model.vocab
        for t in tokens:
            if not 0 <= t < vocab:
                raise StepError(f"token id {t} is outside the vocabulary of {vocab}")
        ones = [1] * len(self.slots)
        for slot in self.slots:
            eng.check_positions(slot, 1)
        try:
            cache.reserve(self.slots, ones)
        except CacheError as e:
            raise StepError(str(e)) from None
        key = self._key()
        ctx = self._ctx.pop(key, None)
        if ctx is None:
            ctx = _StaticContext(eng, *key)
            while len(self._ctx) >= MAX_GRAPHS:          # the shape unused for longest goes, with
                self._forget(next(iter(self._ctx)))      # its pinned buffers and its recordings
        self._ctx[key] = ctx                             # most recently used last
        ctx.refresh(cache, self.slots, tokens)
        gkey = (*key, choose)
        entry = self._graphs.pop(gkey, None)
        if entry is not None:
            self._graphs[gkey] = entry          # most recently used last
            entry[0].replay()
            logits = entry[1]
        else:
            logits = eng.forward(ctx)
            self._choose(logits, ctx, choose)
            n = self._uses[gkey] = self._uses.pop(gkey, 0) + 1
            if self.use_graph and n >= CAPTURE_AFTER:
                self._capture(gkey, ctx, choose)
                del self._uses[gkey]                     # counted only until it is recorded
            while len(self._uses) > 4 * MAX_GRAPHS:      # choices seen once or twice and not again
                del self._uses[next(iter(self._uses))]
        cache.advance(self.slots, ones)
        live = len(self.slots)
        return logits[:live], ctx.next_ids[:live]

    def _capture(self, gkey, ctx, choose) -> None:
        """Record the launches of a step of this shape.  Capture runs nothing; replays read the
        ids, positions and page tables that ``refresh`` puts into the fixed buffers."""
        torch.cuda.synchronize()
        # Python's collector must not run inside the capture: what it finalizes (the pinned
        # buffers of earlier steps' contexts, graphs of loops long gone, anything that waited in
        # a reference cycle) calls into the HIP runtime, which refuses such calls on a capturing
        # stream, and the process aborts.  So it runs now, and not again until the capture ends.
        gc.collect()
        collecting = gc.isenabled()
        gc.disable()
        try:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                logits = self.engine.forward(ctx)
                self._choose(logits, ctx, choose)
        finally:
            if collecting:
                gc.enable()
        while len(self._graphs) >= MAX_GRAPHS:
            oldest = next(iter(self._graphs))
            del self._graphs[oldest]            # its memory pool goes with it
            if not any(k[:2] == oldest[:2] for k in self._graphs) and oldest[:2] != gkey[:2]:
                self._ctx.pop(oldest[:2], None)         # no recording reads these buffers any more
        self._graphs[gkey] = (graph, logits)

    def _forget(self, key: Tuple[int, int]) -> None:
        """Drop a step shape: its fixed buffers, and the recordings and counts that belong to it."""
        self._ctx.pop(key, None)
        for table in (self._graphs, self._uses):
            for k in [k for k in table if k[:2] == key]:
                del table[k]

    def step(self, draw=None) -> List[int]:
        """Feed the pending tokens and choose on the device, greedily or with ``draw`` (what
        :meth:`Sampler.device_draw` gives); the new token of every sequence, which is also what
        the next step feeds."""
        _, ids = self._run(self.pending, choose=draw if draw else True)
        self.pending = ids.tolist()
        return self.pending

    def step_logits(self, tokens: Optional[Sequence[int]] = None) -> torch.Tensor:
        """Feed ``tokens`` (default: the pending ones); float32 logits [B, vocab] of the new
        positions, valid until the next step."""
        if tokens is not None:
            self.pending = [int(t) for t in tokens]
        logits, _ = self._run(self.pending, choose=False)
        return logits

    def keep(self, flags: Sequence[bool], tokens: Optional[Sequence[int]] = None) -> None:
        """Go on with the sequences whose flag is true; ``tokens`` (default: the pending ones)
        are filtered alike and become what the next step feeds."""
        src = self.pending if tokens is None else [int(t) for t in tokens]
        self.slots = [s for s, k in zip(self.slots, flags) if k]
        self.pending = [t for t, k in zip(src, flags) if k]

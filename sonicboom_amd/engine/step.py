"""The step function: a batch of sequences, the tokens each brings, logits back.

A step carries, for every sequence, either its whole prompt (all sequences of
the batch start together, lengths differ) or one more token.  The rows of all
sequences are laid end to end — there is no padding — and run as one batch
through the model from the cache that earlier steps left: row r of sequence s
sits at position ``length(s) + r``, stores its key and value there, and sees
the keys at or before its own position.  The logits come back only for the
rows that were asked for, in the order of the entries and of their ``want``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Sequence

import numpy as np
import torch

from ..cache.paged import CacheError, PagedCache
from .model import DecoderModel


# Rows that run as one batch.  More than this and a step runs in portions: the tiled products
# are at their best rate from a few thousand rows on, and their operands (rows x inner width,
# two bytes each) must stay below 4 GiB.
MAX_STEP_ROWS = 16384


def portion_rows(n_new: Sequence[int], limit: int):
    """Cut a step of ``n_new[i]`` rows per sequence into portions of at most ``limit`` rows:
    a list of portions, each a list of (sequence, first row, end row).  Sequences stay in
    order and a sequence's rows ascend over the portions; a sequence is cut only where a
    portion is full."""
    if limit <= 0:
        raise ValueError("the row limit of a step must be positive")
    portions, cur, room = [], [], limit
    for i, n in enumerate(n_new):
        a = 0
        while a < n:
            b = min(n, a + room)
            cur.append((i, a, b))
            room -= b - a
            a = b
            if room == 0:
                portions.append(cur)
                cur, room = [], limit
    if cur:
        portions.append(cur)
    return portions


class StepError(ValueError):
    """A step that cannot run: unknown slot, token outside the vocabulary, no room in the cache."""


@dataclass
class StepEntry:
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()        # indices into ``tokens`` whose logits are wanted


class StepContext:
    """Row and sequence bookkeeping of one step, on the host and on the device.

    Device tensors (int32): ``ids`` [rows], ``row_pos`` [rows] absolute
    positions, ``row_seq`` [rows] index of the row's sequence in the batch,
    ``cu_rows`` [seqs+1] first row of every sequence, ``len_before`` [seqs]
    cached length before the step, ``slots`` [seqs] (rows of the state
    tensors), ``want_rows`` [wanted]; ``row_tiles(h)`` [n, 4] (first row, rows <= h,
    sequence, 0: runs of consecutive rows of one sequence, for every height ``h`` that a
    mixer of the model has asked for with its ``row_tile`` attribute);
    ``page_table(group)`` [seqs, pages].
    Host: ``n_rows``, ``n_seqs``, ``n_new`` list, ``lengths_before`` list,
    ``is_decode`` (every sequence brings one token), ``max_new``,
    ``max_len_after``.
    """

    def __init__(self, cache: PagedCache, entries: Sequence[StepEntry], device, row_tiles: Sequence[int] = ()):
        self.n_seqs = len(entries)
        self.n_new = [len(e.tokens) for e in entries]
        self.slot_list = [e.slot for e in entries]
        self.lengths_before = [cache.length(s) for s in self.slot_list]
        self.n_rows = sum(self.n_new)
        self.is_decode = all(n == 1 for n in self.n_new)
        self.max_new = max(self.n_new)
        self.max_len_after = max(l + n for l, n in zip(self.lengths_before, self.n_new))
        cu = np.zeros(self.n_seqs + 1, dtype=np.int32)
        cu[1:] = np.cumsum(self.n_new)
        ids = np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries]).astype(np.int32)
        row_seq = np.repeat(np.arange(self.n_seqs, dtype=np.int32), self.n_new)
        row_pos = (np.arange(self.n_rows, dtype=np.int32) - cu[row_seq]
                   + np.asarray(self.lengths_before, dtype=np.int32)[row_seq]).astype(np.int32)
        want = [int(cu[i]) + int(w) for i, e in enumerate(entries) for w in e.want]
        self.n_wanted = len(want)
        tables = [cache.page_table(g, self.slot_list) for g in range(len(cache.groups))]
        # runs of up to h consecutive rows of one sequence: (first row, rows, sequence, 0)
        heights = sorted({int(h) for h in row_tiles})
        tiles = [np.asarray([(int(cu[i]) + r0, min(h, n - r0), i, 0)
                             for i, n in enumerate(self.n_new) for r0 in range(0, n, h)], dtype=np.int32)
                 for h in heights]
        parts = [ids, row_pos, row_seq, cu, np.asarray(self.lengths_before, dtype=np.int32),
                 np.asarray(self.slot_list, dtype=np.int32), np.asarray(want, dtype=np.int32)]
        parts += [t.reshape(-1) for t in tiles]
        parts += [t.reshape(-1) for t in tables]
        sizes = [p.size for p in parts]
        # One pinned staging buffer, one copy to the device, views into it.
        host = torch.empty(sum(sizes), dtype=torch.int32, pin_memory=(torch.device(device).type == "cuda"))
        host.numpy()[:] = np.concatenate(parts) if parts else np.zeros(0, np.int32)
        dev = host.to(device, non_blocking=True)
        self._host = host
        views, off = [], 0
        for n in sizes:
            views.append(dev[off:off + n])
            off += n
        (self.ids, self.row_pos, self.row_seq, self.cu_rows, self.len_before, self.slots,
         self.want_rows) = views[:7]
        self._tiles = {h: v.view(-1, 4) for h, v in zip(heights, views[7:7 + len(heights)])}
        self._tables = [v.view(t.shape) for v, t in zip(views[7 + len(heights):], tables)]
        self.host_row_pos = row_pos
        self.trace = None            # set by the engine while a tracer listens

    def page_table(self, group: int) -> torch.Tensor:
        return self._tables[group]

    def row_tiles(self, height: int) -> torch.Tensor:
        """The step's rows in runs of up to ``height`` consecutive rows of one sequence."""
        try:
            return self._tiles[int(height)]
        except KeyError:
            raise StepError(f"no mixer of the model has asked for row tiles of {height} rows "
                            f"(a mixer asks with its row_tile attribute; asked for: {sorted(self._tiles)})") from None


class Engine:
    """A model with its cache: slots, the step function, and the device."""

    def __init__(self, model: DecoderModel, max_tokens: int, max_slots: Optional[int] = None,
                 max_step_rows: int = MAX_STEP_ROWS, max_positions: Optional[int] = None):
        """``max_positions``: the longest sequence a step accepts; None takes the model's own
        bound (its configuration's maximum of positions), 0 sets none."""
        self.model = model
        self.max_step_rows = int(max_step_rows)
        own = int(getattr(model.spec, "max_positions", 0) or 0)
        self.max_positions = own if max_positions is None else int(max_positions)
        self.device = model.rt.device
        self.cache = model.new_cache(max_tokens, max_slots)
        self.bindings = model.bindings(self.cache)
        self.use_graphs = True
        self._loop = None
        # set to a callable (name, tensor) to receive a step's named intermediates, in the order of
        # the computation: "embedding", "entry<i>.after_mixer", "entry<i>.after_ffn", "logits"
        self.tracer = None

    def decode_loop(self):
        """The engine's loop for single-token steps (one per engine: it keeps the captured graphs)."""
        if self._loop is None:
            from .decode import DecodeLoop
            self._loop = DecodeLoop(self, use_graph=self.use_graphs)
        return self._loop

    # ---- slots -----------------------------------------------------------------
    def alloc_slot(self) -> int:
        return self.cache.alloc_slot()

    def free_slot(self, slot: int) -> None:
        self.cache.free_slot(slot)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    # ---- the step ----------------------------------------------------------------
    def _check(self, entries: Sequence[StepEntry]) -> None:
        if not entries:
            raise StepError("a step needs at least one sequence")
        vocab = self.model.vocab
        for e in entries:
            n = len(e.tokens)
            if n == 0:
                raise StepError(f"slot {e.slot}: a step must bring at least one token")
            lo, hi = min(e.tokens), max(e.tokens)
            if lo < 0 or hi >= vocab:
                raise StepError(f"slot {e.slot}: token id {hi if hi >= vocab else lo} is outside the vocabulary of {vocab}")
            for w in e.want:
                if not 0 <= w < n:
                    raise StepError(f"slot {e.slot}: wanted row {w} is not among the {n} tokens of this step")
            self.check_positions(e.slot, n)

    def check_positions(self, slot: int, n_new: int) -> None:
        """Refuse ``n_new`` more tokens of ``slot`` when they pass the bound on positions."""
        if self.max_positions > 0:
            try:
                after = self.cache.length(slot) + n_new
            except CacheError as e:
                raise StepError(str(e)) from None
            if after > self.max_positions:
                raise StepError(f"slot {slot}: {after} tokens pass the model's {self.max_positions} positions")

    def step(self, entries: Sequence[StepEntry]) -> torch.Tensor:
        """Run the entries' tokens; float32 logits [wanted rows, vocab] on the device.

        A step of more than ``max_step_rows`` rows runs in portions, one after the other from
        the cache the earlier ones left: whole sequences while they fit, a sequence cut where
        the portion is full.  The logits come back in the order of the entries and of their
        ``want`` all the same."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        try:
            self._check(entries)
            slots = [e.slot for e in entries]
            n_new = [len(e.tokens) for e in entries]
            self.cache.reserve(slots, n_new)
        except CacheError as e:
            raise StepError(str(e)) from None
        portions = portion_rows(n_new, self.max_step_rows)
        if len(portions) == 1:
            ctx = StepContext(self.cache, entries, self.device, self.model.row_tiles)
            logits = self.forward(ctx)
            self.cache.advance(slots, n_new)
            return logits
        pieces, place = [], []          # place[i] = (entry, index in its want) of output row i
        for portion in portions:
            sub = []
            for i, a, b in portion:
                e = entries[i]
                picked = [(k, w - a) for k, w in enumerate(e.want) if a <= w < b]
                sub.append(StepEntry(e.slot, e.tokens[a:b], [w for _, w in picked]))
                place += [(i, k) for k, _ in picked]
            ctx = StepContext(self.cache, sub, self.device, self.model.row_tiles)
            pieces.append(self.forward(ctx))
            self.cache.advance([e.slot for e in sub], [len(e.tokens) for e in sub])
        logits = torch.cat(pieces, dim=0)
        order = sorted(range(len(place)), key=place.__getitem__)
        if order != list(range(len(place))):
            logits = logits[torch.tensor(order, dtype=torch.long, device=logits.device)]
        return logits

    def forward(self, ctx) -> torch.Tensor:
        """The device work of a step whose bookkeeping ``ctx`` holds: embedding, the blocks in
        their run order, and for the wanted rows the final norm and the head."""
        model = self.model
        tracer = self.tracer
        x = model.embedding.forward(ctx.ids)
        if tracer is not None:
            tracer("embedding", x)
        h = None
        for i, e in enumerate(model.order):
            nxt = model.order[i + 1].block if i + 1 < len(model.order) else None
            next_norm = getattr(model.blocks[nxt], "first_norm", None) if nxt is not None else None
            # a block reports what it has computed through ctx.trace, if it cares to
            ctx.trace = (lambda what, t, _i=i: tracer(f"entry{_i}.{what}", t)) if tracer is not None else None
            h = model.blocks[e.block].forward(x, ctx, self.bindings[i], h=h, next_norm=next_norm)
        ctx.trace = None
        if ctx.n_wanted == 0:
            return torch.empty((0, model.vocab), dtype=torch.float32, device=self.device)
        h = model.final_norm.forward(x, model.rt.act_dtype, rows=ctx.want_rows)
        logits = model.head.forward(h)
        if tracer is not None:
            tracer("logits", logits)
        return logits

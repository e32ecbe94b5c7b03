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


class ContextLayout:
    """The int32 tables of a step and where each lies in the one buffer that carries them to the
    device: the single description of that buffer, for a step whose tables are computed on the
    spot (:class:`StepContext`) and for the decode loop's fixed buffers that are refilled every
    step (``engine/decode.py``).

    Fields, in order: ``ids``, ``row_pos``, ``row_seq`` [rows]; ``cu_rows`` [seqs + 1];
    ``len_before``, ``slots`` [seqs]; ``want_rows`` [wanted]; for every row-tile height ``h``
    that a mixer of the model has asked for, ``("tiles", h)`` [n, 4] = (first row, rows <= h,
    sequence, 0); for every cache group ``g``, ``("table", g)`` [seqs, width]."""

    def __init__(self, n_rows: int, n_seqs: int, n_wanted: int, tiles, tables):
        """``tiles``: {height: number of runs}; ``tables``: per cache group (rows, width)."""
        self.heights = sorted(int(h) for h in tiles)
        self.shapes = {"ids": (n_rows,), "row_pos": (n_rows,), "row_seq": (n_rows,), "cu_rows": (n_seqs + 1,),
                       "len_before": (n_seqs,), "slots": (n_seqs,), "want_rows": (n_wanted,)}
        for h in self.heights:
            self.shapes[("tiles", h)] = (int(tiles[h]), 4)
        for g, shape in enumerate(tables):
            self.shapes[("table", g)] = tuple(int(n) for n in shape)
        self.n_groups = len(tables)
        self.offsets, off = {}, 0
        for key, shape in self.shapes.items():
            self.offsets[key] = off
            off += int(np.prod(shape, dtype=np.int64))
        self.total = off

    def view(self, buffer, key):
        """The part of ``buffer`` (a torch tensor or NumPy array of ``total`` int32) that holds ``key``."""
        shape = self.shapes[key]
        off = self.offsets[key]
        return buffer[off:off + int(np.prod(shape, dtype=np.int64))].reshape(shape)

    def bind(self, ctx, device_buffer) -> None:
        """Give ``ctx`` its device tensors as views of ``device_buffer``."""
        for name in ("ids", "row_pos", "row_seq", "cu_rows", "len_before", "slots", "want_rows"):
            setattr(ctx, name, self.view(device_buffer, name))
        ctx._tiles = {h: self.view(device_buffer, ("tiles", h)) for h in self.heights}
        ctx._tables = [self.view(device_buffer, ("table", g)) for g in range(self.n_groups)]


def row_runs(n_new: Sequence[int], cu, height: int) -> np.ndarray:
    """int32 [n, 4]: the rows of a step in runs of up to ``height`` consecutive rows of one
    sequence, as (first row, rows, sequence, 0)."""
    runs = [(int(cu[i]) + r0, min(height, n - r0), i, 0) for i, n in enumerate(n_new) for r0 in range(0, n, height)]
    return np.asarray(runs, dtype=np.int32).reshape(-1, 4)


class _Context:
    """What the parts read of a step's bookkeeping (see :class:`StepContext`)."""

    trace = None            # set by the engine while a tracer listens

    def page_table(self, group: int) -> torch.Tensor:
        return self._tables[group]

    def row_tiles(self, height: int) -> torch.Tensor:
        """The step's rows in runs of up to ``height`` consecutive rows of one sequence."""
        try:
            return self._tiles[int(height)]
        except KeyError:
            raise StepError(f"no mixer of the model has asked for row tiles of {height} rows "
                            f"(a mixer asks with its row_tile attribute; asked for: {sorted(self._tiles)})") from None


class StepContext(_Context):
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
    ``max_len_after``, ``host_row_pos``.
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
        row_seq = np.repeat(np.arange(self.n_seqs, dtype=np.int32), self.n_new)
        row_pos = (np.arange(self.n_rows, dtype=np.int32) - cu[row_seq]
                   + np.asarray(self.lengths_before, dtype=np.int32)[row_seq]).astype(np.int32)
        want = [int(cu[i]) + int(w) for i, e in enumerate(entries) for w in e.want]
        self.n_wanted = len(want)
        values = {
            "ids": np.concatenate([np.asarray(e.tokens, dtype=np.int64) for e in entries]).astype(np.int32),
            "row_pos": row_pos, "row_seq": row_seq, "cu_rows": cu,
            "len_before": np.asarray(self.lengths_before, dtype=np.int32),
            "slots": np.asarray(self.slot_list, dtype=np.int32), "want_rows": np.asarray(want, dtype=np.int32),
        }
        for h in sorted({int(h) for h in row_tiles}):
            values[("tiles", h)] = row_runs(self.n_new, cu, h)
        for g in range(len(cache.groups)):
            values[("table", g)] = cache.page_table(g, self.slot_list)
        layout = ContextLayout(self.n_rows, self.n_seqs, self.n_wanted,
                               {k[1]: len(v) for k, v in values.items() if isinstance(k, tuple) and k[0] == "tiles"},
                               [values[("table", g)].shape for g in range(len(cache.groups))])
        # One pinned staging buffer, one copy to the device, views into it.
        host = torch.empty(layout.total, dtype=torch.int32, pin_memory=(torch.device(device).type == "cuda"))
        flat = host.numpy()
        for key, v in values.items():
            layout.view(flat, key)[...] = v
        self._host = host
        layout.bind(self, host.to(device, non_blocking=True))
        self.host_row_pos = row_pos


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
        self.cache = model.new_cache(max_tokens, max_slots, step_rows=self.max_step_rows)
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
        ``want`` all the same.  When a portion fails (a kernel refuses a size, memory runs out),
        the portions before it stay in the cache, the sequences' lengths count them, the pages
        reserved for the rest are given back and the logits of the step are lost: free the slots,
        or look at ``length(slot)`` and feed the remaining tokens again."""
        entries = [e if isinstance(e, StepEntry) else StepEntry(*e) for e in entries]
        cache = self.cache
        slots = [e.slot for e in entries]
        n_new = [len(e.tokens) for e in entries]
        portions = portion_rows(n_new, self.max_step_rows)
        try:
            self._check(entries)
            # all or nothing: the groups that keep every key take the pages of all rows now;
            # windowed groups, whose pools hold a window and one portion a sequence, take theirs
            # portion by portion (a single portion: everything at once)
            cache.reserve(slots, n_new, None if len(portions) == 1 else cache.windowed(False))
        except CacheError as e:
            raise StepError(str(e)) from None
        if len(portions) == 1:
            ctx = StepContext(cache, entries, self.device, self.model.row_tiles)
            try:
                logits = self.forward(ctx)
            except BaseException:
                cache.trim(slots)               # the rows did not run: their pages go back
                raise
            cache.advance(slots, n_new)
            return logits
        pieces, place = [], []          # place[i] = (entry, index in its want) of output row i
        try:
            for portion in portions:
                sub = []
                for i, a, b in portion:
                    e = entries[i]
                    picked = [(k, w - a) for k, w in enumerate(e.want) if a <= w < b]
                    sub.append(StepEntry(e.slot, e.tokens[a:b], [w for _, w in picked]))
                    place += [(i, k) for k, _ in picked]
                sub_slots, sub_new = [e.slot for e in sub], [len(e.tokens) for e in sub]
                cache.reserve(sub_slots, sub_new, cache.windowed(True))
                ctx = StepContext(cache, sub, self.device, self.model.row_tiles)
                pieces.append(self.forward(ctx))
                cache.advance(sub_slots, sub_new)
        except BaseException as e:
            # A portion failed.  The portions before it have run: their rows are in the cache and
            # the sequences' lengths say so; what was reserved for the rows that did not run goes
            # back.  The caller frees the slots or feeds the remaining tokens again.
            cache.trim(slots)
            if isinstance(e, CacheError):
                raise StepError(str(e)) from None
            raise
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
        x = model.embedding.forward(ctx.ids, ctx)
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

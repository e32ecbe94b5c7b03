"""The cache: a slot per sequence, paged keys and values per layer, and
per-sequence state of fixed size.

* A **slot** stands for one live sequence: its length and, per group, the list
  of physical pages that hold its keys and values.  Slots are handed out by
  :meth:`PagedCache.alloc_slot`, given back by :meth:`free_slot` and used again.
* Cache entries (one per mixer that stores keys) with the same needs
  (kv heads, head size, window) form a **group** with storage and a page pool
  of its own: ``K: [entries, pages, kv_heads, PAGE, head_dim]`` and ``V`` with
  the last two axes swapped.  A mixer may keep something else per token instead:
  rows of a shape of its own, ``[entries, pages, PAGE, *shape]``, in groups by
  (shape, window).  A group
  that only reads a window of keys gives pages back as the window leaves them.
* ``max_tokens`` sizes the pools: the most tokens live sequences hold at any
  time, each sequence's count rounded up to a whole page (PAGE = 64 tokens).
  A group that keeps every key gets that many pages.  A group with a window
  never holds more of a sequence than its window and the rows of the step
  that is running, so with ``max_slots`` sequences and steps of at most
  ``step_rows`` rows its pool is ``max_slots * (pages(window) + 2) +
  pages(step_rows)`` pages when that is less (:func:`pool_pages`).
* **State**: an entry whose mixer asks for fixed-size state gets a tensor
  ``[max_slots, *shape]``; a slot's row is zeroed when the slot is handed out,
  because a recurrence reads its state before it writes it.  Keys and values
  of a reused page are not cleared: nothing may depend on them.

The reference keeps one sequence per session, position j at row j mod n_slots
(/root/reference/core/src/planner/kv_cache.h:69-89, :125-170), with per-layer
specs {kv_heads, head_dim, window} (:96-117) and opaque per-block states
(:140-152); the batch of slots and the pages are this engine's own.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from ..csrc.header import PAGE          # tokens per page: SB_PAGE of csrc/sb_hip.h


class CacheError(RuntimeError):
    """Out of pages or slots, or a slot used wrongly (unknown, freed twice)."""


def pages_for(tokens: int) -> int:
    return (tokens + PAGE - 1) // PAGE


class PagePool:
    """Free list of physical page numbers; refuses a double free."""

    def __init__(self, n_pages: int):
        self.n_pages = n_pages
        self._free = list(range(n_pages - 1, -1, -1))
        self._held = [False] * n_pages

    @property
    def free_count(self) -> int:
        return len(self._free)

    def alloc(self) -> int:
        if not self._free:
            raise CacheError("out of cache pages")
        p = self._free.pop()
        self._held[p] = True
        return p

    def free(self, page: int) -> None:
        if not 0 <= page < self.n_pages or not self._held[page]:
            raise CacheError(f"page {page} freed while not held")
        self._held[page] = False
        self._free.append(page)


@dataclass(frozen=True)
class GroupSpec:
    kv_heads: int
    head_dim: int
    window: int                  # 0: every key is kept
    entries: Tuple[int, ...]     # cache entry numbers stored in this group
    row_shape: Tuple[int, ...] = ()   # not empty: a row of this shape per token instead of keys and values


@dataclass
class _Slot:
    length: int = 0
    pages: List[List[int]] = field(default_factory=list)   # per group: logical page -> physical or -1


def pool_pages(n_pages: int, window: int, max_slots: int, step_rows: int) -> int:
    """Pages of a group's pool in a cache of ``n_pages``: all of them for a group that keeps
    every key (``window`` 0); for a windowed group what ``max_slots`` sequences can hold at
    once, if that is less: after a step a sequence keeps the pages its window touches
    (pages(window) + 1 at most), and a step of up to ``step_rows`` rows adds pages(rows) + 1 pages
    a sequence before the old ones are given back."""
    if window <= 0 or step_rows <= 0:
        return n_pages
    return min(n_pages, max_slots * (pages_for(window) + 2) + pages_for(step_rows))


class PagedCache:
    def __init__(self, groups: Sequence[GroupSpec], max_tokens: int, dtype=None, device=None,
                 state_shapes: Optional[Dict[int, tuple]] = None, max_slots: Optional[int] = None,
                 allocate: bool = True, step_rows: int = 0):
        """``step_rows``: the most rows the caller feeds between two calls of :meth:`advance`
        (0: no bound is promised, and every group gets pages for ``max_tokens``)."""
        if max_tokens <= 0:
            raise CacheError("max_tokens must be positive")
        self.groups = list(groups)
        self.n_pages = pages_for(max_tokens)
        self.max_slots = max_slots if max_slots is not None else self.n_pages
        self.step_rows = int(step_rows)
        self.pools = [PagePool(pool_pages(self.n_pages, g.window, self.max_slots, self.step_rows))
                      for g in self.groups]
        self._slots: Dict[int, _Slot] = {}
        self._free_slots = list(range(self.max_slots - 1, -1, -1))
        self.entry_place: Dict[int, Tuple[int, int]] = {}      # entry -> (group, index within group)
        for g, spec in enumerate(self.groups):
            for i, e in enumerate(spec.entries):
                if e in self.entry_place:
                    raise CacheError(f"cache entry {e} is in two groups")
                self.entry_place[e] = (g, i)
        self.k: List = []
        self.v: List = []
        self.state: Dict[int, object] = {}
        self.dtype, self.device = dtype, device
        if allocate:
            import torch
            for spec, pool in zip(self.groups, self.pools):
                n, pages = len(spec.entries), pool.n_pages
                if spec.row_shape:
                    self.k.append(torch.zeros((n, pages, PAGE, *spec.row_shape), dtype=dtype, device=device))
                    self.v.append(None)
                    continue
                # keys [.., position, d]; values transposed [.., d, position] (see csrc/sb_hip.h)
                self.k.append(torch.zeros((n, pages, spec.kv_heads, PAGE, spec.head_dim),
                                          dtype=dtype, device=device))
                self.v.append(torch.zeros((n, pages, spec.kv_heads, spec.head_dim, PAGE),
                                          dtype=dtype, device=device))
            for key, (shape, sdtype) in (state_shapes or {}).items():
                self.state[key] = torch.zeros((self.max_slots, *shape), dtype=sdtype, device=device)

    # ---- slots -------------------------------------------------------------
    def alloc_slot(self) -> int:
        if not self._free_slots:
            raise CacheError("out of sequence slots")
        s = self._free_slots.pop()
        self._slots[s] = _Slot(0, [[] for _ in self.groups])
        for st in self.state.values():
            st[s].zero_()
        return s

    def free_slot(self, slot: int) -> None:
        sl = self._slots.pop(slot, None)
        if sl is None:
            raise CacheError(f"slot {slot} freed while not in use")
        for g, pages in enumerate(sl.pages):
            for p in pages:
                if p >= 0:
                    self.pools[g].free(p)
        self._free_slots.append(slot)

    def _slot(self, slot: int) -> _Slot:
        try:
            return self._slots[slot]
        except KeyError:
            raise CacheError(f"slot {slot} is not in use") from None

    def length(self, slot: int) -> int:
        return self._slot(slot).length

    @property
    def live_slots(self) -> List[int]:
        return sorted(self._slots)

    def free_pages(self) -> int:
        """Pages that every group can still hand out (the least over the groups' pools)."""
        return min((p.free_count for p in self.pools), default=self.n_pages)

    def free_slots(self) -> int:
        return len(self._free_slots)

    def held_pages(self, group: int = 0) -> int:
        return self.pools[group].n_pages - self.pools[group].free_count

    # ---- a step ------------------------------------------------------------
    def _first_needed_page(self, g: int, length: int) -> int:
        """Logical page of the oldest key that a query at position ``length`` still reads."""
        w = self.groups[g].window
        if w <= 0:
            return 0
        return max(0, length - w + 1) // PAGE

    def windowed(self, flag: bool) -> List[int]:
        """The groups that read a window of keys (``flag`` true) or every key (false)."""
        return [g for g, spec in enumerate(self.groups) if (spec.window > 0) == flag]

    def reserve(self, slots: Sequence[int], n_new: Sequence[int], groups: Optional[Sequence[int]] = None) -> None:
        """Pages for ``n_new[i]`` more tokens of ``slots[i]``, all or nothing; ``groups``: in
        these groups only (a long step reserves the groups that keep every key for all its rows
        at once, and the windowed ones portion by portion, as their pools are sized)."""
        if len(set(slots)) != len(slots):
            raise CacheError("a slot appears twice in one step")
        groups = range(len(self.groups)) if groups is None else list(groups)
        need = {g: 0 for g in groups}
        for s, n in zip(slots, n_new):
            if n <= 0:
                raise CacheError("a step must bring at least one token for every sequence")
            sl = self._slot(s)
            for g in groups:
                need[g] += max(0, pages_for(sl.length + n) - len(sl.pages[g]))
        for g, n in need.items():
            if n > self.pools[g].free_count:
                raise CacheError(
                    f"out of cache pages: the step needs {n} more pages of {PAGE} tokens, "
                    f"{self.pools[g].free_count} of {self.pools[g].n_pages} are free")
        for s, n in zip(slots, n_new):
            sl = self._slots[s]
            for g in groups:
                while len(sl.pages[g]) < pages_for(sl.length + n):
                    sl.pages[g].append(self.pools[g].alloc())

    def trim(self, slots: Sequence[int]) -> None:
        """Give back the pages that ``slots`` hold beyond their lengths: what a step reserved
        for rows that did not run."""
        for s in slots:
            sl = self._slot(s)
            for g, pages in enumerate(sl.pages):
                while len(pages) > pages_for(sl.length):
                    p = pages.pop()
                    if p >= 0:
                        self.pools[g].free(p)

    def page_table(self, group: int, slots: Sequence[int], min_width: int = 1) -> np.ndarray:
        """int32 [len(slots), width]: logical page -> physical page, -1 for none."""
        rows = [self._slot(s).pages[group] for s in slots]
        width = max([min_width] + [len(r) for r in rows])
        t = np.full((len(rows), width), -1, dtype=np.int32)
        for i, r in enumerate(rows):
            t[i, :len(r)] = r
        return t

    def advance(self, slots: Sequence[int], n_new: Sequence[int]) -> None:
        """The step has run: lengths grow; windowed groups give back pages no later query reads."""
        for s, n in zip(slots, n_new):
            sl = self._slot(s)
            sl.length += n
            for g in range(len(self.groups)):
                first = self._first_needed_page(g, sl.length)
                pages = sl.pages[g]
                for i in range(min(first, len(pages))):
                    if pages[i] >= 0:
                        self.pools[g].free(pages[i])
                        pages[i] = -1

    # ---- taking a sequence back ----------------------------------------------
    def can_truncate(self, slot: int, length: int) -> bool:
        """Whether ``slot`` can go back to its first ``length`` tokens: not when a mixer keeps
        per-sequence state (a recurrence cannot be run backwards), and not below what a windowed
        group still holds (the pages its window has left are gone)."""
        sl = self._slot(slot)
        if not 0 <= length <= sl.length:
            return False
        if length == sl.length:
            return True
        if self.state:
            return False
        return all(self._first_needed_page(g, sl.length) == self._first_needed_page(g, length)
                   for g in range(len(self.groups)))

    def truncate(self, slot: int, length: int) -> None:
        """Forget all but the first ``length`` tokens of ``slot``: the next step's rows start at
        position ``length`` and see the keys before it, as if the later tokens had never been
        fed.  Pages past the new end go back to their pools (what a kept page holds past the new
        end is never read: a row sees keys up to its own position only)."""
        if not self.can_truncate(slot, length):
            sl = self._slot(slot)
            raise CacheError(f"slot {slot} holds {sl.length} tokens and cannot go back to {length}"
                             + (": its per-sequence state cannot be taken back" if self.state and 0 <= length < sl.length
                                else ": a windowed group has given up the keys before it" if 0 <= length < sl.length else ""))
        sl = self._slots[slot]
        sl.length = length
        self.trim([slot])

    # ---- storage -------------------------------------------------------------
    def entry_views(self, entry: int):
        """(keys [pages, kv_heads, PAGE, head_dim], values [pages, kv_heads, head_dim, PAGE]) of one
        cache entry, and its group; for an entry of a group of rows (rows [pages, PAGE, *shape], None)."""
        g, i = self.entry_place[entry]
        return self.k[g][i], (None if self.v[g] is None else self.v[g][i]), g


def group_entries(specs: Dict[int, tuple]) -> List[GroupSpec]:
    """Group cache entries {entry: (kv_heads, head_dim, window)}, or {entry: ("rows", shape, window)}
    for entries that keep a row of their own shape per token, by equal needs, in order of first use."""
    by_need: Dict[tuple, List[int]] = {}
    for e in sorted(specs):
        by_need.setdefault(tuple(specs[e]), []).append(e)
    return [GroupSpec(0, 0, k[2], tuple(v), tuple(k[1])) if k[0] == "rows" else GroupSpec(k[0], k[1], k[2], tuple(v))
            for k, v in by_need.items()]

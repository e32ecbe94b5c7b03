"""Sequences that stay in the cache after their request has ended, so that a later request which
starts with the same tokens feeds only what is new.

The reference's session keeps the tokens it has prefilled and, at the next prompt, reuses their
longest common prefix (/root/reference/core/include/sonicboom/planner/kv_cache.h:131, :163-169),
capped at n - 1 because the last prompt token's own row is what gives the next token's logits
(/root/reference/capi/src/capi.cpp:2386-2393).  Here a session holds many sequences: every
request of a call that asks for it leaves its slot behind with the tokens that are in the cache;
the next call gives each of its prompts the kept sequence it shares the longest prefix with,
takes that sequence back to the shared prefix and feeds the rest.  Kept sequences that no prompt
of the next call continues are freed when that call starts: a session remembers one call back,
as the reference's remembers one prompt back.

The logits of a reused request are those of the same request fed whole: the rows it feeds run
from the cache exactly as the rows of a prompt cut into steps do (to the bit in 32-bit).
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple


def common_prefix_len(a: Sequence[int], b: Sequence[int]) -> int:
    n = min(len(a), len(b))
    i = 0
    while i < n and a[i] == b[i]:
        i += 1
    return i


class KeptSequences:
    def __init__(self, engine):
        self.engine = engine
        self.items: List[Tuple[int, List[int]]] = []      # (slot, the tokens its cache holds)
        self.reused: List[int] = []                       # per request of the last call: tokens not fed again

    def put(self, slot: int, tokens: Sequence[int]) -> None:
        """Keep ``slot``; ``tokens`` are what has been fed to it (its cached length)."""
        tokens = list(tokens)
        if len(tokens) != self.engine.length(slot):
            raise ValueError(f"slot {slot} holds {self.engine.length(slot)} tokens, not the {len(tokens)} given")
        self.items.append((slot, tokens))

    def match(self, prompts: Sequence[Sequence[int]]) -> List[Optional[Tuple[int, int]]]:
        """For every prompt, in order, the kept sequence with the longest common prefix that can
        be taken back to it: (slot, tokens reused) with the slot already cut to those tokens, or
        None.  A prompt reuses at most all but its last token.  Matched sequences leave the
        store."""
        out: List[Optional[Tuple[int, int]]] = []
        cache = self.engine.cache
        for p in prompts:
            best, best_n = -1, 0
            for k, (slot, tokens) in enumerate(self.items):
                n = min(common_prefix_len(tokens, p), len(p) - 1)
                if n > best_n and cache.can_truncate(slot, n):
                    best, best_n = k, n
            if best < 0:
                out.append(None)
                continue
            slot, _ = self.items.pop(best)
            cache.truncate(slot, best_n)
            out.append((slot, best_n))
        self.reused = [m[1] if m else 0 for m in out]
        return out

    def make_room(self, pages: int, slots: int) -> None:
        """Free kept sequences, the oldest first, until the cache can hand out ``pages`` pages
        and ``slots`` slots (or none is left to free)."""
        cache = self.engine.cache
        while self.items and (cache.free_pages() < pages or cache.free_slots() < slots):
            slot, _ = self.items.pop(0)
            self.engine.free_slot(slot)

    def drop_all(self) -> None:
        """Free every kept sequence."""
        for slot, _ in self.items:
            self.engine.free_slot(slot)
        self.items = []

    def __len__(self) -> int:
        return len(self.items)

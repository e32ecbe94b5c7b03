"""The step function's bookkeeping on the CPU, with a model that computes nothing: portions of a
long step, what a failure in a later portion leaves behind, and the one layout of a step's
tables."""
import numpy as np
import pytest
import torch

from sonicboom_amd.cache import GroupSpec, PagedCache
from sonicboom_amd.engine.step import ContextLayout, Engine, StepContext, StepEntry, StepError, row_runs

VOCAB = 50


class NoModel:
    """What Engine asks of a model, without parts: two cache groups (all keys, a window of 40)."""
    vocab, row_tiles = VOCAB, (16,)

    class spec:
        max_positions = 0

    class rt:
        device = torch.device("cpu")

    def new_cache(self, max_tokens, max_slots=None, step_rows=0):
        groups = [GroupSpec(1, 16, 0, (0,)), GroupSpec(1, 16, 40, (1,))]
        return PagedCache(groups, max_tokens, allocate=False, max_slots=max_slots, step_rows=step_rows)

    def bindings(self, cache):
        return []


def engine(fail_at=None, **options):
    eng = Engine(NoModel(), **options)
    eng.calls = []

    def forward(ctx):
        eng.calls.append((list(ctx.slot_list), list(ctx.n_new), list(ctx.lengths_before)))
        if fail_at is not None and len(eng.calls) == fail_at:
            raise RuntimeError("the kernel refused")
        return torch.zeros((ctx.n_wanted, VOCAB))
    eng.forward = forward
    return eng


def held(eng):
    return [eng.cache.held_pages(g) for g in range(2)]


def test_a_failure_in_a_later_portion_gives_the_unused_pages_back():
    eng = engine(fail_at=2, max_tokens=64 * 8, max_slots=2, max_step_rows=64)
    a, b = eng.alloc_slot(), eng.alloc_slot()
    ta, tb = list(range(40)) + list(range(49)) + [1] * 11, [3] * 60
    with pytest.raises(RuntimeError, match="refused"):
        eng.step([StepEntry(a, ta, (99,)), StepEntry(b, tb, (59,))])
    # the first portion (64 rows of a) has run and is counted; nothing else is held
    assert eng.calls == [([a], [64], [0]), ([a, b], [36, 28], [64, 0])]
    assert (eng.length(a), eng.length(b)) == (64, 0)
    assert held(eng) == [1, 1]
    # the caller feeds the rest again: the sequences end where the whole step would have
    eng.forward = lambda ctx: torch.zeros((ctx.n_wanted, VOCAB))
    out = eng.step([StepEntry(a, ta[64:], (35,)), StepEntry(b, tb, (59,))])
    assert tuple(out.shape) == (2, VOCAB) and (eng.length(a), eng.length(b)) == (100, 60)
    assert held(eng) == [3, 3]          # a: pages 0 and 1, b: page 0; the window of 40 keeps a's second page
    eng.free_slot(a)
    eng.free_slot(b)
    assert held(eng) == [0, 0]


def test_a_failure_in_a_step_of_one_portion_leaves_nothing_behind():
    eng = engine(fail_at=1, max_tokens=64 * 8)
    a = eng.alloc_slot()
    with pytest.raises(RuntimeError):
        eng.step([StepEntry(a, [1] * 70, ())])
    assert eng.length(a) == 0 and held(eng) == [0, 0]


def test_a_step_that_does_not_fit_reserves_nothing():
    eng = engine(max_tokens=64 * 3, max_step_rows=64)
    a = eng.alloc_slot()
    with pytest.raises(StepError, match="out of cache pages"):
        eng.step([StepEntry(a, [1] * 200, ())])
    assert not eng.calls and held(eng) == [0, 0] and eng.length(a) == 0


def test_one_layout_for_both_kinds_of_context():
    """The tables of a step lie where ContextLayout says, whoever fills them."""
    layout = ContextLayout(7, 3, 2, {4: 3, 16: 3}, [(3, 2), (3, 5)])
    sizes = {"ids": 7, "row_pos": 7, "row_seq": 7, "cu_rows": 4, "len_before": 3, "slots": 3, "want_rows": 2,
             ("tiles", 4): 12, ("tiles", 16): 12, ("table", 0): 6, ("table", 1): 15}
    assert {k: int(np.prod(v)) for k, v in layout.shapes.items()} == sizes and layout.total == sum(sizes.values())
    flat = np.arange(layout.total, dtype=np.int32)
    seen = np.concatenate([layout.view(flat, k).reshape(-1) for k in layout.shapes])
    assert np.array_equal(seen, flat)                         # every element in exactly one table, in order
    assert row_runs([5, 1, 9], [0, 5, 6, 15], 4).tolist() == [[0, 4, 0, 0], [4, 1, 0, 0], [5, 1, 1, 0], [6, 4, 2, 0],
                                                             [10, 4, 2, 0], [14, 1, 2, 0]]
    cache = NoModel().new_cache(64 * 8)
    s0, s1 = cache.alloc_slot(), cache.alloc_slot()
    cache.reserve([s0, s1], [70, 3])
    ctx = StepContext(cache, [StepEntry(s0, [5] * 70, (0, 69)), StepEntry(s1, [7, 8, 9], (2,))], "cpu", (16,))
    assert ctx.ids.tolist() == [5] * 70 + [7, 8, 9] and ctx.want_rows.tolist() == [0, 69, 72]
    assert ctx.row_pos.tolist() == list(range(70)) + [0, 1, 2] and ctx.cu_rows.tolist() == [0, 70, 73]
    assert ctx.row_tiles(16).tolist() == [[0, 16, 0, 0], [16, 16, 0, 0], [32, 16, 0, 0], [48, 16, 0, 0],
                                          [64, 6, 0, 0], [70, 3, 1, 0]]
    assert ctx.page_table(0).shape == (2, 2) and ctx.page_table(0)[1].tolist()[1] == -1
    with pytest.raises(StepError, match="row tiles of 8"):
        ctx.row_tiles(8)

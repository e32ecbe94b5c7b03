"""The generation loop's decisions, on the CPU with an engine whose "model" is a table:
batches one after another, unequal prompts, stop tokens, sequences that end earlier, slots
given back and used again, positions of the draws."""
import numpy as np
import pytest

from sonicboom_amd.cache import GroupSpec, PagedCache
from sonicboom_amd.engine.generate import generate, plan_batches
from sonicboom_amd.sampling import SamplingParams

VOCAB = 50


class TableEngine:
    """next token = (7 * last token + position) % VOCAB, delivered as one-hot logits.  Keeps the
    cache's books exactly as the real engine does and records every step."""

    def __init__(self, max_tokens, max_slots=None):
        self.cache = PagedCache([GroupSpec(1, 16, 0, (0,))], max_tokens, allocate=False, max_slots=max_slots)
        self.steps = []
        self.max_live = 0
        self.slot_uses = {}

    def alloc_slot(self):
        s = self.cache.alloc_slot()
        self.slot_uses[s] = self.slot_uses.get(s, 0) + 1
        self.max_live = max(self.max_live, len(self.cache.live_slots))
        return s

    def free_slot(self, s):
        self.cache.free_slot(s)

    def length(self, s):
        return self.cache.length(s)

    def step(self, entries):
        slots = [e.slot for e in entries]
        n_new = [len(e.tokens) for e in entries]
        self.cache.reserve(slots, n_new)
        rows = []
        for e in entries:
            base = self.cache.length(e.slot)
            for w in e.want:
                row = np.full(VOCAB, -1.0, dtype=np.float32)
                row[(7 * e.tokens[w] + base + w) % VOCAB] = 1.0
                rows.append(row)
        self.cache.advance(slots, n_new)
        self.steps.append([(e.slot, len(e.tokens)) for e in entries])
        return np.stack(rows)


class HostSampler:
    def __init__(self):
        self.positions = []

    def pick(self, logits, positions, histories):
        self.positions.append(list(positions))
        assert all(len(h) == p for h, p in zip(histories, positions))
        return [int(np.argmax(r)) for r in logits]


def expected(prompt, n, stop=()):
    seq, out = list(prompt), []
    for _ in range(n):
        t = (7 * seq[-1] + len(seq) - 1) % VOCAB
        out.append(t)
        seq.append(t)
        if t in stop:
            break
    return out


def test_unequal_prompts_in_one_batch():
    eng, smp = TableEngine(64 * 8), HostSampler()
    prompts = [[1, 2, 3, 4, 5], [9] * 9, [4] * 13]
    outs = generate(eng, prompts, SamplingParams(max_tokens=8), stop_tokens=(), sampler=smp)
    assert outs == [expected(p, 8) for p in prompts]
    assert eng.steps[0] == [(0, 5), (1, 9), (2, 13)]                 # the prompts in one step
    assert all(n == 1 for st in eng.steps[1:] for _, n in st)         # then one token each
    assert len(eng.steps) == 8                                        # the last token is not fed back
    assert smp.positions[0] == [5, 9, 13] and smp.positions[1] == [6, 10, 14]
    assert not eng.cache.live_slots and eng.cache.held_pages() == 0


def test_stop_token_is_emitted_and_ends_only_its_sequence():
    prompts = [[1, 2, 3], [5, 6], [8]]
    free = [expected(p, 10) for p in prompts]
    stop = (free[1][3],)
    want = [expected(p, 10, stop) for p in prompts]
    assert len(want[1]) == 4 and want[1][-1] == stop[0]
    eng = TableEngine(64 * 8)
    outs = generate(eng, prompts, SamplingParams(max_tokens=10), stop_tokens=stop, sampler=HostSampler())
    assert outs == want
    sizes = [len(st) for st in eng.steps]
    assert sizes[0] == 3 and min(sizes) < 3                           # the batch shrinks when one ends
    assert not eng.cache.live_slots


def test_batches_one_after_another_reuse_slots_and_pages():
    eng = TableEngine(64 * 3, max_slots=2)                            # room for two short requests at a time
    prompts = [[i + 1] * (3 + i) for i in range(7)]
    outs = generate(eng, prompts, SamplingParams(max_tokens=5), stop_tokens=(), max_batch=4, sampler=HostSampler())
    assert outs == [expected(p, 5) for p in prompts]
    assert eng.max_live == 2 and sum(eng.slot_uses.values()) == 7 and max(eng.slot_uses.values()) >= 3
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


def test_callback_and_max_tokens():
    eng = TableEngine(64 * 4)
    seen = []

    def cb(i, t):
        seen.append((i, t))
        return i == 0 and len([1 for j, _ in seen if j == 0]) == 3    # end request 0 at its third token

    outs = generate(eng, [[1, 2], [3]], SamplingParams(max_tokens=4), stop_tokens=(), callback=cb, sampler=HostSampler())
    # the token the callback refused is not reported (the reference's rule); it was shown to the callback
    assert outs == [expected([1, 2], 2), expected([3], 4)]
    assert [t for i, t in seen if i == 0] == expected([1, 2], 3)
    assert [t for i, t in seen if i == 1] == outs[1]
    assert generate(eng, [[1]], SamplingParams(max_tokens=0), sampler=HostSampler()) == [[]]
    assert generate(eng, [], SamplingParams(), sampler=HostSampler()) == []


def test_slots_come_back_when_a_step_fails():
    eng = TableEngine(64 * 4)

    def boom(entries):
        raise RuntimeError("device lost")
    eng.step = boom
    with pytest.raises(RuntimeError):
        generate(eng, [[1, 2, 3]], SamplingParams(max_tokens=3), sampler=HostSampler())
    assert not eng.cache.live_slots and eng.cache.held_pages() == 0


def test_plan_batches():
    assert plan_batches([5, 9, 13], 8, n_pages=8, max_batch=64) == [[0, 1, 2]]
    assert plan_batches([5, 9, 13], 8, n_pages=8, max_batch=2) == [[0, 1], [2]]
    assert plan_batches([60, 60, 60], 8, n_pages=4, max_batch=64) == [[0, 1], [2]]      # 2 pages each
    assert plan_batches([1] * 5, 1, n_pages=100, max_batch=64, max_slots=2) == [[0, 1], [2, 3], [4]]
    with pytest.raises(ValueError, match="request 1"):
        plan_batches([5, 300], 8, n_pages=4, max_batch=64)
    with pytest.raises(ValueError, match="empty prompt"):
        plan_batches([0], 8, n_pages=4, max_batch=64)


def test_portions_of_a_long_step():
    """A step above the row limit is cut into portions: sequences in order, a sequence cut only
    where a portion is full, every row exactly once."""
    from sonicboom_amd.engine.step import portion_rows
    assert portion_rows([3, 4], 10) == [[(0, 0, 3), (1, 0, 4)]]
    assert portion_rows([10], 10) == [[(0, 0, 10)]]
    assert portion_rows([11], 10) == [[(0, 0, 10)], [(0, 10, 11)]]
    # the second sequence starts in the first portion's last two rows and ends in the third
    assert portion_rows([8, 14, 1], 10) == [[(0, 0, 8), (1, 0, 2)], [(1, 2, 12)], [(1, 12, 14), (2, 0, 1)]]
    rng = np.random.default_rng(3)
    for _ in range(200):
        n_new = [int(n) for n in rng.integers(1, 40, size=rng.integers(1, 9))]
        limit = int(rng.integers(1, 50))
        portions = portion_rows(n_new, limit)
        assert all(sum(b - a for _, a, b in p) <= limit for p in portions)
        assert all(sum(b - a for _, a, b in p) == limit for p in portions[:-1])      # only the last is short
        flat = [(i, r) for p in portions for i, a, b in p for r in range(a, b)]
        assert flat == [(i, r) for i, n in enumerate(n_new) for r in range(n)]
    with pytest.raises(ValueError):
        portion_rows([3], 0)


def test_masks_reach_the_sampler_and_a_request_that_may_choose_nothing_ends():
    """``allowed`` is asked before every choice with the request's index and history; its bitmaps
    go to the sampler as ``masks``; a sampler's -1 (nothing may be chosen) ends that request
    without a token, frees its slot at once, and the others go on."""
    asked = []

    class MaskedSampler(HostSampler):
        def pick(self, logits, positions, histories, masks=None):
            assert masks is not None and len(masks) == len(positions)
            picks = super().pick(logits, positions, histories)
            return [-1 if m == b"\x00" else t for t, m in zip(picks, masks)]

    def allowed(i, history):
        asked.append((i, len(history)))
        return b"\x00" if i == 1 and len(history) >= 9 + 3 else None

    eng, smp = TableEngine(64 * 8), MaskedSampler()
    prompts = [[1, 2, 3, 4, 5], [9] * 9, [4] * 13]
    outs = generate(eng, prompts, SamplingParams(max_tokens=6), stop_tokens=(), sampler=smp, allowed=allowed)
    assert outs == [expected(prompts[0], 6), expected(prompts[1], 3), expected(prompts[2], 6)]
    assert asked[:3] == [(0, 5), (1, 9), (2, 13)] and (1, 12) in asked and (1, 13) not in asked
    assert eng.steps[4] == [(0, 1), (2, 1)]                           # request 1 has left the batch
    assert not eng.cache.live_slots and eng.cache.held_pages() == 0
    # without ``allowed`` a sampler of the three-argument form is called as before
    assert generate(TableEngine(64 * 8), prompts, SamplingParams(max_tokens=2), stop_tokens=(), sampler=HostSampler()) \
        == [expected(p, 2) for p in prompts]


# ---- sequences kept for the next call ------------------------------------------------------------
def test_a_kept_sequence_feeds_only_what_is_new():
    from sonicboom_amd.engine.prefix import KeptSequences, common_prefix_len
    assert common_prefix_len([1, 2, 3], [1, 2, 4, 5]) == 2 and common_prefix_len([], [1]) == 0
    eng = TableEngine(64 * 8)
    kept = KeptSequences(eng)
    first = [[3] * 24, [5, 6, 7]]
    outs = generate(eng, first, SamplingParams(max_tokens=4), stop_tokens=(), sampler=HostSampler(), kept=kept)
    assert outs == [expected(p, 4) for p in first] and kept.reused == [0, 0]
    # both sequences stay, with every token that was fed (the last produced one was not)
    assert sorted(len(t) for _, t in kept.items) == [3 + 3, 24 + 3] and len(eng.cache.live_slots) == 2
    eng.steps.clear()
    # the same conversation goes on: 24 tokens + 3 of the 4 produced + 13 new ones
    longer = first[0] + outs[0][:3] + [9] * 13
    other = [8] * 10                                          # starts like nothing that was kept
    outs2 = generate(eng, [other, longer], SamplingParams(max_tokens=5), stop_tokens=(), sampler=HostSampler(), kept=kept)
    assert outs2 == [expected(other, 5), expected(longer, 5)] and kept.reused == [0, 27]
    assert sorted(n for _, n in eng.steps[0]) == [10, 13]     # only the 13 new tokens were fed
    # the sequence no prompt continued was freed at the start; the two new ones are kept now
    assert len(kept) == 2 and len(eng.cache.live_slots) == 2
    # a prompt the session holds in full still feeds its last token; a shorter one cuts the sequence back
    eng.steps.clear()
    again = longer[:20]
    outs3 = generate(eng, [again], SamplingParams(max_tokens=2), stop_tokens=(), sampler=HostSampler(), kept=kept)
    assert outs3 == [expected(again, 2)] and kept.reused == [19] and eng.steps[0] == [(eng.steps[0][0][0], 1)]
    assert len(kept) == 1 and eng.cache.held_pages() == 1
    kept.drop_all()
    assert not eng.cache.live_slots and eng.cache.held_pages() == 0


def test_kept_sequences_never_cost_a_request_its_room():
    """Pages and slots of kept sequences count while earlier batches run; when they leave an
    earlier request no room, the call goes without them."""
    from sonicboom_amd.engine.prefix import KeptSequences
    assert plan_batches([128, 64, 64], 0, 3, 8) == [[0, 1], [2]]
    assert plan_batches([128, 64, 64], 0, 3, 8, held=[0, 0, 1]) == [[0], [1, 2]]     # request 2's page is taken meanwhile
    assert plan_batches([64, 64, 64], 0, 8, 8, max_slots=2, held=[0, 0, 1]) == [[0], [1, 2]]     # and so is its slot
    eng = TableEngine(64 * 4, max_slots=2)
    kept = KeptSequences(eng)
    a, b = [1] * 100, [2] * 100
    generate(eng, [a, b], SamplingParams(max_tokens=2), stop_tokens=(), sampler=HostSampler(), kept=kept)
    assert len(kept) == 2 and eng.cache.held_pages() == 4
    # a request that needs three pages of the four comes first; b's kept sequence would leave it two
    big = [3] * 150
    outs = generate(eng, [big, b + [7]], SamplingParams(max_tokens=2), stop_tokens=(), sampler=HostSampler(), kept=kept)
    assert outs == [expected(big, 2), expected(b + [7], 2)] and kept.reused == [0, 0]
    kept.drop_all()
    assert not eng.cache.live_slots and eng.cache.held_pages() == 0
    # an exception on the way frees what the call held
    generate(eng, [a], SamplingParams(max_tokens=2), stop_tokens=(), sampler=HostSampler(), kept=kept)

    def refuse(i, t):
        raise RuntimeError("stop")
    with pytest.raises(RuntimeError):
        generate(eng, [a + [4]], SamplingParams(max_tokens=2), stop_tokens=(), sampler=HostSampler(), kept=kept,
                 callback=refuse)
    assert not eng.cache.live_slots and eng.cache.held_pages() == 0 and len(kept) == 0


def test_truncate_refuses_what_cannot_be_taken_back():
    from sonicboom_amd.cache import CacheError
    c = PagedCache([GroupSpec(1, 16, 0, (0,)), GroupSpec(1, 16, 100, (1,))], 64 * 16, allocate=False)
    s = c.alloc_slot()
    c.reserve([s], [300])
    c.advance([s], [300])
    assert c.can_truncate(s, 300) and c.can_truncate(s, 292) and not c.can_truncate(s, 290) and not c.can_truncate(s, 301)
    with pytest.raises(CacheError, match="windowed group"):
        c.truncate(s, 100)
    c.reserve([s], [30])
    c.advance([s], [30])
    assert c.held_pages(0) == 6
    c.truncate(s, 292)                         # back over a page's edge: the sixth page goes
    assert c.length(s) == 292 and c.held_pages(0) == 5 and c.held_pages(1) == 2
    c.reserve([s], [60])
    c.advance([s], [60])
    assert c.length(s) == 352
    # a cache whose mixers keep per-sequence state only goes back to where it is
    state = PagedCache([GroupSpec(1, 16, 0, (0,))], 64 * 4, allocate=False)
    import torch
    state.state[0] = torch.zeros((state.max_slots, 3))
    t = state.alloc_slot()
    state.reserve([t], [10])
    state.advance([t], [10])
    assert state.can_truncate(t, 10) and not state.can_truncate(t, 9)
    with pytest.raises(CacheError, match="state"):
        state.truncate(t, 5)

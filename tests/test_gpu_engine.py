"""The engine against the plain implementation, on the GPU, in float32 and bfloat16:
each request alone and whole; with its last 32 tokens one by one; in batches of
unequal lengths whose shorter requests end earlier, batch after batch on a cache
too small to hold them all at once, so that slots and pages are used again."""
import numpy as np
import pytest

from conftest import TINY, random_prompt
from helpers import (assert_logits_close, plain_logits, run_batch, run_tail_one_by_one, run_whole)

pytestmark = pytest.mark.gpu

DTYPES = ["float32", "bfloat16"]
_ENGINES = {}


def engine_for(folder, dtype, max_tokens=64 * 24):
    from sonicboom_amd.engine import DecoderModel, Engine
    key = (folder, dtype, max_tokens)
    if key not in _ENGINES:
        # requests here run past tiny A's 128 positions on purpose: the arithmetic has no such bound
        _ENGINES[key] = Engine(DecoderModel.from_folder(folder, dtype), max_tokens, max_positions=0)
    return _ENGINES[key]


def requests_for(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [random_prompt(rng, TINY[name]["vocab_size"], n) for n in lengths]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_whole_requests(model_folders, name, dtype):
    eng = engine_for(model_folders[name], dtype)
    for tokens in requests_for(name, [1, 5, 33, 64, 65, 130]):
        got = run_whole(eng, tokens)
        assert_logits_close(got, plain_logits(model_folders[name], tokens), dtype, f"{name} whole n={len(tokens)}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_last_32_tokens_one_by_one(model_folders, name, dtype):
    eng = engine_for(model_folders[name], dtype)
    for tokens in requests_for(name, [40, 97, 150], seed=1):
        got = run_tail_one_by_one(eng, tokens)
        assert_logits_close(got, plain_logits(model_folders[name], tokens), dtype, f"{name} tail n={len(tokens)}")
        if dtype == "float32":
            # in 32-bit the cut must not matter by a bit
            assert np.array_equal(got, run_whole(eng, tokens))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_unequal_batches_one_after_another(model_folders, name, dtype):
    folder = model_folders[name]
    # 6 pages of cache: every batch fills most of it, so the next batch gets used pages and slots.
    eng = engine_for(folder, dtype, max_tokens=64 * 6)
    lens = {"A": [(5, 8), (9, 3), (13, 12)], "B": [(1, 12), (7, 2), (20, 9), (33, 5)]}[name]
    for round_ in range(3):
        reqs = requests_for(name, [p + d for p, d in lens], seed=10 + round_)
        got = run_batch(eng, reqs, [p for p, _ in lens])
        for r, (p, _), g in zip(reqs, lens, got):
            want = plain_logits(folder, r)
            assert_logits_close(g[:p], want[:p], dtype, f"{name} batch prompt")
            assert_logits_close(g[p:], want[p:], dtype, f"{name} batch decode")
        assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name, n_req", [("A", 40), ("B", 23)])
def test_many_short_requests_in_one_batch(model_folders, name, n_req, dtype):
    """Dozens of requests in one batch: the decode steps bring 17 to 64 rows, which take other
    product kernels than a handful of rows does.  Prompts of 1 to 9 tokens, 2 to 6 decoded."""
    folder = model_folders[name]
    eng = engine_for(folder, dtype, max_tokens=64 * 48)
    rng = np.random.default_rng(77)
    prompts = [int(n) for n in rng.integers(1, 10, size=n_req)]
    decoded = [int(n) for n in rng.integers(2, 7, size=n_req)]
    reqs = requests_for(name, [p + d for p, d in zip(prompts, decoded)], seed=21)
    got = run_batch(eng, reqs, prompts)
    for i, (r, g) in enumerate(zip(reqs, got)):
        assert_logits_close(g, plain_logits(folder, r), dtype, f"{name} request {i} of {n_req}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("dtype, pages", [("float32", 0), ("bfloat16", 0), ("bfloat16", 2), ("bfloat16", 8)])
def test_large_batch_of_longer_requests(model_folders, dtype, pages):
    """64 requests of 130 to 200 tokens decoded together, through the engine; in bfloat16 also
    with the decode attention kernel's waves taking 2 and 8 pages in a row, as they do when the
    page table is wide."""
    from sonicboom_amd import ops
    folder = model_folders["A"]
    eng = engine_for(folder, dtype, max_tokens=64 * 4 * 64)
    rng = np.random.default_rng(91)
    prompts = [int(n) for n in rng.integers(120, 190, size=64)]
    reqs = requests_for("A", [p + 10 for p in prompts], seed=33)
    head_dim = TINY["A"]["hidden_size"] // TINY["A"]["num_attention_heads"]
    with ops.attention_decode_pages_per_wave(head_dim, pages):
        got = run_batch(eng, reqs, prompts)
    for i, (r, g) in enumerate(zip(reqs, got)):
        assert_logits_close(g, plain_logits(folder, r), dtype, f"request {i}")
    assert eng.cache.held_pages() == 0 and not eng.cache.live_slots


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_float32_logits_do_not_depend_on_cut_batch_slot_or_capacity(model_folders, sharp_folders, name):
    """The 32-bit path bit for bit: a request's logits are the same whole, with its tail one by
    one, inside a batch in any order of the batch, in whatever slot and pages it lands, and with
    a cache of another size (/root/reference/tests/core/test_guarantees.cpp:300-326: determinism,
    capacity independence)."""
    from sonicboom_amd.engine import StepEntry
    for folder in (model_folders[name], sharp_folders[name]):
        eng = engine_for(folder, "float32")
        lens = [(5, 8), (70, 3), (13, 12), (1, 40), (130, 2)]
        reqs = requests_for(name, [p + d for p, d in lens], seed=5)
        prompts = [p for p, _ in lens]
        whole = [run_whole(eng, r) for r in reqs]
        for r, w in zip(reqs, whole):
            assert np.array_equal(run_tail_one_by_one(eng, r), w)
        got = run_batch(eng, reqs, prompts)
        for g, w in zip(got, whole):
            assert np.array_equal(g, w)
        # another order of the batch, while other requests hold the first slots and pages
        held = [eng.alloc_slot() for _ in range(3)]
        eng.step([StepEntry(s, reqs[1][:40 + 30 * i], ()) for i, s in enumerate(held)])
        order = [3, 0, 4, 2, 1]
        got = run_batch(eng, [reqs[i] for i in order], [prompts[i] for i in order])
        for i, g in zip(order, got):
            assert np.array_equal(g, whole[i])
        for s in held:
            eng.free_slot(s)
        # a cache of another size
        small = engine_for(folder, "float32", max_tokens=64 * 9)
        got = run_batch(small, reqs, prompts)
        for g, w in zip(got, whole):
            assert np.array_equal(g, w)
        assert small.cache.held_pages() == 0 and eng.cache.held_pages() == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_sharp_models_whole_tail_and_batches(sharp_folders, name, dtype):
    """The same three cuttings on the models whose attention scores spread over several units:
    here a wrong scale, rope base, bias or position moves the logits by many times the bound."""
    folder = sharp_folders[name]
    eng = engine_for(folder, dtype)
    for tokens in requests_for(name, [1, 33, 65, 150], seed=3):
        want = plain_logits(folder, tokens)
        assert_logits_close(run_whole(eng, tokens), want, dtype, f"sharp {name} whole n={len(tokens)}", sharp=True)
        assert_logits_close(run_tail_one_by_one(eng, tokens), want, dtype, f"sharp {name} tail n={len(tokens)}", sharp=True)
    lens = [(1, 12), (7, 2), (20, 9), (33, 5), (90, 40)]
    small = engine_for(folder, dtype, max_tokens=64 * 8)
    for round_ in range(2):
        reqs = requests_for(name, [p + d for p, d in lens], seed=40 + round_)
        got = run_batch(small, reqs, [p for p, _ in lens])
        for r, g in zip(reqs, got):
            assert_logits_close(g, plain_logits(folder, r), dtype, f"sharp {name} batch", sharp=True)
        assert small.cache.held_pages() == 0 and not small.cache.live_slots


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B"])
def test_steps_above_the_row_limit_run_in_portions(model_folders, sharp_folders, name, dtype):
    """A step of more rows than the engine's limit runs in portions from the cache.  Limits are
    chosen so that portions end inside a request, start with a request's last two tokens, hold a
    single token of one, and leave whole requests out; wanted rows sit at portion starts and ends
    and come back in the order of the entries.  32-bit: the same bits as the step in one piece."""
    from sonicboom_amd.engine import DecoderModel, Engine, StepEntry
    folder = sharp_folders[name]
    lens = [30, 2, 41, 1, 17, 9]
    reqs = requests_for(name, lens, seed=8)
    wants = [list(range(n)) for n in lens]
    wants[2] = [40, 0, 7, 8]                  # not ascending: the order of ``want`` is kept
    wants[4] = []
    model = engine_for(folder, dtype).model
    whole = Engine(model, 64 * 8, max_positions=0)
    slots = [whole.alloc_slot() for _ in reqs]
    ref = whole.step([StepEntry(s, r, w) for s, r, w in zip(slots, reqs, wants)]).cpu().numpy()
    plain = np.concatenate([plain_logits(folder, r)[w] for r, w in zip(reqs, wants) if w])
    assert_logits_close(ref, plain, dtype, "one piece", sharp=True)
    # 8: portion edges inside requests; 31: a portion that starts with the last row of request 0 and
    # holds request 1 whole; 73: request 3 alone ends a portion; 1: every row its own portion
    for limit in (8, 31, 32, 73, 1):
        eng = Engine(model, 64 * 8, max_step_rows=limit, max_positions=0)
        slots = [eng.alloc_slot() for _ in reqs]
        got = eng.step([StepEntry(s, r, w) for s, r, w in zip(slots, reqs, wants)]).cpu().numpy()
        assert [eng.length(s) for s in slots] == lens
        if dtype == "float32":
            assert np.array_equal(got, ref), f"limit {limit}"
        else:
            assert_logits_close(got, plain, dtype, f"limit {limit}", sharp=True)
        # the cache the portions left continues like any other
        nxt = eng.step([StepEntry(slots[2], [5], [0]), StepEntry(slots[3], [6], [0])]).cpu().numpy()
        want_next = np.stack([plain_logits(folder, reqs[2] + [5])[-1], plain_logits(folder, reqs[3] + [6])[-1]])
        assert_logits_close(nxt, want_next, dtype, f"limit {limit}, next step", sharp=True)
        for s in slots:
            eng.free_slot(s)
        assert eng.cache.held_pages() == 0

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
        _ENGINES[key] = Engine(DecoderModel.from_folder(folder, dtype), max_tokens)
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
            # the cut must not matter beyond rounding: compare with the whole run too
            np.testing.assert_allclose(got, run_whole(eng, tokens), atol=2e-6, rtol=1e-5)


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

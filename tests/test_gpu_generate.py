"""Generation through the Python entry point and the command line, on the GPU: greedy tokens
against the plain implementation, seeded sampling, stop tokens, batches, long decoding and
the first tokens of a sequence."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest

from conftest import ROOT, TINY, random_prompt
from helpers import BF16_MAX, BF16_REL, assert_logits_close, plain_logits, plain_model
from plain import qwen2_plain, sampling_plain

pytestmark = pytest.mark.gpu

_MODELS = {}


def model_for(folder, dtype):
    from sonicboom_amd.api import Model
    if (folder, dtype) not in _MODELS:
        _MODELS[(folder, dtype)] = Model.load(folder, dtype=dtype)
    return _MODELS[(folder, dtype)]


def prompts_for(name, lengths, seed=0):
    rng = np.random.default_rng(seed)
    return [random_prompt(rng, TINY[name]["vocab_size"], n) for n in lengths]


def test_greedy_float32_equals_the_plain_implementation(model_folders):
    """Tiny A: 3 prompts of 5/9/13 tokens, 8 greedy steps, as one batch."""
    folder = model_folders["A"]
    cfg, w = plain_model(folder)
    prompts = prompts_for("A", [5, 9, 13])
    session = model_for(folder, "float32").session(max_tokens=64 * 4)
    got = session.generate(prompts, max_tokens=8, stop_tokens=())
    assert got == [qwen2_plain.greedy(cfg, w, p, 8) for p in prompts]
    # each prompt alone gives the same tokens: the batch changes nothing
    assert [session.generate([p], max_tokens=8, stop_tokens=())[0] for p in prompts] == got
    assert not session.engine.cache.live_slots


def test_greedy_bfloat16_follows_the_plain_logits(model_folders):
    """In bfloat16 a near tie may flip: every chosen token must be within a small margin of the
    plain implementation's best logit for the history the engine itself produced."""
    for name in ("A", "B", "C"):
        folder = model_folders[name]
        prompts = prompts_for(name, [3, 17, 40], seed=2)
        session = model_for(folder, "bfloat16").session(max_tokens=64 * 6)
        outs = session.generate(prompts, max_tokens=10, stop_tokens=())
        for p, out in zip(prompts, outs):
            logits = plain_logits(folder, p + out)
            for i, t in enumerate(out):
                row = logits[len(p) - 1 + i]
                # the chosen token's plain logit trails the best by no more than bfloat16 moves two logits
                slack = 2 * (BF16_MAX["tiny"] * float(row.std()) + BF16_REL * float(np.abs(row).max()))
                assert row[t] >= row.max() - slack, (name, i, float(row.max() - row[t]), slack)


def test_temperature_sampling_tiny_b(model_folders):
    """Tiny B: prompts of 1/7/20/33 tokens, 12 steps at temperature 0.8 with a fixed seed."""
    folder = model_folders["B"]
    prompts = prompts_for("B", [1, 7, 20, 33], seed=4)
    session = model_for(folder, "float32").session(max_tokens=64 * 8)
    kw = dict(temperature=0.8, seed=1234, max_tokens=12, stop_tokens=())
    a = session.generate(prompts, **kw)
    assert a == session.generate(prompts, **kw)                                   # same seed, same tokens
    assert a != session.generate(prompts, **{**kw, "seed": 1235})                 # another seed differs
    assert [session.generate([p], **kw)[0] for p in prompts] == a                 # alone or in a batch
    assert all(len(o) == 12 for o in a)
    # the plain sampler over the plain logits draws the same tokens (teacher-forced on the
    # engine's history, so one flipped near-tie would not cascade)
    for p, out in zip(prompts, a):
        logits = plain_logits(folder, p + out)
        for i, t in enumerate(out):
            want = sampling_plain.sample_token(logits[len(p) - 1 + i], len(p) + i, temperature=0.8, seed=1234)
            assert t == want, (len(p), i)


@pytest.mark.parametrize("temperature", [0.0, 0.9])
def test_masks_of_constrained_decoding(model_folders, temperature):
    """A bitmap of allowed ids per request and step: the engine's tokens are the plain sampler's
    under the same masks (after the penalties), a request without a mask is not constrained, and a
    request that may choose nothing ends there."""
    folder = model_folders["A"]
    prompts = prompts_for("A", [6, 11, 9], seed=8)
    session = model_for(folder, "float32").session(max_tokens=64 * 4)
    vocab = session.model.vocab_size
    n_bytes = (vocab + 7) // 8

    def allowed(i, history):
        if i == 1:
            return None                                   # unconstrained
        if i == 2 and len(history) >= len(prompts[2]) + 4:
            return bytes(n_bytes)                         # nothing may follow the fourth token
        rng = np.random.default_rng(1000 * i + len(history))
        bits = rng.integers(0, 256, size=n_bytes if i == 0 else n_bytes // 2, dtype=np.uint8)   # a short bitmap too
        return bytes(bits)

    kw = dict(temperature=temperature, seed=21, top_k=30, repeat_penalty=1.2, presence_penalty=0.1,
              max_tokens=8, stop_tokens=())
    outs = session.generate(prompts, allowed=allowed, **kw)
    assert [len(o) for o in outs] == [8, 8, 4]
    for r, (p, out) in enumerate(zip(prompts, outs)):
        logits = plain_logits(folder, p + out)
        hist = list(p)
        for i, t in enumerate(out):
            mask = allowed(r, hist)
            want = sampling_plain.sample_token(logits[len(p) - 1 + i], len(p) + i, temperature=temperature, seed=21,
                                               top_k=30, repeat_penalty=1.2, presence_penalty=0.1, history=hist,
                                               mask=mask)
            assert t == want, (r, i)
            if mask:
                assert (mask[t >> 3] >> (t & 7)) & 1
            hist.append(t)
    # alone or in the batch, the same tokens
    assert [session.generate([p], allowed=lambda i, h, r=r: allowed(r, h), **kw)[0] for r, p in enumerate(prompts)] == outs


def test_sampling_filters_and_penalties_run_on_the_device(model_folders):
    folder = model_folders["A"]
    prompts = prompts_for("A", [6, 11], seed=5)
    session = model_for(folder, "float32").session(max_tokens=64 * 4)
    kw = dict(temperature=1.1, seed=9, top_k=12, top_p=0.9, min_p=0.02, repeat_penalty=1.3, repeat_last_n=8,
              presence_penalty=0.1, frequency_penalty=0.05, max_tokens=10, stop_tokens=())
    outs = session.generate(prompts, **kw)
    for p, out in zip(prompts, outs):
        logits = plain_logits(folder, p + out)
        hist = list(p)
        for i, t in enumerate(out):
            want = sampling_plain.sample_token(
                logits[len(p) - 1 + i], len(p) + i, temperature=1.1, seed=9, top_k=12, top_p=0.9, min_p=0.02,
                repeat_penalty=1.3, repeat_last_n=8, presence_penalty=0.1, frequency_penalty=0.05, history=hist)
            assert t == want, (len(p), i)
            hist.append(t)
    # greedy with penalties takes the other arithmetic path
    g = session.generate(prompts, repeat_penalty=1.5, presence_penalty=0.3, max_tokens=6, stop_tokens=())
    for p, out in zip(prompts, g):
        logits = plain_logits(folder, p + out)
        hist = list(p)
        for i, t in enumerate(out):
            assert t == sampling_plain.sample_token(logits[len(p) - 1 + i], 0, repeat_penalty=1.5,
                                                    presence_penalty=0.3, history=hist)
            hist.append(t)


def test_stop_tokens_and_batches_on_a_small_cache(model_folders):
    folder = model_folders["B"]                      # its config.json names eos 7
    cfg, w = plain_model(folder)
    prompts = prompts_for("B", [4, 9, 2, 30, 12, 5, 21], seed=6)
    free = [qwen2_plain.greedy(cfg, w, p, 9) for p in prompts]
    session = model_for(folder, "float32").session(max_tokens=64 * 3, max_slots=3)
    assert model_for(folder, "float32").eos == (7,)
    # a stop token that some sequence produces early
    stop = free[3][2]
    want = [qwen2_plain.greedy(cfg, w, p, 9, stop=(stop,)) for p in prompts]
    assert any(len(o) < 9 for o in want)
    got = session.generate(prompts, max_tokens=9, stop_tokens=(stop,), max_batch=3)
    assert got == want
    assert not session.engine.cache.live_slots and session.engine.cache.held_pages() == 0


def test_graph_replay_gives_the_same_tokens(model_folders):
    folder = model_folders["C"]
    prompts = prompts_for("C", [5, 61, 20], seed=7)
    model = model_for(folder, "bfloat16")
    with_graph = model.session(max_tokens=64 * 12)
    without = model.session(max_tokens=64 * 12)
    without.engine.use_graphs = False
    a = with_graph.generate(prompts, max_tokens=150, stop_tokens=())     # crosses pages, replays many times
    b = without.generate(prompts, max_tokens=150, stop_tokens=())
    assert a == b and all(len(o) == 150 for o in a)
    assert with_graph.engine.decode_loop()._graphs, "the decode loop never captured a graph"
    s = with_graph.generate(prompts, temperature=0.7, seed=3, max_tokens=40, stop_tokens=())
    assert s == without.generate(prompts, temperature=0.7, seed=3, max_tokens=40, stop_tokens=())


def test_the_collector_stays_out_of_graph_captures(model_folders):
    """While a decode step is being recorded Python's garbage collector is switched off (what it
    finalizes may call into the HIP runtime, which a capturing stream refuses), and it has run
    just before; afterwards it is on again."""
    import gc
    import torch
    folder = model_folders["A"]
    session = model_for(folder, "bfloat16").session(max_tokens=64 * 4)
    eng = session.engine
    seen = []
    forward = eng.forward

    def watched(ctx):
        if torch.cuda.is_current_stream_capturing():
            seen.append(gc.isenabled())
        return forward(ctx)
    eng.forward = watched
    try:
        assert gc.isenabled()
        session.generate(prompts_for("A", [5, 11], seed=2), max_tokens=8, stop_tokens=())
    finally:
        eng.forward = forward
    assert seen and not any(seen)            # at least one step was recorded, none with the collector on
    assert gc.isenabled()


def test_batches_run_in_buckets_with_rows_that_do_nothing(model_folders):
    """The decode loop runs a batch of more than eight sequences at the next bucket's size (12,
    16, 24, ...): the rows it adds have no pages, store nothing and see no key.  A batch of 21
    whose sequences end one by one must give every sequence the tokens it gets alone, pass
    through a handful of recorded shapes, not one per size, and leave the cache empty."""
    from sonicboom_amd.engine.decode import batch_bucket
    assert [batch_bucket(n) for n in (1, 7, 8, 9, 12, 13, 17, 24, 25, 33, 64, 65, 100)] == \
        [1, 7, 8, 12, 12, 16, 24, 24, 32, 48, 64, 96, 128]
    folder = model_folders["B"]
    model = model_for(folder, "float32")
    prompts = prompts_for("B", [3 + (7 * i) % 40 for i in range(21)], seed=31)
    session = model.session(max_tokens=64 * 64)
    lone = model.session(max_tokens=64 * 4)
    lone.engine.use_graphs = False
    # every sequence stops at its own length: the batch shrinks by one again and again
    counts = [4 + i for i in range(21)]
    want = [lone.generate([p], max_tokens=n, stop_tokens=())[0] for p, n in zip(prompts, counts)]
    ends = {}

    def cut(i, t):
        ends[i] = ends.get(i, 0) + 1
        return ends[i] > counts[i]
    got = session.generate(prompts, max_tokens=40, stop_tokens=(), callback=cut)
    assert got == want
    shapes = sorted({k[0] for k in session.engine.decode_loop()._graphs})
    assert shapes and set(shapes) <= {1, 2, 3, 4, 5, 6, 7, 8, 12, 16, 24}, shapes
    assert not session.engine.cache.live_slots and session.engine.cache.held_pages() == 0
    # sampled, in bfloat16, graph against kernel by kernel: the same tokens with added rows in the batch
    model16 = model_for(folder, "bfloat16")
    a, b = model16.session(max_tokens=64 * 64), model16.session(max_tokens=64 * 64)
    b.engine.use_graphs = False
    ta = a.generate(prompts[:11], temperature=0.9, seed=5, max_tokens=12, stop_tokens=())
    tb = b.generate(prompts[:11], temperature=0.9, seed=5, max_tokens=12, stop_tokens=())
    assert ta == tb


def test_graph_replay_when_the_page_table_grows(tmp_path):
    """Decoding across 1,024 tokens: the decode loop's buffers are keyed by the page table's
    width (steps of 16 pages), so the step is recorded a second time there; tokens with and
    without graphs agree, and the logits on both sides of the edge are the plain ones."""
    from sonicboom_amd.api import Model
    from sonicboom_amd.engine import StepEntry
    from sonicboom_amd.weights import write_random_model
    cfg = dict(TINY["A"], max_position_embeddings=2048)
    folder = str(tmp_path / "long_a")
    write_random_model(folder, cfg, seed=77, dtype="bfloat16")
    model = Model.load(folder, dtype="bfloat16")
    rng = np.random.default_rng(12)
    prompts = [random_prompt(rng, cfg["vocab_size"], n) for n in (1000, 30)]
    with_graph = model.session(max_tokens=64 * 24)
    without = model.session(max_tokens=64 * 24)
    without.engine.use_graphs = False
    a = with_graph.generate(prompts, max_tokens=60, stop_tokens=())
    b = without.generate(prompts, max_tokens=60, stop_tokens=())
    assert a == b and all(len(o) == 60 for o in a)
    widths = sorted(k[1] for k in with_graph.engine.decode_loop()._graphs)
    assert widths == [16, 32], f"graphs recorded for table widths {widths}"
    # the produced tokens, fed back whole: logits around position 1,024 against the plain model
    whole = prompts[0] + a[0]
    eng = without.engine
    s = eng.alloc_slot()
    got = eng.step([StepEntry(s, whole, range(1000, len(whole)))]).cpu().numpy()
    eng.free_slot(s)
    assert_logits_close(got, plain_logits(folder, whole)[1000:], "bfloat16", "around the edge of the table")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_token_by_token_from_the_first_token(model_folders, dtype):
    """A sequence fed one token at a time from its very first token, over several pages,
    together with a second sequence that starts from a prompt: logits at every position."""
    from sonicboom_amd.engine import StepEntry
    folder = model_folders["B"]
    a, b = prompts_for("B", [260, 200], seed=8)
    # 260 tokens: past tiny B's 256 positions on purpose
    eng = model_for(folder, dtype).session(max_tokens=64 * 10, max_positions=0).engine
    sa, sb = eng.alloc_slot(), eng.alloc_slot()
    got_a, got_b = [], []
    out = eng.step([StepEntry(sa, a[:1], [0]), StepEntry(sb, b[:70], range(70))]).cpu().numpy()
    got_a.append(out[:1])
    got_b.append(out[1:])
    for i in range(1, 260):
        entries = [StepEntry(sa, [a[i]], [0])]
        if 70 + i - 1 < 200:
            entries.append(StepEntry(sb, [b[70 + i - 1]], [0]))
        out = eng.step(entries).cpu().numpy()
        got_a.append(out[:1])
        if len(entries) == 2:
            got_b.append(out[1:])
    eng.free_slot(sa)
    eng.free_slot(sb)
    assert_logits_close(np.concatenate(got_a), plain_logits(folder, a), dtype, "token by token from position 0")
    assert_logits_close(np.concatenate(got_b), plain_logits(folder, b), dtype, "prompt of 70, then token by token")


def test_step_errors(model_folders):
    from sonicboom_amd.engine import StepEntry, StepError
    eng = model_for(model_folders["A"], "float32").session(max_tokens=64 * 2).engine
    s = eng.alloc_slot()
    with pytest.raises(StepError, match="outside the vocabulary"):
        eng.step([StepEntry(s, [256], [0])])
    with pytest.raises(StepError, match="at least one token"):
        eng.step([StepEntry(s, [], [])])
    with pytest.raises(StepError, match="wanted row"):
        eng.step([StepEntry(s, [1, 2], [2])])
    with pytest.raises(StepError, match="not in use"):
        eng.step([StepEntry(99, [1], [0])])
    with pytest.raises(StepError, match="out of cache pages"):
        eng.step([StepEntry(s, [1] * 70, [0]), StepEntry(eng.alloc_slot(), [1] * 70, [0])])
    assert eng.step([StepEntry(s, [1, 2, 3], [])]).shape == (0, 256)     # nothing wanted
    assert eng.length(s) == 3
    eng.free_slot(s)
    # the model's own bound on positions (tiny A: 128), unless the session lifts it
    eng = model_for(model_folders["A"], "float32").session(max_tokens=64 * 4).engine
    s = eng.alloc_slot()
    eng.step([StepEntry(s, [1] * 127, [])])
    eng.step([StepEntry(s, [1], [])])
    with pytest.raises(StepError, match="128 positions"):
        eng.step([StepEntry(s, [1], [0])])
    loop = eng.decode_loop()
    loop.start([s], [1])
    with pytest.raises(StepError, match="128 positions"):
        loop.step()
    assert eng.length(s) == 128
    eng.free_slot(s)


def test_generation_ends_at_the_bound_on_positions(model_folders):
    session = model_for(model_folders["A"], "float32").session(max_tokens=64 * 4)
    prompts = prompts_for("A", [120, 10], seed=4)
    out = session.generate(prompts, max_tokens=20, stop_tokens=())
    assert [len(o) for o in out] == [9, 20]          # 120 + 9 = 129 tokens: the last one is never fed
    free = model_for(model_folders["A"], "float32").session(max_tokens=64 * 4, max_positions=0)
    longer = free.generate(prompts, max_tokens=20, stop_tokens=())
    assert longer[0][:9] == out[0] and len(longer[0]) == 20
    with pytest.raises(ValueError, match="128 positions"):
        session.generate([[1] * 129], max_tokens=2)


def test_command_line(model_folders, tmp_path):
    folder = model_folders["A"]
    cfg, w = plain_model(folder)
    prompts = prompts_for("A", [4, 10], seed=9)
    tokens = tmp_path / "prompts.txt"
    tokens.write_text("\n".join(" ".join(map(str, p)) for p in prompts) + "\n")
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "-m", folder, "--tokens", str(tokens), "-n", "6",
           "--dtype", "fp32", "--stop", ""]
    out = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    got = [[int(t) for t in line.split()] for line in out.stdout.strip().splitlines()]
    assert got == [qwen2_plain.greedy(cfg, w, p, 6) for p in prompts]
    # random weights from a configuration file, sampled
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(TINY["B"]))
    cmd = [sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "--random", str(cfg_file), "--seed", "3",
           "--tokens", str(tokens), "-n", "5", "--temperature", "0.8", "--sample-seed", "11", "--top-k", "20"]
    one = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    two = subprocess.run(cmd, capture_output=True, text=True, timeout=300)
    assert one.returncode == 0 and one.stdout == two.stdout and len(one.stdout.split()) <= 10
    bad = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "sb-gen"), "--tokens", str(tokens)],
                         capture_output=True, text=True, timeout=60)
    assert bad.returncode == 2 and "usage" in bad.stderr


def test_prefix_reuse_gives_the_bits_of_the_whole_prompt(model_folders):
    """A conversation that goes on: 24 tokens, 16 more on the kept sequence, against the 40 fed
    whole (/root/reference/tests/core/test_guarantees.cpp:300-326): in 32-bit the same logits to
    the bit and the same tokens, greedy and drawn; only the new tokens are fed."""
    import torch
    from sonicboom_amd.api import Model
    from sonicboom_amd.engine import StepEntry
    model = Model.load(model_folders["B"], dtype="float32")
    rng = np.random.default_rng(21)
    head, more = random_prompt(rng, 384, 24), random_prompt(rng, 384, 16)
    other = random_prompt(rng, 384, 30)
    for sampling in (dict(), dict(temperature=0.9, seed=5, top_p=0.95)):
        whole = model.session(64 * 8)
        want = whole.generate([head + more, other], max_tokens=12, stop_tokens=[], **sampling)
        ses = model.session(64 * 8)
        fed = []
        step = ses.engine.step
        ses.engine.step = lambda entries: (fed.append([len(e.tokens) for e in entries]), step(entries))[1]
        first = ses.generate([head], max_tokens=3, stop_tokens=[], keep=True, **sampling)[0]
        assert ses.reused == [0] and len(ses.kept) == 1
        fed.clear()
        got = ses.generate([other, head + more], max_tokens=12, stop_tokens=[], keep=True, **sampling)
        # the kept sequence holds the 24 tokens and two of the three produced; the new prompt shares the 24
        assert ses.reused == [0, 24] and fed[0] == [30, 16]
        assert got == [want[1], want[0]]
        assert len(ses.kept) == 2
        ses.forget()
        assert not ses.engine.cache.live_slots and ses.engine.cache.held_pages() == 0
    # the logits themselves: 24 + 16 on the same slot against 40 at once
    eng = model.session(64 * 4).engine
    a, b = eng.alloc_slot(), eng.alloc_slot()
    eng.step([StepEntry(a, head + random_prompt(rng, 384, 9), ())])        # a sequence that went elsewhere
    eng.cache.truncate(a, 24)                                              # back to the shared prefix
    cut = eng.step([StepEntry(a, more, range(16))])
    full = eng.step([StepEntry(b, head + more, range(24, 40))])
    assert torch.equal(cut, full)


def test_prefix_reuse_in_bfloat16_stays_within_the_bounds(model_folders):
    from helpers import assert_logits_close, plain_logits
    from sonicboom_amd.api import Model
    from sonicboom_amd.engine import StepEntry
    folder = model_folders["A"]
    eng = Model.load(folder, dtype="bfloat16").session(64 * 8).engine
    rng = np.random.default_rng(3)
    head, more = random_prompt(rng, 256, 70), random_prompt(rng, 256, 30)
    s = eng.alloc_slot()
    eng.step([StepEntry(s, head + random_prompt(rng, 256, 20), ())])
    eng.cache.truncate(s, 70)
    got = eng.step([StepEntry(s, more, range(30))]).cpu().numpy()
    assert_logits_close(got, plain_logits(folder, head + more)[70:], "bfloat16", "on a sequence taken back")

"""Sampling on the host: the plain sampler against the reference's test vectors, and the
product's host stages (filters, Philox, Gumbel draw) against the plain sampler."""

import numpy as np
import pytest

from plain import sampling_plain as SP
from sonicboom_amd.sampling import (SamplingParams, draw_rows, filter_candidates, gumbel_draw, penalty_items,
                                    philox4x32_10)

F32 = np.float32


def test_philox_known_answer():
    """/root/reference/tests/core/test_sampling.cpp:42-49 (Random123, zero counter and key)."""
    want = [0x6627E8D5, 0xE169C58D, 0xBC57AC4C, 0x9B00DBD8]
    assert SP.philox4x32_10([0, 0, 0, 0], 0) == want
    assert [int(w) for w in philox4x32_10(0, 0, 0, 0, 0)] == want
    # the vectorised form agrees with the plain one on other counters and a 64-bit key
    key = 0x0123456789ABCDEF
    ids = np.array([0, 1, 77, 152063], dtype=np.uint64)
    got = philox4x32_10(12345, 6, ids, 0, key)
    for i, t in enumerate(ids):
        assert [int(w[i]) for w in got] == SP.philox4x32_10([12345, 6, int(t), 0], key)


def test_greedy_and_top_k_one():
    """test_sampling.cpp:51-69."""
    assert SP.sample_token(np.array([0.2, 0.2, 0.9, 0.1], F32), 0) == 2
    assert SP.sample_token(np.array([0.5, 0.5, 0.1], F32), 0) == 0
    logits = np.array([0.5, 2.5, 1.5, -1.0], F32)
    for pos in range(32):
        assert SP.sample_token(logits, pos, temperature=1.0, top_k=1) == 1


def test_filter_sets():
    """test_sampling.cpp:71-117: top-k, min-p and nucleus surviving sets."""
    assert SP.surviving_ids(np.array([3, 2, 1, 0], F32), 1.0, top_k=2) == [0, 1]
    assert SP.surviving_ids(np.zeros(4, F32), 1.0, top_k=2) == [0, 1]                 # ties by id
    z = np.array([0.0, -1.0, -3.0], F32)
    assert SP.surviving_ids(z, 1.0, min_p=0.1) == [0, 1]                              # ln 0.1 = -2.30
    assert SP.surviving_ids(z, 1.0, min_p=0.5) == [0]
    four = np.zeros(4, F32)
    assert SP.surviving_ids(four, 1.0, top_p=0.6) == [0, 1, 2]
    assert SP.surviving_ids(four, 1.0, top_p=0.5) == [0, 1]
    assert SP.surviving_ids(four, 1.0, top_p=0.24) == [0]
    # the window of 30 below the best z
    assert SP.surviving_ids(np.array([0.0, -29.0, -31.0], F32), 1.0) == [0, 1]
    assert SP.surviving_ids(np.array([0.0, -29.0, -31.0], F32), 0.5) == [0]          # z = l / T


def test_penalties():
    """test_sampling.cpp:119-169."""
    assert SP.sample_token(np.array([1.5, 1.0], F32), 0, repeat_penalty=2.0, history=[0]) == 1
    assert SP.sample_token(np.array([-0.5, -0.8], F32), 0, repeat_penalty=2.0, history=[0]) == 1
    assert SP.sample_token(np.array([1.0, 0.9], F32), 0, presence_penalty=0.2, history=[0]) == 1
    assert SP.sample_token(np.array([1.0, 0.9], F32), 0, frequency_penalty=0.04, history=[0, 0, 0]) == 1
    # outside the window of repeat_last_n nothing is penalised
    assert SP.sample_token(np.array([1.0, 0.9], F32), 0, presence_penalty=0.2, repeat_last_n=2,
                           history=[0, 1, 1]) == 0
    assert penalty_items([[1, 2, 2, 49], [], [7] * 10], 64, 50) == ([0, 0, 0, 2], [1, 2, 49, 7], [1, 2, 1, 10])
    assert penalty_items([[1, 2, 3]], 2, 50) == ([0, 0], [2, 3], [1, 1])
    assert penalty_items([[1, 99]], 64, 50) == ([0], [1], [1])


def test_candidate_cap_and_order():
    """test_sampling.cpp:171-258: 256 candidates, (z descending, id ascending), z = l / T."""
    r = np.random.default_rng(0)
    logits = r.standard_normal(1000).astype(F32)
    logits[10] = logits[500] = 9.0
    c = SP.select_candidates(logits, 0.7)
    assert len(c) == 256 and c[0][0] == 10 and c[1][0] == 500
    assert all((a[1] > b[1]) or (a[1] == b[1] and a[0] < b[0]) for a, b in zip(c, c[1:]))
    assert all(z == F32(logits[i] / F32(0.7)) for i, z in c)


def test_seed_and_position_fix_the_draw():
    """test_sampling.cpp:260-281."""
    logits = np.random.default_rng(1).standard_normal(64).astype(F32)
    a = [SP.sample_token(logits, p, temperature=1.0, seed=7) for p in range(64)]
    assert a == [SP.sample_token(logits, p, temperature=1.0, seed=7) for p in range(64)]
    assert a != [SP.sample_token(logits, p, temperature=1.0, seed=8) for p in range(64)]
    assert len(set(a)) > 8


def test_draws_follow_the_softmax():
    """test_sampling.cpp:283-313 with fewer draws: chi-square of the draw counts against the softmax."""
    logits = np.array([1.0, 0.5, 0.0, -0.5, -1.0], F32)
    cands = SP.select_candidates(logits, 1.0)
    n = 20000
    counts = np.zeros(5)
    for pos in range(n):
        counts[SP.draw(cands, 99, pos)] += 1
    p = np.exp(logits.astype(np.float64))
    p /= p.sum()
    chi2 = (((counts - n * p) ** 2) / (n * p)).sum()
    assert chi2 < 18.47                       # 4 degrees of freedom, p = 0.001


@pytest.mark.parametrize("params", [
    dict(temperature=0.8), dict(temperature=1.3, top_k=5), dict(temperature=0.5, top_p=0.7),
    dict(temperature=1.0, min_p=0.2), dict(temperature=0.9, top_k=40, top_p=0.9, min_p=0.01),
])
def test_product_host_stages_equal_the_plain_sampler(params):
    r = np.random.default_rng(5)
    for trial in range(20):
        logits = (r.standard_normal(400) * 3).astype(F32)
        cands = SP.select_candidates(logits, params["temperature"])
        ids = np.array([c[0] for c in cands], dtype=np.int32)
        z = np.array([c[1] for c in cands], dtype=np.float32)
        sp = SamplingParams(seed=trial, **params)
        kept_ids, kept_z = filter_candidates(ids, z, sp)
        want = SP.filter_candidates(cands, params.get("top_k", 0), params.get("top_p", 1.0), params.get("min_p", 0.0))
        assert kept_ids.tolist() == [c[0] for c in want]
        for pos in (0, 17, 2 ** 33 + 5):
            assert gumbel_draw(kept_ids, kept_z, trial, pos) == SP.draw(want, trial, pos)


@pytest.mark.parametrize("params", [
    dict(temperature=0.8), dict(temperature=1.3, top_k=5), dict(temperature=0.5, top_p=0.7),
    dict(temperature=1.0, min_p=0.2), dict(temperature=0.9, top_k=40, top_p=0.9, min_p=0.01),
    dict(temperature=0.05, top_p=0.5), dict(temperature=2.0, top_k=1), dict(temperature=1.0, top_p=1e-9, min_p=1.0),
])
def test_all_rows_at_once_equal_the_plain_sampler_row_by_row(params):
    """A step's rows filtered and drawn together: every row gets the token the plain sampler
    gives it alone, whatever the other rows hold (flat and peaked rows, ties, far positions)."""
    r = np.random.default_rng(11)
    rows = []
    for i in range(24):
        logits = (r.standard_normal(400) * (0.2 if i % 5 == 0 else 3.0)).astype(F32)
        if i % 7 == 3:
            logits[10:20] = logits[5]                    # ties among the best
        if i % 6 == 1:
            logits[3] = 80.0                             # one candidate far above the window
        rows.append(logits)
    cands = [SP.select_candidates(l, params["temperature"]) for l in rows]
    ids = np.array([[c[0] for c in cs] for cs in cands], dtype=np.int32)
    z = np.array([[c[1] for c in cs] for cs in cands], dtype=np.float32)
    positions = [int(q) for q in r.integers(0, 5000, size=len(rows))]
    positions[0], positions[1] = 0, 2 ** 33 + 5
    sp = SamplingParams(seed=77, **params)
    got = draw_rows(ids, z, positions, sp)
    for i, cs in enumerate(cands):
        kept = SP.filter_candidates(cs, params.get("top_k", 0), params.get("top_p", 1.0), params.get("min_p", 0.0))
        assert got[i] == SP.draw(kept, 77, positions[i]), f"row {i}"
        one = draw_rows(ids[i:i + 1], z[i:i + 1], positions[i:i + 1], sp)
        assert one == [got[i]]


def test_mask_of_constrained_decoding():
    """The plain sampler's mask (/root/reference/core/src/nn/sampling.cpp:266-274, :334-339): bit i & 7
    of byte i >> 3 allows id i, an id past the bitmap is not allowed, an empty mask allows all."""
    logits = np.array([0.1, 5.0, 0.3, 4.0, -1.0, 4.5, 0.0, 0.2, 9.0, 3.0], dtype=F32)
    only = lambda *ids: bytes(sum(1 << (i & 7) for i in ids if i >> 3 == b) for b in range(2))  # noqa: E731
    assert SP.sample_token(logits, 0) == 8 and SP.sample_token(logits, 0, mask=b"") == 8
    assert SP.sample_token(logits, 0, mask=only(3, 5, 9)) == 5           # the best of the allowed
    assert SP.sample_token(logits, 0, mask=only(3, 5, 9)[:1]) == 5       # a bitmap of one byte: ids 0..7
    assert SP.sample_token(logits, 0, mask=bytes([0xFF])) == 1           # 8 and 9 lie past it
    assert SP.sample_token(logits, 0, mask=bytes(2)) == -1               # nothing allowed
    assert SP.sample_token(logits, 0, temperature=0.7, seed=3, mask=bytes(2)) == -1
    # penalties come first: the penalised best of the allowed loses to the next one
    assert SP.sample_token(logits, 3, mask=only(3, 5), history=[5, 5, 5], frequency_penalty=1.0) == 3
    # sampled: only allowed ids are ever drawn, every allowed id within the window is drawn sometimes
    mask = only(0, 3, 5, 9)
    drawn = {SP.sample_token(logits, pos, temperature=1.5, seed=11, mask=mask) for pos in range(300)}
    assert drawn == {0, 3, 5, 9}
    cands = SP.select_candidates(logits, 1.5, mask=mask)
    assert [c[0] for c in cands] == [5, 3, 9, 0]
    # an allowed id is drawn as it would be from the same candidates without a mask
    sub = np.full(10, -np.inf, dtype=F32)
    sub[[0, 3, 5, 9]] = logits[[0, 3, 5, 9]]
    for pos in range(50):
        assert SP.sample_token(logits, pos, temperature=1.5, seed=11, mask=mask) == \
            SP.sample_token(sub, pos, temperature=1.5, seed=11)


def test_params_validation():
    assert SamplingParams(repeat_penalty=0.0).validated().repeat_penalty == 1.0
    assert not SamplingParams().has_penalties and SamplingParams(presence_penalty=0.1).has_penalties
    assert not SamplingParams(presence_penalty=0.1, repeat_last_n=0).has_penalties
    for bad in (dict(temperature=-1.0), dict(top_p=1.5), dict(min_p=-0.1), dict(top_k=-1), dict(repeat_penalty=-2.0),
                dict(seed=2 ** 64)):
        with pytest.raises(ValueError):
            SamplingParams(**bad).validated()


def test_how_close_a_draw_comes_to_a_tie():
    """The winner of a draw is the largest z + g in float64, and g = -ln(-ln u) comes from the
    math library at hand: the device's on the GPU, the host's in the plain sampler and the host
    twins, which may differ in the last bit.  A last bit only matters where the two best scores are
    that close.  Over 40,000 draws of 256 candidates each (a vectorised copy of the plain draw,
    held to it on a sample), the smallest gap between the best and the second score is counted in
    units of the last bit of the best: it stays above a million such units, so a math library
    that is off by a few of them names the same token; equal bits of device and host draws are
    then a matter of these margins, not of equal libraries."""
    from sonicboom_amd.sampling.philox import philox4x32_10 as philox_many
    rng = np.random.default_rng(17)
    n_draws, k = 40000, 256
    ids = np.stack([rng.choice(152064, size=k, replace=False) for _ in range(200)])      # 200 candidate sets
    z = np.sort(rng.standard_normal((200, k)).astype(np.float32) * 3.0, axis=1)[:, ::-1]
    smallest = np.inf
    for seed in (0, 7, 2 ** 40 + 3):
        for start in range(0, n_draws // 3, 200):
            pos = np.arange(start, start + 200, dtype=np.uint64)[:, None] + np.uint64(1000)
            w = philox_many(pos & np.uint64(0xFFFFFFFF), pos >> np.uint64(32), ids.astype(np.uint64), np.uint64(0), seed)[0]
            u = (w.astype(np.float64) + 0.5) / 4294967296.0
            score = z.astype(np.float64) - np.log(-np.log(u))
            top = np.sort(score, axis=1)
            gap = (top[:, -1] - top[:, -2]) / np.spacing(np.abs(top[:, -1]))
            smallest = min(smallest, float(gap.min()))
            if start == 0:       # the vectorised draw is the plain sampler's
                for row in (0, 57, 199):
                    cands = [(int(i), np.float32(v)) for i, v in zip(ids[row], z[row])]
                    assert SP.draw(cands, seed, int(pos[row, 0])) == int(ids[row][np.argmax(score[row])])
    assert smallest > 1e6, f"two scores within {smallest:.3g} units of the last bit"

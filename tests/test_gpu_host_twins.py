"""Every kernel against its plain C++ twin on host memory (sonicboom_amd/csrc/plain_host.cpp),
at sizes other than the engine's.  The twins themselves are pinned, without a GPU, by the
reference's vectors and by the NumPy implementation (test_host_twins_agree_with_the_plain_implementation)."""
import ctypes
import math

import numpy as np
import pytest
import torch

from plain import qwen2_plain as P
from plain import sampling_plain as SP
from sonicboom_amd.cache import layout

F32, BF16 = torch.float32, torch.bfloat16
DEV = "cuda:0"


def twins():
    from sonicboom_amd.csrc import build
    lib = ctypes.CDLL(build.ensure_plain_host())
    for name in ("sbp_embed", "sbp_rmsnorm", "sbp_reduce_resid_norm", "sbp_gemm", "sbp_silu_mul", "sbp_add_into",
                 "sbp_rope_kv_store", "sbp_attention", "sbp_argmax", "sbp_penalize", "sbp_mask_logits",
                 "sbp_top_candidates", "sbp_draw"):
        getattr(lib, name).restype = ctypes.c_int
    return lib


def ptr(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def f32(*shape, seed=0, scale=1.0):
    return (np.random.default_rng(seed).standard_normal(shape) * scale).astype(np.float32)


def i32(values):
    return np.ascontiguousarray(values, dtype=np.int32)


C = ctypes.c_int


def host_gemm(lib, x, w, bias=None, resid=None):
    y = np.empty((x.shape[0], w.shape[0]), np.float32)
    assert lib.sbp_gemm(ptr(y), ptr(x), ptr(w), ptr(bias), ptr(resid), C(x.shape[0]), C(w.shape[0]), C(x.shape[1])) == 0
    return y


def host_rmsnorm(lib, x, w, eps, rows=None):
    n = x.shape[0] if rows is None else len(rows)
    y = np.empty((n, x.shape[1]), np.float32)
    assert lib.sbp_rmsnorm(ptr(y), ptr(x), ptr(w), ptr(rows), C(n), C(x.shape[1]), ctypes.c_float(eps)) == 0
    return y


def host_paged(lib, qkv, bias, inv_freq, ff, rot, pos, seq, table, n_pages, hq, hkv, hd):
    """(q, k_cache, v_cache) of the rotate-and-store twin on empty caches."""
    n = qkv.shape[0]
    q = np.empty((n, hq * hd), np.float32)
    kc = np.zeros((n_pages, hkv, 64, hd), np.float32)
    vc = np.zeros((n_pages, hkv, hd, 64), np.float32)
    assert lib.sbp_rope_kv_store(ptr(q), ptr(qkv), C(qkv.shape[1]), ptr(bias), ptr(inv_freq), ptr(ff), C(rot),
                                 ptr(pos), ptr(seq), ptr(kc), ptr(vc), ptr(table), C(table.shape[1]), C(n_pages),
                                 C(n), C(hq), C(hkv), C(hd)) == 0
    return q, kc, vc


def host_attention(lib, q, kc, vc, table, pos, seq, hq, hkv, hd, scale, window):
    out = np.empty((q.shape[0], hq * hd), np.float32)
    assert lib.sbp_attention(ptr(out), ptr(q), C(q.shape[1]), ptr(kc), ptr(vc), ptr(table), C(table.shape[1]),
                             C(kc.shape[0]), ptr(pos), ptr(seq), C(q.shape[0]), C(hq), C(hkv), C(hd),
                             ctypes.c_float(scale), C(window)) == 0
    return out


# ---- the twins themselves, without a GPU -------------------------------------------------------
def test_host_twins_agree_with_the_plain_implementation():
    lib = twins()
    # norm: the reference's vectors (/root/reference/tests/core/test_nn.cpp:172-219), then NumPy
    assert np.allclose(host_rmsnorm(lib, np.full((1, 4), 2, np.float32), None, 0.0), 1.0, atol=1e-6)
    assert np.array_equal(host_rmsnorm(lib, np.array([[1, 0, 0, 0]], np.float32), None, 0.75), [[1, 0, 0, 0]])
    x, w = f32(5, 201, seed=1, scale=3.0), f32(201, seed=2)
    assert np.allclose(host_rmsnorm(lib, x, w, 1e-5), P.rms_norm(x, w, 1e-5), atol=1e-6)
    assert np.array_equal(host_rmsnorm(lib, x, w, 1e-5, i32([4, 0])), host_rmsnorm(lib, x, w, 1e-5)[[4, 0]])
    # product, bias, residual
    x, w, b, r = f32(7, 50, seed=3), f32(13, 50, seed=4), f32(13, seed=5), f32(7, 13, seed=6)
    assert np.allclose(host_gemm(lib, x, w, b, r), P.linear(x, w, b) + r, atol=1e-5)
    # silu * up
    gu = f32(3, 24, seed=7, scale=3.0)
    out = np.empty((3, 12), np.float32)
    assert lib.sbp_silu_mul(ptr(out), ptr(gu), C(3), C(12)) == 0
    assert np.allclose(out, P.silu(gu[:, :12]) * gu[:, 12:], atol=1e-6)
    # rotation (pairs (i, i + half): the vector of test_nn.cpp:221-290), store, attention
    hq, hkv, hd = 4, 2, 8
    inv = np.exp(-2.0 * np.arange(hd // 2, dtype=np.float32) / hd * np.log(np.float32(1e4))).astype(np.float32)
    pos, seq = i32([0, 1, 2, 70, 0]), i32([0, 0, 0, 1, 1])
    table = i32([[2, 5], [1, 0]])
    qkv, bias = f32(5, (hq + 2 * hkv) * hd, seed=8), f32((hq + 2 * hkv) * hd, seed=9, scale=0.1)
    q, kc, vc = host_paged(lib, qkv, bias, inv, None, hd, pos, seq, table, 6, hq, hkv, hd)
    full = qkv + bias
    assert np.allclose(q, P.rope_neox(full[:, :hq * hd], pos, hd, 1e4), atol=1e-6)
    k_want = P.rope_neox(full[:, hq * hd:(hq + hkv) * hd], pos, hd, 1e4).reshape(5, hkv, hd)
    assert np.allclose(kc[2, :, 1, :], k_want[1], atol=1e-6) and np.allclose(kc[0, :, 6, :], k_want[3], atol=1e-6)
    # (head size 8: rows of keys keep the plain order; rows of values never do)
    assert np.array_equal(vc[1][:, np.arange(hd), layout.value_positions(hd)[:, 0]], full[4, (hq + hkv) * hd:].reshape(hkv, hd))
    # a head size whose rows are kept in the cache's own order: what the twin (the C functions of
    # sb_hip.h) stores is found where cache.layout (their Python face) says
    hq2, hkv2, hd2 = 2, 2, 32
    inv2 = np.exp(-2.0 * np.arange(hd2 // 2, dtype=np.float32) / hd2 * np.log(np.float32(1e4))).astype(np.float32)
    qkv2 = f32(3, (hq2 + 2 * hkv2) * hd2, seed=18)
    pos2, seq2, table2 = i32([5, 27, 64 + 40]), i32([0, 0, 0]), i32([[1, 0]])
    _, kc2, vc2 = host_paged(lib, qkv2, None, inv2, None, hd2, pos2, seq2, table2, 2, hq2, hkv2, hd2)
    k2 = P.rope_neox(qkv2[:, hq2 * hd2:(hq2 + hkv2) * hd2], pos2, hd2, 1e4).reshape(3, hkv2, hd2)
    v2 = qkv2[:, (hq2 + hkv2) * hd2:].reshape(3, hkv2, hd2)
    for r, (page, slot) in enumerate([(1, 5), (1, 27), (0, 40)]):
        assert np.allclose(kc2[page, :, slot][:, layout.key_positions(hd2)[slot]], k2[r], atol=1e-6)
        assert np.array_equal(vc2[page][:, np.arange(hd2), layout.value_positions(hd2)[:, slot]], v2[r])
    assert not np.allclose(kc2[1, :, 27], k2[1], atol=1e-6)          # slot 27's groups are not in the plain order
    y = np.array([[1.0, 0.0, 2.0, 3.0] * 3], np.float32)
    quarter = np.full(2, math.pi / 2, np.float32)
    qq, _, _ = host_paged(lib, y, None, quarter, None, 4, i32([1]), i32([0]), i32([[0]]), 1, 1, 1, 4)
    assert np.allclose(qq, [[-2.0, -3.0, 1.0, 0.0]], atol=1e-6)
    # attention over the three keys of sequence 0, against the plain routine; a window of 2 drops key 0
    for window in (0, 2):
        got = host_attention(lib, q[:3], kc, vc, table, pos[:3], seq[:3], hq, hkv, hd, 0.35, window)
        v_rows = full[:3, (hq + hkv) * hd:]
        want = P.attention(q[:3], k_want[:3].reshape(3, -1), v_rows, pos[:3], pos[:3], hq, hkv, hd, 0.35, window=window)
        assert np.allclose(got, want, atol=1e-6)
    ids = np.empty(3, np.int32)
    logits = np.array([[0.5, 0.5, 0.1], [1, 3, 3], [-np.inf] * 3], np.float32)
    assert lib.sbp_argmax(ptr(ids), ptr(logits), C(3), C(3)) == 0 and ids.tolist() == [0, 1, 0]


def host_penalize(lib, logits, rows, toks, counts, rp, pp, fp, exact):
    out = np.array(logits, np.float32, copy=True)
    assert lib.sbp_penalize(ptr(out), C(out.shape[1]), ptr(i32(rows)), ptr(i32(toks)), ptr(i32(counts)), C(len(rows)),
                            ctypes.c_float(rp), ctypes.c_float(pp), ctypes.c_float(fp), C(int(exact))) == 0
    return out


def host_mask(lib, logits, bitmaps):
    out = np.array(logits, np.float32, copy=True)
    assert lib.sbp_mask_logits(ptr(out), C(out.shape[0]), C(out.shape[1]), ptr(bitmaps), C(bitmaps.shape[1])) == 0
    return out


def host_candidates(lib, logits, k, temperature):
    ids, z = np.empty((logits.shape[0], k), np.int32), np.empty((logits.shape[0], k), np.float32)
    assert lib.sbp_top_candidates(ptr(ids), ptr(z), ptr(logits), C(logits.shape[0]), C(logits.shape[1]), C(k),
                                  ctypes.c_float(temperature)) == 0
    return ids, z


def host_draw(lib, ids, z, positions, top_k, min_p, top_p, seed):
    out = np.empty(ids.shape[0], np.int32)
    pos = np.ascontiguousarray(positions, dtype=np.int64)
    log_min_p = float(np.log(np.float32(min_p))) if min_p > 0.0 else 0.0
    assert lib.sbp_draw(ptr(out), ptr(ids), ptr(z), ptr(pos), C(ids.shape[0]), C(ids.shape[1]), C(top_k),
                        C(int(min_p > 0.0)), ctypes.c_float(log_min_p), C(int(0.0 < top_p < 1.0)),
                        ctypes.c_double(float(np.float32(top_p))), ctypes.c_uint64(seed)) == 0
    return out


def sampling_rows(vocab, n=24, seed=11):
    r = np.random.default_rng(seed)
    rows = (r.standard_normal((n, vocab)) * 3.0).astype(np.float32)
    rows[::5] *= 0.07                      # flat rows
    rows[3, 10:20] = rows[3, 5]            # ties among the best
    rows[1, 3] = 80.0                      # one candidate far above the window
    positions = [int(q) for q in r.integers(0, 5000, size=n)]
    positions[0], positions[1] = 0, 2 ** 33 + 5
    return rows, positions


SAMPLING_CASES = [dict(temperature=0.8), dict(temperature=1.3, top_k=5), dict(temperature=0.5, top_p=0.7),
                  dict(temperature=1.0, min_p=0.2), dict(temperature=0.9, top_k=40, top_p=0.9, min_p=0.01),
                  dict(temperature=1.0, top_p=1e-9, min_p=1.0)]


def test_sampling_twins_agree_with_the_plain_sampler():
    lib = twins()
    rows, positions = sampling_rows(400)
    # penalties, both arithmetic forms
    history = [5, 9, 5, 399, 5, 17]
    for exact in (False, True):
        want = SP.penalize(rows[0], exact, repeat_penalty=1.3, repeat_last_n=64, presence_penalty=0.25,
                           frequency_penalty=0.125, history=history)
        got = host_penalize(lib, rows[:1], [0, 0, 0, 0], [5, 9, 399, 17], [3, 1, 1, 1], 1.3, 0.25, 0.125, exact)
        assert np.array_equal(got[0], want)
    seed = 0x9E3779B97F4A7C15
    for case in SAMPLING_CASES:
        t = case["temperature"]
        ids, z = host_candidates(lib, rows, 256, t)
        got = host_draw(lib, ids, z, positions, case.get("top_k", 0), case.get("min_p", 0.0), case.get("top_p", 1.0), seed)
        for i in range(rows.shape[0]):
            cands = SP.select_candidates(rows[i], t)
            assert ids[i].tolist() == [c[0] for c in cands] and z[i].tolist() == [float(c[1]) for c in cands]
            kept = SP.filter_candidates(cands, case.get("top_k", 0), case.get("top_p", 1.0), case.get("min_p", 0.0))
            assert got[i] == SP.draw(kept, seed, positions[i]), (case, i)
    # a row shorter than the candidates asked for is filled with id -1
    ids, z = host_candidates(lib, rows[:2, :40], 64, 1.0)
    assert (ids[:, 40:] == -1).all() and (ids[:, :40] >= 0).all()
    # the mask: the candidates of the masked row are the plain sampler's under the same mask
    bitmaps = np.zeros((2, 12), np.uint8)            # 96 ids of 400: the rest is past the bitmap
    bitmaps[0, [0, 3, 11]] = [0b00001001, 0xFF, 0x80]
    bitmaps[1, :] = 0xFF
    masked = host_mask(lib, rows[:2], bitmaps)
    allowed0 = [0, 3] + list(range(24, 32)) + [95]
    assert np.isneginf(np.delete(masked[0], allowed0)).all() and np.array_equal(masked[0, allowed0], rows[0, allowed0])
    assert np.array_equal(masked[1, :96], rows[1, :96]) and np.isneginf(masked[1, 96:]).all()
    ids, z = host_candidates(lib, masked, 256, 0.8)
    want = SP.select_candidates(rows[0], 0.8, mask=bytes(bitmaps[0]))
    assert ids[0, :len(want)].tolist() == [c[0] for c in want] and np.isneginf(z[0, len(want):]).all()


# ---- kernels against twins ---------------------------------------------------------------------
@pytest.mark.gpu
def test_kernels_equal_their_host_twins():
    from sonicboom_amd import ops
    lib = twins()
    dev = lambda a, dt=None: None if a is None else torch.from_numpy(a).to(DEV if dt is None else DEV).to(dt or torch.from_numpy(a).dtype)  # noqa: E731
    # embedding
    table, ids = f32(37, 50, seed=1), i32([0, 36, 5, 5])
    want = np.empty((4, 50), np.float32)
    assert lib.sbp_embed(ptr(want), ptr(table), ptr(ids), C(4), C(50), C(37)) == 0
    assert np.array_equal(ops.embed(dev(table), dev(ids)).cpu().numpy(), want)
    # norm, float32 out: to rounding of the sum's order; rows picked
    for width, n_rows in ((96, 3), (3584, 5), (1001, 300)):
        x, w = f32(n_rows, width, seed=width, scale=2.0), f32(width, seed=2)
        got = ops.rmsnorm(dev(x), dev(w), 1e-6, F32).cpu().numpy()
        assert np.allclose(got, host_rmsnorm(lib, x, w, 1e-6), atol=1e-6, rtol=1e-6), width
    rows = i32([2, 0])
    assert np.allclose(ops.rmsnorm(dev(x), dev(w), 1e-6, F32, dev(rows)).cpu().numpy(),
                       host_rmsnorm(lib, x, w, 1e-6, rows), atol=1e-6, rtol=1e-6)
    # the plain product: the same fused multiply-adds in the same order, equal to the bit
    for t, n, k in ((3, 70, 33), (65, 17, 128), (9, 300, 1000)):
        x, w, b, r = f32(t, k, seed=t), f32(n, k, seed=n), f32(n, seed=3), f32(t, n, seed=4)
        got = ops.gemm_plain(dev(x), dev(w), dev(b), dev(r), F32).cpu().numpy()
        assert np.array_equal(got, host_gemm(lib, x, w, b, r)), (t, n, k)
    # the matrix-core products (bf16 operands, float sums) against the twin on the same rounded operands
    for t, n, k in ((8, 512, 256), (40, 200, 264), (300, 384, 512)):
        x = torch.from_numpy(f32(t, k, seed=5)).to(BF16)
        w = torch.from_numpy(f32(n, k, seed=6, scale=0.05)).to(BF16)
        want = host_gemm(lib, x.float().numpy(), w.float().numpy())
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(w.to(DEV)), None, None, F32, packed_shape=(n, k))
        assert np.allclose(got.cpu().numpy(), want, atol=2e-3, rtol=2e-3), (t, n, k)
    # slices + bias + residual + norm in one pass
    part, b, x, w = f32(3, 6, 256, seed=7), f32(256, seed=8), f32(6, 256, seed=9), f32(256, seed=10)
    x_host, y_host = x.copy(), np.empty((6, 256), np.float32)
    assert lib.sbp_reduce_resid_norm(ptr(y_host), ptr(x_host), ptr(part), C(3), ptr(b), ptr(w), C(6), C(256),
                                     ctypes.c_float(1e-5), C(1)) == 0
    x_dev = dev(x)
    y_dev = ops.reduce_resid_norm(dev(part), dev(b), x_dev, dev(w), 1e-5, F32)
    assert np.array_equal(x_dev.cpu().numpy(), x_host) and np.allclose(y_dev.cpu().numpy(), y_host, atol=1e-6)
    # silu * up, add
    gu = f32(5, 2 * 77, seed=11, scale=3.0)
    want = np.empty((5, 77), np.float32)
    lib.sbp_silu_mul(ptr(want), ptr(gu), C(5), C(77))
    assert np.allclose(ops.silu_mul(dev(gu), F32).cpu().numpy(), want, atol=1e-6, rtol=1e-6)
    # rotate-and-store, then attention over what was stored: both kernels against both twins
    for hq, hkv, hd, rot in ((6, 2, 48, 48), (4, 4, 64, 32), (8, 1, 128, 128)):
        lens = [130, 3, 64]
        table = i32([[4, 0, 7], [1, -1, -1], [5, -1, -1]])
        pos = i32(np.concatenate([np.arange(n) for n in lens]))
        seq = i32(np.concatenate([np.full(n, s) for s, n in enumerate(lens)]))
        width = (hq + 2 * hkv) * hd
        qkv, bias = f32(len(pos), width, seed=hd), f32(width, seed=12, scale=0.2)
        inv = np.exp(-2.0 * np.arange(rot // 2, dtype=np.float32) / rot * np.log(np.float32(5e4))).astype(np.float32)
        ff = (1.0 + np.arange(rot // 2, dtype=np.float32) / rot).astype(np.float32)
        q_h, kc_h, vc_h = host_paged(lib, qkv, bias, inv, ff, rot, pos, seq, table, 8, hq, hkv, hd)
        kc = torch.zeros((8, hkv, 64, hd), device=DEV)
        vc = torch.zeros((8, hkv, hd, 64), device=DEV)
        q_d = ops.rope_kv_store(dev(qkv), F32, dev(inv), dev(ff), rot, dev(pos), dev(seq), kc, vc, dev(table), hq, hkv,
                                hd, bias=dev(bias))
        for got, want in ((q_d, q_h), (kc, kc_h), (vc, vc_h)):
            assert np.allclose(got.cpu().numpy(), want, atol=2e-5, rtol=1e-5), (hq, hkv, hd)
        for window in (0, 50):
            want = host_attention(lib, q_h, kc_h, vc_h, table, pos, seq, hq, hkv, hd, hd ** -0.5, window)
            got = ops.attention_plain(q_d, kc, vc, dev(table), dev(pos), dev(seq), hq, hkv, hd, hd ** -0.5, window)
            assert np.allclose(got.cpu().numpy(), want, atol=1e-5, rtol=1e-4), (hq, hkv, hd, window)
    # the first maximum
    logits = f32(4, 20001, seed=13)
    logits[1, 7] = logits[1, 15000] = 9.0
    ids = np.empty(4, np.int32)
    lib.sbp_argmax(ptr(ids), ptr(logits), C(4), C(20001))
    assert ops.argmax(dev(logits)).cpu().numpy().tolist() == ids.tolist() and ids[1] == 7
    # penalties, candidates, filters and draw
    rows, positions = sampling_rows(5000, n=16, seed=21)
    item_rows, item_toks, item_counts = [0, 0, 3, 15], [7, 4999, 0, 123], [2, 1, 4, 1]
    for exact in (False, True):
        want = host_penalize(lib, rows, item_rows, item_toks, item_counts, 1.3, 0.25, 0.125, exact)
        got = dev(rows).clone()
        ops.penalize(got, dev(i32(item_rows)), dev(i32(item_toks)), dev(i32(item_counts)), 1.3, 0.25, 0.125, exact=exact)
        assert np.array_equal(got.cpu().numpy(), want)
    bitmaps = np.random.default_rng(5).integers(0, 256, size=(rows.shape[0], 500), dtype=np.uint8)   # 4,000 ids of 5,000
    masked = dev(rows).clone()
    ops.mask_logits(masked, dev(bitmaps))
    assert np.array_equal(masked.cpu().numpy(), host_mask(lib, rows, bitmaps))
    seed = 0x9E3779B97F4A7C15
    for case in SAMPLING_CASES:
        t = case["temperature"]
        ids_h, z_h = host_candidates(lib, rows, 256, t)
        ids_d, z_d = ops.top_candidates(dev(rows), t, 256)
        assert np.array_equal(ids_d.cpu().numpy(), ids_h) and np.array_equal(z_d.cpu().numpy(), z_h)
        min_p, top_p = case.get("min_p", 0.0), case.get("top_p", 1.0)
        want = host_draw(lib, ids_h, z_h, positions, case.get("top_k", 0), min_p, top_p, seed)
        got = ops.draw(ids_d, z_d, positions, case.get("top_k", 0),
                       float(np.log(np.float32(min_p))) if min_p > 0.0 else None,
                       float(np.float32(top_p)) if 0.0 < top_p < 1.0 else None, seed)
        assert got.cpu().numpy().tolist() == want.tolist(), case

"""Each kernel alone against a plain reference of the same operation, at sizes other
than the engine's tiny configurations: widths that are no power of two, ragged row
counts, head sizes in steps of 16, any number of heads and groups."""
import math

import numpy as np
import pytest
import torch

from plain import qwen2_plain as plain
from plain import sampling_plain
from sonicboom_amd.cache import layout

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF16, F32 = torch.bfloat16, torch.float32


def randn(*shape, dtype=F32, scale=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * scale).to(dtype)


def close(got, want, atol, rtol, what=""):
    got = got.detach().float().cpu().double()
    want = torch.as_tensor(want).double()
    assert got.shape == want.shape, f"{what}: {tuple(got.shape)} vs {tuple(want.shape)}"
    assert torch.isfinite(got).all(), f"{what}: not finite"
    err = (got - want).abs()
    bound = atol + rtol * want.abs()
    assert (err <= bound).all(), f"{what}: max |diff| {err.max():.3g} (worst excess {(err - bound).max():.3g})"


# -------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_embed(dtype):
    from sonicboom_amd import ops
    table = randn(301, 72, dtype=dtype)
    ids = torch.tensor([0, 300, 7, 7, 150], dtype=torch.int32)
    got = ops.embed(table.to(DEV), ids.to(DEV))
    assert got.dtype == F32 and torch.equal(got.cpu(), table.float()[ids.long()])
    bad = ops.embed(table.to(DEV), torch.tensor([301, -1], dtype=torch.int32, device=DEV))
    assert torch.isnan(bad).all()          # an id outside the table never reads memory it does not own


@pytest.mark.parametrize("n_rows", [7, 300])       # few rows and many rows take different block shapes
@pytest.mark.parametrize("width", [64, 201, 338, 3584, 5000, 8192, 9004])     # up to 4,096, up to 8,192, beyond
@pytest.mark.parametrize("out_dtype, w_dtype", [(F32, F32), (BF16, BF16), (BF16, F32)])
def test_rmsnorm(width, out_dtype, w_dtype, n_rows):
    from sonicboom_amd import ops
    x = randn(n_rows, width, scale=3.0)
    w = (1.0 + randn(width, scale=0.1)).to(w_dtype)
    eps = 1e-5
    want = plain.rms_norm(x.numpy(), w.float().numpy(), eps)
    got = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out_dtype)
    tol = dict(atol=1e-6, rtol=2e-6) if out_dtype == F32 else dict(atol=1e-2, rtol=8e-3)
    close(got, want, what="rmsnorm", **tol)
    rows = torch.tensor([5, 0, 5], dtype=torch.int32)
    picked = ops.rmsnorm(x.to(DEV), w.to(DEV), eps, out_dtype, rows.to(DEV))
    assert torch.equal(picked.cpu(), got.cpu()[rows.long()])


@pytest.mark.parametrize("width", [64, 100, 3584, 5120, 8192])
@pytest.mark.parametrize("n_slices", [1, 5, 8])
@pytest.mark.parametrize("out_dtype", [F32, BF16])
def test_reduce_resid_norm(width, n_slices, out_dtype):
    """x += slices (+ bias), then the norm of the new x, in one pass: rows narrower and wider than
    what a thread keeps in one group of four."""
    from sonicboom_amd import ops
    rows, eps = 9, 1e-6
    partial = randn(n_slices, rows, width, seed=1)
    x = randn(rows, width, scale=2.0, seed=2)
    bias = randn(width, scale=0.1, seed=3)
    w = 1.0 + randn(width, scale=0.1, seed=4)
    new_x = x.double() + partial.double().sum(0) + bias.double()
    want_y = plain.rms_norm(new_x.float().numpy(), w.numpy(), eps)
    xd = x.to(DEV)
    y = ops.reduce_resid_norm(partial.to(DEV), bias.to(DEV), xd, w.to(DEV), eps, out_dtype)
    close(xd, new_x, atol=2e-6 * n_slices, rtol=2e-6, what="residual")
    tol = dict(atol=2e-5, rtol=2e-5) if out_dtype == F32 else dict(atol=1e-2, rtol=8e-3)
    close(y, want_y, what="normed", **tol)
    # without a norm: only the sum
    xd2 = x.to(DEV)
    assert ops.reduce_resid_norm(partial.to(DEV), None, xd2, None, eps, None) is None
    close(xd2, x.double() + partial.double().sum(0), atol=2e-6 * n_slices, rtol=2e-6, what="sum only")


def test_rmsnorm_reference_vectors():
    """/root/reference/tests/core/test_nn.cpp:172-219."""
    from sonicboom_amd import ops
    x = torch.tensor([[2.0, 2.0, 2.0, 2.0]], device=DEV)
    assert torch.allclose(ops.rmsnorm(x, None, 0.0, F32).cpu(), torch.ones(1, 4), atol=1e-6)
    w3 = torch.full((4,), 3.0, device=DEV)
    assert torch.allclose(ops.rmsnorm(x, w3, 0.0, F32).cpu(), torch.full((1, 4), 3.0), atol=1e-6)
    e = torch.tensor([[1.0, 0.0, 0.0, 0.0]], device=DEV)
    assert torch.equal(ops.rmsnorm(e, None, 0.75, F32).cpu(), torch.tensor([[1.0, 0.0, 0.0, 0.0]]))


def ref_gemm(x, w, bias=None, resid=None):
    y = x.double() @ w.double().T
    if bias is not None:
        y = y + bias.double()
    if resid is not None:
        y = y + resid.double()
    return y


@pytest.mark.parametrize("t, n, k", [(1, 100, 96), (5, 224, 200), (64, 64, 64), (130, 97, 51), (3, 1000, 3584)])
@pytest.mark.parametrize("xd, wd", [(F32, F32), (BF16, BF16), (BF16, F32), (F32, BF16)])
def test_gemm_plain(t, n, k, xd, wd):
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=xd), randn(n, k, dtype=wd, scale=0.05)
    bias, resid = randn(n, scale=0.1), randn(t, n)
    want = ref_gemm(x, w, bias, resid)
    got = ops.gemm_plain(x.to(DEV), w.to(DEV), bias.to(DEV), resid.to(DEV), F32)
    close(got, want, atol=2e-5 * math.sqrt(k), rtol=1e-5, what="gemm_plain")
    # in place on the residual, and without the extras
    r = resid.to(DEV)
    ops.gemm_plain(x.to(DEV), w.to(DEV), None, r, F32, out=r)
    close(r, ref_gemm(x, w, None, resid), atol=2e-5 * math.sqrt(k), rtol=1e-5, what="gemm_plain in place")


def test_gemm_plain_does_not_depend_on_the_batch():
    """The same row gives the same bits alone and among 200 others."""
    from sonicboom_amd import ops
    x, w = randn(200, 333).to(DEV), randn(150, 333, scale=0.05).to(DEV)
    whole = ops.gemm_plain(x, w, None, None, F32)
    for r in (0, 63, 64, 199):
        alone = ops.gemm_plain(x[r:r + 1].contiguous(), w, None, None, F32)
        assert torch.equal(alone[0], whole[r])


@pytest.mark.parametrize("t", [1, 5, 16, 17, 33, 64, 65, 128, 300])
@pytest.mark.parametrize("n, k", [(96, 64), (100, 96), (224, 200), (3584, 512), (1000, 3584), (72, 18944 // 8)])
def test_gemm_bf16_matrix_cores(t, n, k):
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    bias, resid = randn(n, scale=0.1), randn(t, n)
    want = ref_gemm(x, w, bias, resid)
    got = ops.gemm_bf16(x.to(DEV), w.to(DEV), bias.to(DEV), resid.to(DEV), F32)
    assert got is not None
    close(got, want, atol=3e-5 * math.sqrt(k), rtol=1e-5, what=f"gemm_bf16 t={t}")
    got16 = ops.gemm_bf16(x.to(DEV), w.to(DEV), None, None, BF16)
    close(got16, ref_gemm(x, w), atol=2e-2, rtol=8e-3, what=f"gemm_bf16 bf16 out t={t}")
    r = resid.to(DEV)
    ops.gemm_bf16(x.to(DEV), w.to(DEV), None, r, F32, out=r)
    close(r, ref_gemm(x, w, None, resid), atol=3e-5 * math.sqrt(k), rtol=1e-5, what="in place")


@pytest.mark.parametrize("t", [1, 8, 40, 64, 65, 200])
@pytest.mark.parametrize("inner, k", [(100, 96), (224, 200), (18944 // 4, 512)])
def test_gemm_bf16_gated(t, inner, k):
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(2 * inner, k, dtype=BF16, scale=0.1)
    gu = x.double() @ w.double().T
    g, u = gu[:, :inner], gu[:, inner:]
    want = g / (1.0 + torch.exp(-g)) * u
    got = ops.gemm_bf16(x.to(DEV), w.to(DEV), None, None, F32, gated=True)
    close(got, want, atol=1e-4 * math.sqrt(k), rtol=1e-4, what=f"gated t={t}")


def gelu_tanh(g):
    """0.5 g (1 + tanh(sqrt(2/pi) g (1 + 0.044715 g^2))), /root/reference/core/src/nn/activation.cpp:27-36."""
    return 0.5 * g * (1.0 + torch.tanh(0.7978845608028654 * g * (1.0 + 0.044715 * g * g)))


@pytest.mark.parametrize("t", [1, 8, 40, 64, 65, 128, 300])
def test_gemm_bf16_gate_activations(t):
    """The gate's activation is an argument of every product kernel and of the elementwise
    kernel: SiLU and the tanh form of GELU, through the stream, the K-splitting and the tiled
    kernels, against the formula and against torch's own GELU."""
    from sonicboom_amd import ops
    inner, k = 1040, 264
    x, w = randn(t, k, dtype=BF16), randn(2 * inner, k, dtype=BF16, scale=0.15)
    gu = x.double() @ w.double().T
    g, u = gu[:, :inner], gu[:, inner:]
    assert torch.allclose(gelu_tanh(g), torch.nn.functional.gelu(g, approximate="tanh"), atol=1e-12)
    want = {"silu": g / (1.0 + torch.exp(-g)) * u, "gelu_tanh": gelu_tanh(g) * u}
    assert (want["silu"] - want["gelu_tanh"]).abs().max() > 0.05          # the two differ visibly
    packed = ops.pack_weight(w.to(DEV), True)
    for act in ("silu", "gelu_tanh"):
        for which in ("stream", "skinny", "tiled"):
            if (which == "stream" and t > 128) or (which == "skinny" and t > 64):
                continue
            with ops.gemm_few_rows_kernel(which):
                got = ops.gemm_bf16(x.to(DEV), packed, None, None, F32, gated=act, packed_shape=(2 * inner, k))
            close(got, want[act], atol=1e-4 * math.sqrt(k), rtol=1e-4, what=f"{act} through {which}, t={t}")
        got = ops.gate_mul(gu.float().to(DEV), F32, act)
        close(got, want[act], atol=1e-5, rtol=1e-5, what=f"{act}, elementwise")
    with pytest.raises(ops.KernelLibraryError, match="unknown gate activation"):
        ops.gate_mul(gu.float().to(DEV), F32, "relu")


@pytest.mark.parametrize("shape", [0, 1, 2])
@pytest.mark.parametrize("packed", [False, True])
@pytest.mark.parametrize("t, n, k", [(65, 100, 96), (300, 224, 200), (520, 264, 128), (257, 1000, 448), (130, 72, 2368)])
def test_gemm_bf16_every_tile_shape(shape, packed, t, n, k):
    """Each tile shape of the tiled product, with K a multiple of the stage or not, rows and
    columns that end inside a tile, plain and packed weights, plain and gated."""
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    bias, resid = randn(n, scale=0.1), randn(t, n)
    wd = w.to(DEV)
    # plain (unpacked) weights always take the 128 x 128 tile
    with ops.gemm_tile_shape(shape):
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd) if packed else wd, bias.to(DEV), resid.to(DEV), F32,
                            packed_shape=(n, k) if packed else None)
        close(got, ref_gemm(x, w, bias, resid), atol=3e-5 * math.sqrt(k), rtol=1e-5, what=f"shape {shape}")
        inner = n // 2
        gu = x.double() @ w[:2 * inner].double().T
        g, u = gu[:, :inner], gu[:, inner:]
        wg = wd[:2 * inner].contiguous()
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wg, True) if packed else wg, None, None, F32, gated=True,
                            packed_shape=(2 * inner, k) if packed else None)
        close(got, g / (1.0 + torch.exp(-g)) * u, atol=1e-4 * math.sqrt(k), rtol=1e-4, what=f"gated shape {shape}")


@pytest.mark.parametrize("shape, path", [(0, "direct"), (1, "direct"), (2, "direct"), (3, "direct"), (4, "direct"),
                                         (2, "direct, a block a tile"), (0, "registers"), (2, "registers")])
@pytest.mark.parametrize("t, n, k", [(65, 100, 64), (300, 226, 192), (520, 264, 128), (257, 1001, 448), (130, 72, 2368)])
def test_gemm_bf16_every_path(shape, path, t, n, k):
    """The kernel that loads its tiles straight into LDS (inner sizes in 64s, packed weights) and
    the one that stages them through registers, forced for every tile shape: rows and columns
    that end inside a tile, widths that are no multiple of 4 (single stores in the epilogue),
    bias and residual, bfloat16 and float32 results, plain and gated."""
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    bias, resid = randn(n, scale=0.1), randn(t, n)
    wd = w.to(DEV)
    with ops.gemm_tile_shape(shape, path):
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd), bias.to(DEV), resid.to(DEV), F32, packed_shape=(n, k))
        close(got, ref_gemm(x, w, bias, resid), atol=3e-5 * math.sqrt(k), rtol=1e-5, what=f"shape {shape} {path}")
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd), bias.to(DEV), None, BF16, packed_shape=(n, k))
        close(got, ref_gemm(x, w, bias, None), atol=0.01 * math.sqrt(k) * 0.05 + 0.01, rtol=0.01, what=f"bf16 shape {shape} {path}")
        inner = n // 2
        gu = x.double() @ w[:2 * inner].double().T
        g, u = gu[:, :inner], gu[:, inner:]
        wg = wd[:2 * inner].contiguous()
        for act, want in (("silu", g / (1.0 + torch.exp(-g)) * u),
                          ("gelu_tanh", 0.5 * g * (1 + torch.tanh(0.7978845608028654 * g * (1 + 0.044715 * g * g))) * u)):
            got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wg, True), None, None, F32, gated=act, packed_shape=(2 * inner, k))
            close(got, want, atol=1e-4 * math.sqrt(k), rtol=1e-4, what=f"gated {act} shape {shape} {path}")


def test_gemm_bf16_blocks_that_go_from_tile_to_tile():
    """More 256 x 256 tiles than the GPU has CUs: the blocks of the kernel that loads straight into
    LDS go on to a second tile, whose first stage the first tile's last stage has loaded; in
    bands of eight tiles along the rows, the last band lower.  Every tile has a value of its own."""
    from sonicboom_amd import ops
    t, n, k = 4400, 4200, 128                  # 18 x 17 = 306 tiles; gated: 18 x 33 tiles of 256 x 128
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    want = ref_gemm(x, w, None, None)
    wd = w.to(DEV)
    # (tiles of 192 rows: 23 x 17 = 391)
    for shape, path in ((2, "direct"), (2, "direct, a block a tile"), (4, "direct")):
        with ops.gemm_tile_shape(shape, path):
            got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd), None, None, F32, packed_shape=(n, k))
            close(got, want, atol=3e-5 * math.sqrt(k), rtol=1e-5, what=f"{shape} {path}")
            inner = n // 2
            g, u = want[:, :inner].double(), want[:, inner:2 * inner].double()
            got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd[:2 * inner].contiguous(), True), None, None, F32,
                                gated=True, packed_shape=(2 * inner, k))
            close(got, g / (1.0 + torch.exp(-g)) * u, atol=1e-4 * math.sqrt(k), rtol=1e-4, what=f"gated {shape} {path}")


def test_gemm_bf16_direct_path_refuses_what_it_cannot_take():
    from sonicboom_amd import ops
    x, w = randn(70, 96, dtype=BF16).to(DEV), randn(64, 96, dtype=BF16).to(DEV)
    with ops.gemm_tile_shape(0, "direct"):
        with pytest.raises(ops.KernelLibraryError, match="inner size in 64s"):
            ops.gemm_bf16(x, ops.pack_weight(w), None, None, F32, packed_shape=(64, 96))
    with ops.gemm_tile_shape(3, "registers"):
        with pytest.raises(ops.KernelLibraryError, match="direct path only"):
            ops.gemm_bf16(x, ops.pack_weight(w), None, None, F32, packed_shape=(64, 96))


@pytest.mark.parametrize("t", [1, 16, 17, 40, 64, 65, 100, 128])
@pytest.mark.parametrize("waves", [0, 4, 5, 6, 7, 8])
@pytest.mark.parametrize("n, k", [(100, 96), (1000, 520), (264, 2368), (4099, 264)])
def test_gemm_bf16_stream_kernel(t, waves, n, k):
    """The kernel for few rows against wide matrices, at every count of waves per block: K
    shorter than one staged chunk, ending inside a chunk and inside a k-step; columns that end
    inside a tile and inside a block; plain with bias and residual, and gated."""
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    bias, resid = randn(n, scale=0.1), randn(t, n)
    wd = w.to(DEV)
    with ops.gemm_few_rows_kernel("stream", waves):
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd), bias.to(DEV), resid.to(DEV), F32, packed_shape=(n, k))
        close(got, ref_gemm(x, w, bias, resid), atol=3e-5 * math.sqrt(k), rtol=1e-5, what="stream")
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wd), None, None, BF16, packed_shape=(n, k))
        close(got.float(), ref_gemm(x, w), atol=2e-2, rtol=1e-2, what="stream, bfloat16 out")
        inner = n // 2
        wg = wd[:2 * inner].contiguous()
        gu = x.double() @ w[:2 * inner].double().T
        g, u = gu[:, :inner], gu[:, inner:]
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(wg, True), None, None, F32, gated=True,
                            packed_shape=(2 * inner, k))
        close(got, g / (1.0 + torch.exp(-g)) * u, atol=1e-4 * math.sqrt(k), rtol=1e-4, what="stream, gated")


@pytest.mark.parametrize("t", [8, 17, 64, 100])
def test_gemm_bf16_wide_matrix_with_few_rows(t):
    """Up to 128 rows against a packed matrix wide enough for the stream kernel, and one wave's
    worth of columns less (which stays with the kernel that splits K), plain and gated: the
    choice between the kernels changes no result."""
    from sonicboom_amd import ops
    from sonicboom_amd.ops import kernels
    k = 64
    x = randn(t, k, dtype=BF16)
    edge = 4 * kernels.STREAM_MIN_BLOCKS
    for n in (edge * 32, edge * 32 - 32):
        w = randn(n, k, dtype=BF16, scale=0.05)
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(w.to(DEV)), None, None, F32, packed_shape=(n, k))
        close(got, ref_gemm(x, w), atol=3e-5 * math.sqrt(k), rtol=1e-5, what=f"wide n={n}")
    for inner in (edge * 16, edge * 16 - 16):
        w = randn(2 * inner, k, dtype=BF16, scale=0.05)
        gu = x.double() @ w.double().T
        g, u = gu[:, :inner], gu[:, inner:]
        got = ops.gemm_bf16(x.to(DEV), ops.pack_weight(w.to(DEV), True), None, None, F32, gated=True,
                            packed_shape=(2 * inner, k))
        close(got, g / (1.0 + torch.exp(-g)) * u, atol=1e-4 * math.sqrt(k), rtol=1e-4, what=f"wide gated {inner}")


@pytest.mark.parametrize("t", [1, 8, 16, 17, 40, 64, 65, 130, 300])
@pytest.mark.parametrize("n, k", [(100, 96), (224, 200), (3584, 512), (264, 2368), (72, 18944 // 8)])
@pytest.mark.parametrize("packed", [False, True])
def test_gemm_bf16_partial_slices_add_up(t, n, k, packed):
    """The product in K slices (packed weights: the stream kernel up to 64 rows, the tiled kernel
    beyond; row-major weights: the kernel whose waves split K): the slices add up to x w^T, and
    the consumers that add them give the fused results."""
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    wd = w.to(DEV)
    partial = ops.gemm_bf16_partial(x.to(DEV), ops.pack_weight(wd) if packed else wd,
                                    packed_shape=(n, k) if packed else None)
    if t > 64 and (not packed or partial is None):
        assert partial is None          # no cut that pays: the caller takes the whole product
        return
    assert partial is not None and partial.shape[1:] == (t, n) and 1 <= partial.shape[0] <= 8
    assert t <= 64 or partial.shape[0] > 1
    close(partial.double().sum(0), ref_gemm(x, w), atol=3e-5 * math.sqrt(k), rtol=1e-5, what="sum of the slices")
    if n % 4 == 0:
        resid, bias = randn(t, n), randn(n, scale=0.1)
        rd = resid.to(DEV)
        ops.reduce_resid_norm(partial, bias.to(DEV), rd, None, 1e-6, None)
        close(rd, ref_gemm(x, w, bias, resid), atol=3e-5 * math.sqrt(k), rtol=1e-5, what="slices + bias + residual")


def test_gemm_bf16_partial_in_big_tiles():
    """Two thousand rows against a narrow matrix with a long inner size: 56 tiles of 256 x 256 with
    K cut in four fill the GPU where 224 tiles of 128 x 128 would multiply whole.  The slices add
    up to the product (sampled rows against float64, all of it against the whole product), and
    the pass that adds them gives product + bias + residual and the norm of that."""
    from sonicboom_amd import ops
    t, n, k = 2048, 1792, 18944
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.02)
    xd, wp = x.to(DEV), ops.pack_weight(w.to(DEV))
    partial = ops.gemm_bf16_partial(xd, wp, packed_shape=(n, k))
    assert partial is not None and tuple(partial.shape) == (4, t, n)
    total = partial.double().sum(0)
    rows = [0, 1, 255, 256, 1000, 2047]
    close(total[rows], ref_gemm(x[rows], w), atol=3e-5 * math.sqrt(k), rtol=1e-5, what="sampled rows")
    whole = ops.gemm_bf16(xd, wp, None, None, F32, packed_shape=(n, k))
    close(total, whole.double().cpu(), atol=3e-5 * math.sqrt(k), rtol=1e-5, what="against the whole product")
    resid, bias, nw = randn(t, n), randn(n, scale=0.1), 1.0 + randn(n, scale=0.1)
    rd = resid.to(DEV)
    normed = ops.reduce_resid_norm(partial, bias.to(DEV), rd, nw.to(DEV), 1e-5, F32)
    want = whole.double().cpu() + bias.double() + resid.double()
    close(rd, want, atol=3e-5 * math.sqrt(k), rtol=1e-5, what="slices + bias + residual")
    want_n = want / torch.sqrt((want * want).mean(-1, keepdim=True) + 1e-5) * nw.double()
    close(normed, want_n, atol=1e-4, rtol=1e-4, what="and the norm")
    # a short inner size: the pass over four slices would cost more than the cut saves
    assert ops.gemm_bf16_partial(xd[:, :1024].contiguous(), ops.pack_weight(w[:, :1024].contiguous().to(DEV)),
                                 packed_shape=(n, 1024)) is None


@pytest.mark.parametrize("which, waves, slices", [("stream", 4, 1), ("stream", 5, 3), ("stream", 7, 8), ("stream", 8, 5),
                                                  ("tiled", 0, 0), ("skinny", 0, 0)])
@pytest.mark.parametrize("t", [3, 16, 33, 64])
@pytest.mark.parametrize("n, k", [(100, 96), (1000, 520), (264, 2368), (72, 4744)])
def test_gemm_bf16_partial_every_kernel(which, waves, slices, t, n, k):
    """Each kernel that can cut K, at forced cuts: slices that end inside a staged chunk of 256 k
    and inside a k-step, more slices asked for than K has chunks, columns that end inside a
    tile."""
    from sonicboom_amd import ops
    x, w = randn(t, k, dtype=BF16), randn(n, k, dtype=BF16, scale=0.05)
    with ops.gemm_few_rows_kernel(which, waves, slices):
        partial = ops.gemm_bf16_partial(x.to(DEV), ops.pack_weight(w.to(DEV)), packed_shape=(n, k))
    assert partial is not None and partial.shape[1:] == (t, n) and 1 <= partial.shape[0] <= 8
    if which == "stream" and slices:
        assert partial.shape[0] <= slices
    close(partial.double().sum(0), ref_gemm(x, w), atol=3e-5 * math.sqrt(k), rtol=1e-5, what=f"{which}: sum of the slices")


def test_gemm_bf16_refuses_what_it_cannot_take():
    from sonicboom_amd import ops
    x, w = randn(4, 100, dtype=BF16).to(DEV), randn(8, 100, dtype=BF16).to(DEV)
    assert ops.gemm_bf16(x, w, None, None, F32) is None          # inner size not a multiple of 8
    want = ref_gemm(x.cpu(), w.cpu())
    close(ops.gemm_plain(x, w, None, None, F32), want, atol=1e-3, rtol=1e-5)


@pytest.mark.parametrize("dtype", [F32, BF16])
def test_silu_mul_add_cast(dtype):
    from sonicboom_amd import ops
    gu = randn(9, 2 * 77, scale=3.0)
    gu[0, 0], gu[0, 1], gu[0, 2] = 0.0, 1.0, -100.0
    want = plain.silu(gu[:, :77].numpy()) * gu[:, 77:].numpy()
    got = ops.silu_mul(gu.to(DEV), dtype)
    close(got, want, atol=1e-6 if dtype == F32 else 2e-2, rtol=1e-6 if dtype == F32 else 8e-3)
    # silu(0) = 0, silu(1) = 0.7310586 (/root/reference/tests/core/test_nn.cpp:52-66)
    one = ops.silu_mul(torch.tensor([[0.0, 1.0, 1.0, 1.0]], device=DEV), F32).cpu()
    assert one[0, 0] == 0.0 and abs(one[0, 1].item() - 0.7310586) < 1e-6
    resid = randn(5, 33)
    y = randn(5, 33, dtype=dtype, seed=3)
    r = resid.to(DEV)
    ops.add_into(r, y.to(DEV))
    assert torch.equal(r.cpu(), resid + y.float())
    c = ops.cast(resid.to(DEV), BF16)
    assert torch.equal(c.cpu(), resid.to(BF16))


def make_cache(n_pages, heads_kv, head_dim, dtype, fill=float("nan")):
    """Keys [pages, heads, 64, d] and values [pages, heads, d, 64], filled with NaN: whatever a
    kernel reads beyond what was stored shows in its result.  Within a row the cache keeps its own
    order of elements; the tests read and write through sonicboom_amd.cache.layout."""
    k = torch.full((n_pages, heads_kv, 64, head_dim), fill, dtype=dtype, device=DEV)
    v = torch.full((n_pages, heads_kv, head_dim, 64), fill, dtype=dtype, device=DEV)
    return k, v


@pytest.mark.parametrize("hq, hkv, hd, rot", [(4, 2, 16, 0), (3, 1, 32, 0), (5, 5, 48, 0), (2, 1, 64, 32), (8, 2, 128, 0)])
@pytest.mark.parametrize("dtype", [F32, BF16])
def test_rope_kv_store(hq, hkv, hd, rot, dtype):
    """Rotation against the plain rope; keys and values land where the page table says."""
    from sonicboom_amd import ops
    base = 10000.0
    n = 11
    qkv = randn(n, (hq + 2 * hkv) * hd)
    pos = torch.tensor([0, 1, 2, 63, 64, 65, 130, 7, 200, 1000, 5], dtype=torch.int32)
    seq = torch.tensor([0, 0, 0, 0, 0, 0, 0, 1, 1, 1, 1], dtype=torch.int32)   # row -> sequence
    pos[7:] = torch.tensor([3, 64, 127, 128])
    # scattered physical pages, different per sequence
    table = torch.tensor([[5, 2, 7], [1, 6, 3]], dtype=torch.int32)
    kc, vc = make_cache(8, hkv, hd, dtype)
    dims = rot or hd
    ff = (1.0 + torch.arange(dims // 2, dtype=F32) / 7.0) if rot else None
    log_base = np.log(np.float32(base)).astype(np.float32)
    inv = np.exp((np.float32(-2.0) * np.arange(dims // 2, dtype=np.float32) / np.float32(dims)).astype(np.float32)
                 * log_base).astype(np.float32)
    q = ops.rope_kv_store(qkv.to(DEV), dtype, torch.from_numpy(inv).to(DEV), None if ff is None else ff.to(DEV),
                          dims, pos.to(DEV), seq.to(DEV), kc, vc, table.to(DEV), hq, hkv, hd)
    qw, kvw = hq * hd, hkv * hd
    ffn = None if ff is None else ff.numpy()
    want_q = plain.rope_neox(qkv[:, :qw].numpy(), pos.numpy(), hd, base, rot, ffn)
    want_k = plain.rope_neox(qkv[:, qw:qw + kvw].numpy(), pos.numpy(), hd, base, rot, ffn)
    tol = dict(atol=2e-6, rtol=1e-5) if dtype == F32 else dict(atol=2e-2, rtol=8e-3)
    close(q, want_q, what="q", **tol)
    for r in range(n):
        page = table[seq[r], pos[r] // 64]
        got_k = layout.get_key(kc, int(page), int(pos[r]) % 64).reshape(-1)
        got_v = layout.get_value(vc, int(page), int(pos[r]) % 64).reshape(-1)
        close(got_k, want_k[r], what=f"k row {r}", **tol)
        close(got_v, qkv[r, qw + kvw:].to(dtype).float(), atol=0, rtol=0, what=f"v row {r}")
    # nothing else was written
    assert torch.isnan(kc.float()).sum().item() == kc.numel() - n * kvw


@pytest.mark.parametrize("hq, hkv, hd, rot", [(7, 1, 48, 0), (28, 4, 128, 0), (3, 3, 64, 32)])
def test_rope_kv_store_many_rows_equals_few_rows(hq, hkv, hd, rot):
    """A prompt of 700 rows in one call (all heads of a row in one block) gives bitwise what the
    same rows give in calls of 100 (groups of four heads)."""
    from sonicboom_amd import ops
    n = 700
    qkv = randn(n, (hq + 2 * hkv) * hd).to(DEV)
    bias = randn((hq + 2 * hkv) * hd, scale=0.1, seed=3).to(DEV)
    pos = torch.arange(n, dtype=torch.int32, device=DEV)
    seq = torch.zeros(n, dtype=torch.int32, device=DEV)
    table = torch.tensor([[4, 9, 1, 7, 3, 10, 0, 6, 2, 8, 5]], dtype=torch.int32, device=DEV)
    dims = rot or hd
    inv = torch.exp(-2.0 * torch.arange(dims // 2, dtype=F32) / dims * math.log(1e6)).to(DEV)
    results = []
    for step in (n, 100):
        kc, vc = make_cache(11, hkv, hd, BF16, fill=0.0)
        qs = [ops.rope_kv_store(qkv[r0:r0 + step], BF16, inv, None, dims, pos[r0:r0 + step], seq[r0:r0 + step], kc, vc,
                                table, hq, hkv, hd, bias=bias) for r0 in range(0, n, step)]
        results.append((torch.cat(qs), kc, vc))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    want_q = plain.rope_neox((qkv.cpu() + bias.cpu())[:, :hq * hd].numpy(), pos.cpu().numpy(), hd, 1e6, rot, None)
    close(results[0][0], want_q, atol=2e-2, rtol=8e-3, what="q of the long prompt")


@pytest.mark.parametrize("hq, hkv, hd, rot", [(7, 1, 48, 0), (28, 4, 128, 0), (3, 3, 64, 32), (5, 2, 80, 0), (2, 0, 32, 0)])
@pytest.mark.parametrize("rotate", [True, False])
@pytest.mark.parametrize("in_dtype", [F32, BF16])
def test_rope_kv_store_rows_eight_pairs_at_a_time(hq, hkv, hd, rot, rotate, in_dtype):
    """A prompt step's qkv rows (float32 as the engine has them, or bfloat16; no slices, no bias)
    go through the kernel that moves eight pairs per load and store: bitwise what the same rows
    give in calls of 100, which take the element-wise kernel; with a partial rotary width,
    without rotation, and for a layer that stores no keys."""
    from sonicboom_amd import ops
    n = 700
    qkv = randn(n, (hq + 2 * hkv) * hd, dtype=in_dtype).to(DEV)
    pos = (torch.arange(n, dtype=torch.int32) * 3 % 701).to(DEV)
    seq = torch.zeros(n, dtype=torch.int32, device=DEV)
    table = torch.tensor([[4, 9, 1, 7, 3, 10, 0, 6, 2, 8, 5]], dtype=torch.int32, device=DEV)
    dims = rot or hd
    inv = torch.exp(-2.0 * torch.arange(dims // 2, dtype=F32) / dims * math.log(1e6)).to(DEV) if rotate else None
    results = []
    for step in (n, 100):
        kc, vc = make_cache(11, max(hkv, 1), hd, BF16, fill=0.0)
        qs = [ops.rope_kv_store(qkv[r0:r0 + step], BF16, inv, None, dims, pos[r0:r0 + step], seq[r0:r0 + step], kc, vc,
                                table, hq, hkv, hd) for r0 in range(0, n, step)]
        results.append((torch.cat(qs), kc, vc))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    if rotate:
        want_q = plain.rope_neox(qkv.float().cpu()[:, :hq * hd].numpy(), pos.cpu().numpy(), hd, 1e6, rot, None)
        close(results[0][0], want_q, atol=2e-2, rtol=8e-3, what="q of the long prompt")
    else:
        assert torch.equal(results[0][0], qkv[:, :hq * hd].to(BF16))


@pytest.mark.parametrize("hq, hkv, hd, rot", [(28, 4, 128, 0), (3, 3, 64, 32), (5, 2, 80, 0)])
@pytest.mark.parametrize("slices", [2, 3, 5])
@pytest.mark.parametrize("in_dtype", [F32, BF16])
def test_rope_kv_store_rows_in_slices_with_a_bias(hq, hkv, hd, rot, slices, in_dtype):
    """The same kernel takes a prompt's qkv rows as K slices of the product with the bias still to
    add (what the sliced product of a few hundred rows leaves): slices added in ascending order,
    then the bias, bitwise as the element-wise kernel does it in calls of 100 rows, and the sum is
    the plain rotation of the summed rows."""
    from sonicboom_amd import ops
    n, w = 700, (hq + 2 * hkv) * hd
    parts = randn(slices, n, w, dtype=in_dtype).to(DEV)
    bias = randn(w, scale=0.1, seed=3).to(DEV)
    pos = (torch.arange(n, dtype=torch.int32) * 3 % 701).to(DEV)
    seq = torch.zeros(n, dtype=torch.int32, device=DEV)
    table = torch.tensor([[4, 9, 1, 7, 3, 10, 0, 6, 2, 8, 5]], dtype=torch.int32, device=DEV)
    dims = rot or hd
    inv = torch.exp(-2.0 * torch.arange(dims // 2, dtype=F32) / dims * math.log(1e6)).to(DEV)
    results = []
    for step in (n, 100):
        kc, vc = make_cache(11, hkv, hd, BF16, fill=0.0)
        qs = [ops.rope_kv_store(parts[:, r0:r0 + step].contiguous(), BF16, inv, None, dims, pos[r0:r0 + step],
                                seq[r0:r0 + step], kc, vc, table, hq, hkv, hd, bias=bias) for r0 in range(0, n, step)]
        results.append((torch.cat(qs), kc, vc))
    for a, b in zip(*results):
        assert torch.equal(a, b)
    rows = parts.float().sum(dim=0).cpu() + bias.cpu()
    want_q = plain.rope_neox(rows[:, :hq * hd].numpy(), pos.cpu().numpy(), hd, 1e6, rot, None)
    close(results[0][0], want_q, atol=3e-2, rtol=8e-3, what="q of the long prompt")
    page, slot = int(table[0, int(pos[650]) // 64]), int(pos[650]) % 64
    close(layout.get_value(results[0][2], page, slot).reshape(-1), rows[650, (hq + hkv) * hd:].to(BF16).float(),
          atol=2e-2, rtol=8e-3, what="a value row")


def test_rope_reference_vectors():
    """/root/reference/tests/core/test_nn.cpp:221-290: position 0 is the identity; with
    head size 2 and an angle of pi/2, [1,0] turns into [0,1]; pairs are (i, i+half)."""
    from sonicboom_amd import ops
    kc, vc = make_cache(1, 1, 4, F32)
    table = torch.zeros((1, 1), dtype=torch.int32, device=DEV)
    z = torch.zeros(1, dtype=torch.int32, device=DEV)
    x = torch.tensor([[0.5, -1.25, 2.0, 3.5] * 3], device=DEV)
    inv = torch.tensor([1.0, 0.01], device=DEV)
    q = ops.rope_kv_store(x, F32, inv, None, 4, z, z, kc, vc, table, 1, 1, 4)
    assert torch.equal(q.cpu(), x[:, :4].cpu())
    # angle pi/2 for both pairs at position 1: (x0, x2) -> (-x2, x0), (x1, x3) -> (-x3, x1)
    inv = torch.full((2,), math.pi / 2, device=DEV)
    one = torch.ones(1, dtype=torch.int32, device=DEV)
    x = torch.tensor([[1.0, 0.0, 2.0, 3.0] * 3], device=DEV)
    q = ops.rope_kv_store(x, F32, inv, None, 4, one, z, kc, vc, table, 1, 1, 4).cpu()
    assert torch.allclose(q, torch.tensor([[-2.0, -3.0, 1.0, 0.0]]), atol=1e-6)
    # freq_factors: a huge divisor freezes its pair (test_nn.cpp:272-289)
    ff = torch.tensor([1.0, 1e30], device=DEV)
    q = ops.rope_kv_store(x, F32, inv, ff, 4, one, z, kc, vc, table, 1, 1, 4).cpu()
    assert torch.allclose(q, torch.tensor([[-2.0, 0.0, 1.0, 3.0]]), atol=1e-5)


def fill_cache_from(keys, values, table, dtype):
    """keys/values: list per sequence of [len, hkv, hd] float tensors -> paged caches."""
    hkv, hd = keys[0].shape[1:]
    n_pages = int(table.max()) + 1
    kc, vc = make_cache(n_pages, hkv, hd, dtype)
    for s, (k, v) in enumerate(zip(keys, values)):
        for p in range(k.shape[0]):
            page = table[s, p // 64]
            layout.put_key(kc, int(page), p % 64, k[p])
            layout.put_value(vc, int(page), p % 64, v[p])
    return kc, vc


ATTN_SHAPES = [(4, 2, 16), (3, 1, 32), (5, 5, 48), (6, 2, 80), (8, 2, 128), (2, 1, 256)]


@pytest.mark.parametrize("hq, hkv, hd", ATTN_SHAPES)
@pytest.mark.parametrize("dtype", [F32, BF16])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_plain_kernel(hq, hkv, hd, dtype, window):
    from sonicboom_amd import ops
    lens = [150, 3]
    table = torch.tensor([[4, 0, 2], [1, 3, 5]], dtype=torch.int32)
    keys = [randn(n, hkv, hd, seed=s).to(dtype).float() for s, n in enumerate(lens)]
    vals = [randn(n, hkv, hd, seed=9 + s).to(dtype).float() for s, n in enumerate(lens)]
    kc, vc = fill_cache_from(keys, vals, table, dtype)
    # rows: a few positions of sequence 0 (first, page edges, last), all of sequence 1
    rows = [(0, 0), (0, 63), (0, 64), (0, 100), (0, 149), (1, 0), (1, 1), (1, 2)]
    q = randn(len(rows), hq * hd, seed=5).to(dtype)
    scale = 1.0 / math.sqrt(hd)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32)
    seq = torch.tensor([s for s, _ in rows], dtype=torch.int32)
    got = ops.attention_plain(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), seq.to(DEV), hq, hkv, hd, scale, window)
    for r, (s, p) in enumerate(rows):
        n = lens[s]
        want = plain.attention(q[r:r + 1].float().numpy(), keys[s].reshape(n, -1).numpy(),
                               vals[s].reshape(n, -1).numpy(), [p], np.arange(n), hq, hkv, hd, scale,
                               causal=True, window=window)
        tol = dict(atol=3e-6, rtol=2e-5) if dtype == F32 else dict(atol=2e-2, rtol=1e-2)
        close(got[r:r + 1], want, what=f"row {r} (seq {s}, pos {p})", **tol)


def attention_case(hq, hkv, hd, lens, rows_per_seq, window, seed=0):
    """Random bf16 keys, values and queries for sequences of ``lens`` tokens on scattered pages;
    ``rows_per_seq[s]`` lists the positions of sequence s that ask.  Returns device operands and the
    plain result per row."""
    n_seq = len(lens)
    width = max((n + 63) // 64 for n in lens)
    perm = torch.randperm(n_seq * width + 3, generator=torch.Generator().manual_seed(seed))
    table = torch.full((n_seq, width), -1, dtype=torch.int32)
    it = iter(perm.tolist())
    for s_, n in enumerate(lens):
        for pg in range((n + 63) // 64):
            table[s_, pg] = next(it)
    keys = [randn(n, hkv, hd, seed=seed + s_).to(BF16).float() for s_, n in enumerate(lens)]
    vals = [randn(n, hkv, hd, seed=seed + 50 + s_).to(BF16).float() for s_, n in enumerate(lens)]
    hkv_, hd_ = keys[0].shape[1:]
    kc, vc = make_cache(n_seq * width + 3, hkv_, hd_, BF16)
    for s_, (k, v) in enumerate(zip(keys, vals)):
        for p in range(k.shape[0]):
            page = table[s_, p // 64]
            layout.put_key(kc, int(page), p % 64, k[p])
            layout.put_value(vc, int(page), p % 64, v[p])
    rows = [(s_, p) for s_, ps in enumerate(rows_per_seq) for p in ps]
    q = randn(len(rows), hq * hd, seed=seed + 7).to(BF16)
    scale = 1.0 / math.sqrt(hd)
    want = []
    for r, (s_, p) in enumerate(rows):
        n = lens[s_]
        want.append(plain.attention(q[r:r + 1].float().numpy(), keys[s_].reshape(n, -1).numpy(),
                                    vals[s_].reshape(n, -1).numpy(), [p], np.arange(n), hq, hkv, hd, scale,
                                    causal=True, window=window))
    return q, kc, vc, table, rows, scale, np.concatenate(want, axis=0)


# (groups of 7, 5 and 8 query heads per kv head run prefill with eight waves a block: one, three
# and no wave without a head; the last shape makes a second block of one head and three such waves)
# (from (8, 2, 128) on: every wave of a block of four has a head and all waves share the loads that
# bring a page in; heads of more than 128 in blocks of eight waves: sixteen heads in two blocks,
# five heads and three waves without one, eight heads; groups of one and two heads at usual head sizes)
MFMA_SHAPES = [(4, 2, 16), (3, 1, 32), (5, 5, 48), (6, 2, 80), (28, 4, 128), (2, 1, 256), (40, 2, 64), (10, 2, 128),
               (16, 2, 64), (8, 2, 128), (4, 1, 256), (16, 1, 192), (10, 2, 160), (8, 1, 144), (3, 3, 128), (4, 2, 64),
               (12, 1, 96)]


@pytest.mark.parametrize("hq, hkv, hd", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 70])
def test_attention_decode_matrix_cores(hq, hkv, hd, window):
    """One row per sequence, lengths on both sides of page and chunk (4 pages) edges."""
    from sonicboom_amd import ops
    lens = [1, 2, 64, 65, 255, 256, 257, 700]
    q, kc, vc, table, rows, scale, want = attention_case(hq, hkv, hd, lens, [[n - 1] for n in lens], window)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32)
    got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
    close(got, want, atol=1.5e-2, rtol=1e-2, what="decode")
    for _ in range(3):                       # launch after launch, the same bits
        again = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
        assert torch.equal(got, again)


@pytest.mark.parametrize("window", [0, 100])
@pytest.mark.parametrize("longest", [300, 900])
def test_attention_decode_matrix_cores_many_sequences(window, longest):
    """Two hundred sequences: a block for every CU without cutting the rows, so each block takes
    its row whole (one chunk, a quarter of the table's width per wave, no merge kernel); lengths
    from one key to many pages, with and without a window."""
    from sonicboom_amd import ops
    hq, hkv, hd = 8, 4, 32
    rng = np.random.default_rng(5)
    lens = [int(n) for n in rng.integers(1, longest, size=200)]
    lens[:4] = [1, 64, 65, longest]
    q, kc, vc, table, rows, scale, want = attention_case(hq, hkv, hd, lens, [[n - 1] for n in lens], window, seed=9)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32)
    got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
    close(got, want, atol=1.5e-2, rtol=1e-2, what="decode, 200 sequences")


@pytest.mark.parametrize("window", [0, 300])
@pytest.mark.parametrize("n_seqs, longest", [(30, 2000), (12, 5000), (3, 9000), (70, 1500)])
def test_attention_decode_matrix_cores_long_rows_of_unequal_length(window, n_seqs, longest):
    """Rows long enough for the launcher to deal several pages to a wave and cut the rows into
    chunks of its own choosing; lengths from one key to thousands in one batch, so that chunks
    are full, partly filled and empty side by side.  (70 sequences on 4 kv heads: a few blocks
    more than the GPU has CUs, for which the launcher takes smaller chunks.)"""
    from sonicboom_amd import ops
    hq, hkv, hd = 8, 4, 64
    rng = np.random.default_rng(n_seqs)
    lens = [int(n) for n in rng.integers(1, longest, size=n_seqs)]
    lens[0], lens[-1] = longest, 1
    q, kc, vc, table, rows, scale, want = attention_case(hq, hkv, hd, lens, [[n - 1] for n in lens], window, seed=21)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32)
    got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
    close(got, want, atol=1.5e-2, rtol=1e-2, what=f"decode, {n_seqs} rows up to {longest} keys")


@pytest.mark.parametrize("hq, hkv, hd", [(4, 2, 16), (5, 5, 48), (6, 2, 80), (28, 4, 128), (40, 2, 64)])
@pytest.mark.parametrize("window", [0, 70, 1000])
@pytest.mark.parametrize("pages", [1, 2, 4, 8])
def test_attention_decode_pages_per_wave(hq, hkv, hd, window, pages):
    """Every way of dealing pages to waves (one page each, or 2, 4, 8 in a row with the next half
    page in flight), on lengths around page, wave and chunk edges, a long row, a window that
    starts inside a later chunk, and a table with a hole: a page number outside the cache in a
    page that the window has left behind."""
    from sonicboom_amd import ops
    lens = [1, 64, 65, 129, 256, 257, 513, 700, 2100]
    q, kc, vc, table, rows, scale, want = attention_case(hq, hkv, hd, lens, [[n - 1] for n in lens], window, seed=4)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32)
    if window:
        table[-1, 0] = -1                     # the cache gives such pages back
        table[-1, 1] = kc.shape[0] + 5
    with ops.attention_decode_pages_per_wave(hd, pages):
        got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
        close(got, want, atol=1.5e-2, rtol=1e-2, what=f"decode, {pages} pages per wave")
        again = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
        assert torch.equal(got, again)


@pytest.mark.parametrize("hq, hkv, hd", MFMA_SHAPES)
@pytest.mark.parametrize("window", [0, 70])
def test_attention_prefill_matrix_cores(hq, hkv, hd, window):
    """Whole prompts of unequal lengths, and a continuation on top of cached keys."""
    from sonicboom_amd import ops
    lens = [1, 17, 64, 150, 200]
    starts = [0, 0, 0, 0, 120]           # the last sequence has 120 keys cached and brings 80 rows
    rows_per_seq = [list(range(s0, n)) for s0, n in zip(starts, lens)]
    q, kc, vc, table, rows, scale, want = attention_case(hq, hkv, hd, lens, rows_per_seq, window, seed=3)
    pos = torch.tensor([p for _, p in rows], dtype=torch.int32)
    # tiles of 16 rows, of the height that suits the group (64 and 32 rows for groups of one and two
    # heads), and of 32 rows where the kernel has its form for long prompts
    for height in sorted({16, ops.attention_row_tile(hq, hkv, hd)} | ({32} if ops.attention_tall_ok(hq, hkv, hd) else set())):
        tiles, row0 = [], 0
        for s_, ps in enumerate(rows_per_seq):
            for r0 in range(0, len(ps), height):
                tiles.append((row0 + r0, min(height, len(ps) - r0), s_, 0))
            row0 += len(ps)
        tiles = torch.tensor(tiles, dtype=torch.int32)
        got = ops.attention_prefill_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), tiles.to(DEV), hq, hkv, hd,
                                         scale, window, tile_rows=height)
        close(got, want, atol=1.5e-2, rtol=1e-2, what=f"prefill, tiles of {height} rows")
    assert ops.attention_row_tile(hq, hkv, hd) == (64 if hq == hkv else 32 if hq == 2 * hkv else 16)
    assert ops.attention_tall_ok(hq, hkv, hd) == (hq >= 3 * hkv and hd % 32 == 0 and hd <= 128)
    assert ops.attention_row_tiles(hq, hkv, hd) == ((16, 32) if ops.attention_tall_ok(hq, hkv, hd)
                                                    else (ops.attention_row_tile(hq, hkv, hd),))
    if hq > 2 * hkv:
        with pytest.raises(ops.KernelLibraryError, match="do not suit"):
            ops.attention_prefill_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), tiles.to(DEV), hq, hkv, hd,
                                       scale, window, tile_rows=64)


def test_attention_reference_vectors():
    """/root/reference/tests/core/test_nn.cpp:402-495: one key copies its value; causal
    2x2 gives [2, 3]; GQA maps 4 query heads onto 2 kv heads; window 2 drops key 0;
    scale 1 and 0.5 give 1.0360 and 1.2384."""
    from sonicboom_amd import ops

    def run(q, k, v, hq, hkv, hd, scale, window=0):
        n = len(k)
        keys = [torch.tensor(k, dtype=F32).reshape(n, hkv, hd)]
        vals = [torch.tensor(v, dtype=F32).reshape(n, hkv, hd)]
        table = torch.zeros((1, 1), dtype=torch.int32)
        # pad the head to the kernels' smallest size by zero columns: scores are unchanged
        kc, vc = fill_cache_from(keys, vals, table, F32)
        qt = torch.tensor(q, dtype=F32).reshape(-1, hq * hd)
        pos = torch.arange(qt.shape[0], dtype=torch.int32)
        seq = torch.zeros(qt.shape[0], dtype=torch.int32)
        return ops.attention_plain(qt.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), seq.to(DEV), hq, hkv, hd,
                                   scale, window).cpu()

    assert torch.allclose(run([[1.0, 0, 0, 0]], [[1.0, 0, 0, 0]], [[1.0, 2, 3, 4]], 1, 1, 4, 1.0),
                          torch.tensor([[1.0, 2, 3, 4]]), atol=1e-6)
    out = run([[1.0], [1.0]], [[1.0], [1.0]], [[2.0], [4.0]], 1, 1, 1, 1.0)
    assert torch.allclose(out.flatten(), torch.tensor([2.0, 3.0]), atol=1e-6)
    out = run([[1.0, 1, 1, 1]], [[1.0, 1.0]], [[1.0, 2.0]], 4, 2, 1, 1.0)
    assert torch.allclose(out.flatten(), torch.tensor([1.0, 1.0, 2.0, 2.0]), atol=1e-6)
    out = run([[1.0], [1.0], [1.0]], [[1.0], [1.0], [1.0]], [[1.0], [2.0], [4.0]], 1, 1, 1, 1.0, window=2)
    assert abs(out[2, 0].item() - 3.0) < 1e-6
    # q = 2 at the position of the second key; keys [2, 0], values [1, 3]
    for scale, want in ((1.0, 1.0360), (0.5, 1.2384)):
        out = run([[0.0], [2.0]], [[2.0], [0.0]], [[1.0], [3.0]], 1, 1, 1, scale)
        assert abs(out[1, 0].item() - want) < 1e-3


def test_a_far_key_among_hundreds_is_found():
    """One key far back is made to dominate: the output must be its value, whatever page it is on."""
    from sonicboom_amd import ops
    hq, hkv, hd, n = 4, 2, 32, 700
    keys = [randn(n, hkv, hd, scale=0.1)]
    vals = [randn(n, hkv, hd, seed=2)]
    q = randn(1, hq * hd, seed=4)
    table = torch.tensor([list(reversed(range(11)))], dtype=torch.int32)
    for far in (0, 63, 64, 389, 699):
        k = [keys[0].clone()]
        for h in range(hq):
            k[0][far, h // 2] = q[0, h * hd:(h + 1) * hd] * 40.0 if h % 2 == 0 else k[0][far, h // 2]
        kc, vc = fill_cache_from(k, vals, table, F32)
        out = ops.attention_plain(q.to(DEV), kc, vc, table.to(DEV), torch.tensor([n - 1], dtype=torch.int32, device=DEV),
                                  torch.zeros(1, dtype=torch.int32, device=DEV), hq, hkv, hd, 1.0, 0).cpu()
        for h in (0, 2):
            assert torch.allclose(out[0, h * hd:(h + 1) * hd], vals[0][far, h // 2], atol=1e-4), (far, h)


@pytest.mark.parametrize("hq, hkv, hd", [(14, 2, 128), (4, 2, 64), (3, 1, 32)])
@pytest.mark.parametrize("shape", ["climbing", "falling", "far key"])
def test_attention_matrix_cores_when_the_maximum_moves(hq, hkv, hd, shape):
    """Scores made to climb page after page (the running maximum has to follow, in steps), to
    fall from the first key on (it never moves again), or to peak at one key far back among
    hundreds of small ones: prefill rows and decode rows against the plain softmax."""
    from sonicboom_amd import ops
    n, group = 600, hq // hkv
    scale = 1.0 / math.sqrt(hd)
    keys = randn(n, hkv, hd, scale=0.05, seed=11)
    vals = randn(n, hkv, hd, seed=12)
    rows_pos = list(range(552, 600))                 # 552 keys cached, 48 rows asking
    q = randn(len(rows_pos), hq * hd, scale=0.05, seed=13)
    q.view(len(rows_pos), hq, hd)[:, :, 0] = 8.0      # every head looks along coordinate 0
    ramp = torch.arange(n, dtype=torch.float32) / n   # 0 .. 1 over the sequence
    rise = 56.0 / (8.0 * scale)                       # scores span about 56 (81 in log2 units)
    if shape == "climbing":
        keys[:, :, 0] = (ramp * rise)[:, None]
    elif shape == "falling":
        keys[:, :, 0] = ((1.0 - ramp) * rise)[:, None]
    else:
        keys[389, :, 0] = rise
    keys, vals, q = keys.to(BF16).float(), vals.to(BF16).float(), q.to(BF16)
    table = torch.tensor([[7, 2, 9, 4, 0, 5, 1, 8, 3, 6]], dtype=torch.int32)
    kc, vc = fill_cache_from([keys], [vals], table, BF16)
    want = plain.attention(q.float().numpy(), keys.reshape(n, -1).numpy(), vals.reshape(n, -1).numpy(), rows_pos,
                           np.arange(n), hq, hkv, hd, scale, causal=True, window=0)
    pos = torch.tensor(rows_pos, dtype=torch.int32)
    for height in (16, 32) if ops.attention_tall_ok(hq, hkv, hd) else (16,):
        tiles = torch.tensor([(r0, min(height, len(rows_pos) - r0), 0, 0) for r0 in range(0, len(rows_pos), height)],
                             dtype=torch.int32)
        got = ops.attention_prefill_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), tiles.to(DEV), hq, hkv, hd,
                                         scale, 0, tile_rows=height)
        close(got, want, atol=1.5e-2, rtol=1e-2, what=f"prefill, {shape}, tiles of {height}")
    # the same rows as single decode rows of sequences that share the pages
    for r in (0, 17, 47):
        got1 = ops.attention_decode_mfma(q[r:r + 1].to(DEV), kc, vc, table.to(DEV), pos[r:r + 1].to(DEV), hq, hkv,
                                         hd, scale, 0)
        close(got1, want[r:r + 1], atol=1.5e-2, rtol=1e-2, what=f"decode row {r}, {shape}")
    if shape == "far key":
        # the far key takes all the weight: the output is its value
        v_far = vals[389].repeat_interleave(group, dim=0).reshape(1, -1)
        close(got[-1:], v_far.numpy(), atol=2e-2, rtol=1e-2, what="far key's value")


def _looking_along_zero(n, hq, hkv, hd, n_rows, seed):
    """Small random keys and queries whose coordinate 0 is large in the queries: a key whose
    coordinate 0 is raised takes all of a row's weight.  Returns keys, values, queries, the raise
    that puts one score 56 above the rest, and the scale."""
    scale = 1.0 / math.sqrt(hd)
    keys = randn(n, hkv, hd, scale=0.05, seed=seed)
    vals = randn(n, hkv, hd, seed=seed + 1)
    q = randn(n_rows, hq * hd, scale=0.05, seed=seed + 2)
    q.view(n_rows, hq, hd)[:, :, 0] = 8.0
    return keys.to(BF16).float(), vals.to(BF16).float(), q.to(BF16), 56.0 / (8.0 * scale), scale


@pytest.mark.parametrize("pages", [0, 1, 2, 4, 8])
def test_attention_decode_one_dominant_key_in_each_chunk(pages):
    """A row of 6,500 keys is cut into chunks of 4 x ``pages`` pages whose partial results a
    second kernel merges.  One key at a time is made to dominate: the first key of all, the first
    and last key of a wave's run of pages in a middle chunk, the first key of the second and of
    the last chunk, the row's own key and the one before it.  The output must be that key's
    value: a chunk or a wave's run that is dropped, merged twice or weighted wrongly shows at
    once, where random keys would move the output by less than the tolerance."""
    from sonicboom_amd import ops
    hq, hkv, hd, n = 8, 2, 64, 6500
    keys, vals, q, rise, scale = _looking_along_zero(n, hq, hkv, hd, 1, seed=31)
    width = (n + 63) // 64
    table = torch.randperm(width + 5, generator=torch.Generator().manual_seed(3))[:width].to(torch.int32)[None, :]
    kc, vc = fill_cache_from([keys], [vals], table, BF16)
    pos = torch.tensor([n - 1], dtype=torch.int32, device=DEV)
    run = max(pages, 1)                    # pages of a wave's run; a chunk is four runs
    last_chunk = ((n - 1) // 64 // (4 * run)) * 4 * run * 64
    spots = sorted({0, 4 * run * 64, (4 * run + 2 * run) * 64, (4 * run + 2 * run) * 64 - 1,
                    (4 * run + run) * 64 - 1, last_chunk, last_chunk - 1, n - 2, n - 1})
    group = hq // hkv
    with ops.attention_decode_pages_per_wave(hd, pages):
        for far in spots:
            page, slot = int(table[0, far // 64]), far % 64
            at = int(layout.key_positions(hd)[slot, 0])          # where element 0 of that key lies
            before = kc[page, :, slot, at].clone()
            kc[page, :, slot, at] = rise
            got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos, hq, hkv, hd, scale, 0)
            kc[page, :, slot, at] = before
            want = vals[far].repeat_interleave(group, dim=0).reshape(1, -1)
            close(got, want.numpy(), atol=2e-2, rtol=1e-2, what=f"dominant key at {far}, {pages} pages per wave")


@pytest.mark.parametrize("window", [70, 200, 1000])
@pytest.mark.parametrize("pages", [0, 1, 2, 8])
def test_attention_decode_window_edge(window, pages):
    """The lower edge of the window, to the key: a dominant key at position - window is out of
    the window and must count for nothing; at position - window + 1 it is the window's first key
    and must take all the weight.  On random data the keys before the edge are valid cache
    contents, and one key too many moves the output by less than the tolerance."""
    from sonicboom_amd import ops
    hq, hkv, hd, n = 6, 2, 64, 1500
    keys, vals, q, rise, scale = _looking_along_zero(n, hq, hkv, hd, 1, seed=41)
    table = torch.arange((n + 63) // 64, dtype=torch.int32).flip(0)[None, :].contiguous()
    group = hq // hkv
    for p in (n - 1, 1030, 1024 + window - 1):          # the edge inside a page, and on a page's first key
        p = min(p, n - 1)
        for inside in (False, True):
            k = keys.clone()
            edge = p - window + (1 if inside else 0)
            k[edge, :, 0] = rise
            kc, vc = fill_cache_from([k], [vals], table, BF16)
            pos = torch.tensor([p], dtype=torch.int32, device=DEV)
            with ops.attention_decode_pages_per_wave(hd, pages):
                got = ops.attention_decode_mfma(q.to(DEV), kc, vc, table.to(DEV), pos, hq, hkv, hd, scale, window)
            if inside:
                want = vals[edge].repeat_interleave(group, dim=0).reshape(1, -1).numpy()
            else:
                want = plain.attention(q.float().numpy(), k.reshape(n, -1).numpy(), vals.reshape(n, -1).numpy(), [p],
                                       np.arange(n), hq, hkv, hd, scale, causal=True, window=window)
                assert np.abs(want - vals[edge].repeat_interleave(group, dim=0).reshape(1, -1).numpy()).max() > 0.5
            close(got, want, atol=2e-2, rtol=1e-2, what=f"position {p}, window {window}, key {edge}")


@pytest.mark.parametrize("hq, hkv, hd", [(6, 2, 64), (28, 4, 128), (3, 1, 32)])
@pytest.mark.parametrize("window", [70, 300])
def test_attention_prefill_window_edge(hq, hkv, hd, window):
    """Prompt rows over a window: one dominant key at position d.  Rows up to d + window - 1
    have it as a key of their window (the last of them as its very first key) and must return
    its value; from row d + window on it has left the window and must count for nothing."""
    from sonicboom_amd import ops
    n = 700
    rows_pos = list(range(n - 80, n))
    keys, vals, q, rise, scale = _looking_along_zero(n, hq, hkv, hd, len(rows_pos), seed=51)
    group = hq // hkv
    table = torch.tensor([[7, 2, 9, 4, 0, 5, 1, 8, 3, 6, 10]], dtype=torch.int32)
    pos = torch.tensor(rows_pos, dtype=torch.int32)
    heights = (16, 32) if ops.attention_tall_ok(hq, hkv, hd) else (16,)
    # inside a tile of 16, at its end, at its start; at the end of a tile of 32, at its start
    for last_seeing in (rows_pos[0] + 20, rows_pos[0] + 47, rows_pos[0] + 48, rows_pos[0] + 63, rows_pos[0] + 64):
        d = last_seeing - window + 1
        k = keys.clone()
        k[d, :, 0] = rise
        kc, vc = fill_cache_from([k], [vals], table, BF16)
        want = plain.attention(q.float().numpy(), k.reshape(n, -1).numpy(), vals.reshape(n, -1).numpy(), rows_pos,
                               np.arange(n), hq, hkv, hd, scale, causal=True, window=window)
        v_d = vals[d].repeat_interleave(group, dim=0).reshape(1, -1).numpy()
        r = last_seeing - rows_pos[0]
        assert np.abs(want[r] - v_d).max() < 2e-2 and np.abs(want[r + 1] - v_d).max() > 0.5     # the case is sharp
        for height in heights:
            tiles = torch.tensor([(r0, min(height, len(rows_pos) - r0), 0, 0) for r0 in range(0, len(rows_pos), height)],
                                 dtype=torch.int32)
            got = ops.attention_prefill_mfma(q.to(DEV), kc, vc, table.to(DEV), pos.to(DEV), tiles.to(DEV), hq, hkv, hd,
                                             scale, window, tile_rows=height)
            close(got, want, atol=2e-2, rtol=1e-2, what=f"window {window}, dominant key {d}, tiles of {height}")


FOLDED_SHAPES = [(4, 2, 16, 16), (3, 1, 32, 32), (5, 5, 48, 16), (6, 2, 80, 64), (28, 4, 128, 128), (16, 1, 64, 0),
                 (2, 1, 256, 256)]


@pytest.mark.parametrize("hq, hkv, hd, rot, pages", [(*sh, p) for sh in FOLDED_SHAPES for p in (0, 1, 2, 8)
                                                     if p <= 1 or sh[2] <= 128])     # several pages per wave: up to head size 128
@pytest.mark.parametrize("window", [0, 70])
def test_attention_decode_with_rotation_and_store_folded_in(hq, hkv, hd, rot, window, pages):
    """A decode step's rotation, store and attention in one kernel against the two kernels one
    after the other: the same output and the same cache, bit for bit.  The qkv rows come as one
    array and as three K slices with a bias; rows stand at a page's first and last slot, on the
    first token of a sequence, and behind a window; one row has no page at all (a row added to
    fill a batch: nothing is stored, nothing seen)."""
    from sonicboom_amd import ops
    lens = [1, 64, 65, 128, 300, 700, 1]          # the row is the sequence's last token
    n_seq = len(lens)
    width_pages = max((n + 63) // 64 for n in lens)
    perm = torch.randperm(n_seq * width_pages + 3, generator=torch.Generator().manual_seed(5))
    table = torch.full((n_seq, width_pages), -1, dtype=torch.int32)
    it = iter(perm.tolist())
    for s_, n in enumerate(lens[:-1]):            # the last sequence keeps a table of -1
        for pg in range((n + 63) // 64):
            table[s_, pg] = next(it)
    n_pages = n_seq * width_pages + 3
    kc0 = randn(n_pages, hkv, 64, hd, seed=1).to(BF16)
    vc0 = randn(n_pages, hkv, hd, 64, seed=2).to(BF16)
    pos = torch.tensor([n - 1 for n in lens], dtype=torch.int32)
    pos[-1] = 0
    seq = torch.arange(n_seq, dtype=torch.int32)
    width = (hq + 2 * hkv) * hd
    inv = ff = None
    if rot:
        inv = torch.exp(-2.0 * torch.arange(rot // 2, dtype=F32) / rot * math.log(1e4)).to(DEV)
        ff = (1.0 + torch.arange(rot // 2, dtype=F32) / rot).to(DEV)
    scale = 1.0 / math.sqrt(hd)
    for n_slices in (1, 3):
        qkv = randn(n_slices, n_seq, width, seed=3 + n_slices).to(DEV)
        bias = randn(width, seed=9, scale=0.3).to(DEV) if n_slices > 1 else None
        arg = qkv if n_slices > 1 else qkv[0].contiguous()
        # two kernels
        kc1, vc1 = kc0.clone().to(DEV), vc0.clone().to(DEV)
        q = ops.rope_kv_store(arg, BF16, inv, ff, rot, pos.to(DEV), seq.to(DEV), kc1, vc1, table.to(DEV), hq, hkv, hd,
                              bias=bias)
        with ops.attention_decode_pages_per_wave(hd, pages):
            want = ops.attention_decode_mfma(q, kc1, vc1, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale, window)
            # one kernel
            kc2, vc2 = kc0.clone().to(DEV), vc0.clone().to(DEV)
            assert ops.attention_decode_rope_ok(arg, BF16, BF16, hq, hkv, hd, rot)
            got = ops.attention_decode_rope(arg, inv, ff, rot, kc2, vc2, table.to(DEV), pos.to(DEV), hq, hkv, hd, scale,
                                            window, bias=bias)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"slices {n_slices}"
            assert torch.equal(kc2.view(torch.int16), kc1.view(torch.int16))
            assert torch.equal(vc2.view(torch.int16), vc1.view(torch.int16))
            assert not torch.equal(kc2.view(torch.int16), kc0.to(DEV).view(torch.int16))     # something was stored
            # queries only (a layer that reads another layer's cache): nothing is stored
            kc3, vc3 = kc1.clone(), vc1.clone()
            only_q = arg[..., : hq * hd].contiguous()
            got = ops.attention_decode_rope(only_q, inv, ff, rot, kc3, vc3, table.to(DEV), pos.to(DEV), hq, hkv, hd,
                                            scale, window, bias=bias, store=False)
            assert torch.equal(got.view(torch.int16), want.view(torch.int16))
            assert torch.equal(kc3.view(torch.int16), kc1.view(torch.int16))
    assert not ops.attention_decode_rope_ok(arg, BF16, BF16, 34, 2, hd, rot)          # 17 heads per kv head


@pytest.mark.parametrize("vocab", [5, 256, 1000, 152064])
def test_argmax_first_maximum(vocab):
    from sonicboom_amd import ops
    x = randn(6, vocab)
    x[0, :] = 0.5                                   # all equal: id 0
    x[1, vocab - 1] = 50.0
    x[2, 3] = 60.0
    if vocab > 4:
        x[2, 4] = 60.0                              # a tie: the lower id
    x[3, :] = float("-inf")
    got = ops.argmax(x.to(DEV)).cpu().tolist()
    want = [plain.argmax(r.numpy()) for r in x]
    assert got == want and got[:3] == [0, vocab - 1, 3]


@pytest.mark.parametrize("vocab", [7, 256, 300, 5000, 8192, 8193, 12289, 152064])
@pytest.mark.parametrize("temperature", [1.0, 0.7])
def test_top_candidates(vocab, temperature):
    """Rows short enough for one block, and rows cut into parts of 4,096 whose best are merged
    (from 8,193 on; a last part of one element; a part that holds all of the best)."""
    from sonicboom_amd import ops
    x = randn(6, vocab, scale=2.0)
    x[1] = torch.round(x[1])                        # many ties: ordered by id
    x[2, :] = 1.25                                  # all equal
    x[3, ::3] = -0.0
    x[3, 1::3] = 0.0                                # signed zeros are one value
    x[4, vocab // 3:] = -float("inf")               # fewer finite values than candidates, perhaps
    x[5, -min(300, vocab):] += 50.0                 # all of the best at the row's end
    k = min(256, vocab)
    ids, z = ops.top_candidates(x.to(DEV), temperature, k)
    ids, z = ids.cpu().numpy(), z.cpu().numpy()
    for r in range(6):
        want = sampling_plain.select_candidates(x[r].numpy(), temperature)
        assert [c[0] for c in want] == ids[r].tolist(), f"row {r}"
        assert np.array_equal(np.array([c[1] for c in want], dtype=np.float32), z[r]), f"row {r}"


@pytest.mark.parametrize("params", [
    dict(temperature=0.8), dict(temperature=1.3, top_k=5), dict(temperature=0.5, top_p=0.7),
    dict(temperature=1.0, min_p=0.2), dict(temperature=0.9, top_k=40, top_p=0.9, min_p=0.01),
    dict(temperature=0.05, top_p=0.5), dict(temperature=2.0, top_k=1), dict(temperature=1.0, top_p=1e-9, min_p=1.0),
    dict(temperature=1.0, top_k=300, top_p=0.999),
])
@pytest.mark.parametrize("vocab", [40, 400, 5000])
def test_draw_equals_the_plain_sampler(params, vocab):
    """Filters and Gumbel draw on the device, a wave a row: every row gets the token that the
    plain sampler draws for it alone (flat and peaked rows, ties among the best, one candidate far
    above the window, positions past 2^32, a 64-bit seed, fewer logits than candidates)."""
    from sonicboom_amd import ops
    SP = sampling_plain
    r = np.random.default_rng(vocab)
    rows = []
    for i in range(96):
        logits = (r.standard_normal(vocab) * (0.2 if i % 5 == 0 else 3.0)).astype(np.float32)
        if i % 7 == 3:
            logits[10:20] = logits[5]
        if i % 6 == 1:
            logits[3] = 80.0
        rows.append(logits)
    positions = [int(q) for q in r.integers(0, 5000, size=len(rows))]
    positions[0], positions[1] = 0, 2 ** 33 + 5
    seed = 0x9E3779B97F4A7C15
    t = params["temperature"]
    k = min(ops.MAX_CANDIDATES, vocab)
    ids, z = ops.top_candidates(torch.tensor(np.stack(rows), device=DEV), t, k)
    log_min_p = float(np.log(np.float32(params["min_p"]))) if params.get("min_p", 0.0) > 0.0 else None
    top_p = float(np.float64(np.float32(params["top_p"]))) if 0.0 < params.get("top_p", 1.0) < 1.0 else None
    got = ops.draw(ids, z, positions, params.get("top_k", 0), log_min_p, top_p, seed).tolist()
    for i, logits in enumerate(rows):
        kept = SP.filter_candidates(SP.select_candidates(logits, t), params.get("top_k", 0),
                                    params.get("top_p", 1.0), params.get("min_p", 0.0))
        assert got[i] == SP.draw(kept, seed, positions[i]), f"row {i}"


def test_draw_at_the_positions_after_device_side_lengths():
    """Lengths as a decode step keeps them on the device (int32): the new token's position is
    length + 1, and the tokens are those of the same positions brought from the host."""
    from sonicboom_amd import ops
    r = np.random.default_rng(3)
    logits = torch.tensor((r.standard_normal((40, 3000)) * 2.0).astype(np.float32), device=DEV)
    ids, z = ops.top_candidates(logits, 0.9, ops.MAX_CANDIDATES)
    lengths = [int(q) for q in r.integers(0, 4000, size=40)]
    want = ops.draw(ids, z, [n + 1 for n in lengths], 50, None, 0.9, 12345).tolist()
    out = torch.full((40,), -7, dtype=torch.int32, device=DEV)
    got = ops.draw(ids, z, torch.tensor(lengths, dtype=torch.int32, device=DEV), 50, None, 0.9, 12345, out=out)
    assert got is out and out.tolist() == want
    assert ops.draw(ids, z, lengths, 50, None, 0.9, 12345).tolist() != want       # other positions, other draws


def test_draw_keeps_no_candidate_of_an_empty_row():
    """A row whose candidates all lie outside (ids of -1, as a row shorter than k is filled)
    gives -1; its neighbours are not disturbed."""
    from sonicboom_amd import ops
    ids = torch.tensor([[3, 1, -1, -1], [-1, -1, -1, -1]], dtype=torch.int32, device=DEV)
    z = torch.tensor([[2.0, 1.0, 0.0, 0.0], [0.0, 0.0, 0.0, 0.0]], dtype=torch.float32, device=DEV)
    got = ops.draw(ids, z, [5, 6], 0, None, None, 1).tolist()
    assert got[0] in (3, 1) and got[1] == -1


@pytest.mark.parametrize("exact", [False, True])
def test_penalize(exact):
    from sonicboom_amd import ops
    logits = randn(3, 50)
    hist = [[1, 2, 2, 49], [], [7] * 10]
    rows, toks, counts = [0, 0, 0, 2], [1, 2, 49, 7], [1, 2, 1, 10]
    dev = logits.to(DEV)
    ops.penalize(dev, *(torch.tensor(v, dtype=torch.int32, device=DEV) for v in (rows, toks, counts)),
                 1.3, 0.2, 0.1, exact)
    for r in range(3):
        want = sampling_plain.penalize(logits[r].numpy(), exact, 1.3, 64, 0.2, 0.1, hist[r])
        assert np.array_equal(dev[r].cpu().numpy(), want), f"row {r}"

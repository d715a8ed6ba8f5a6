"""nn.SpatialConvolutionMM on small-integer inputs, where every fp32 sum is exact and the comparison with the
CPU oracle is therefore bit for bit whatever order either side adds in.

The tolerance tests cannot see a fault of the size of a few mis-counted terms in a long reduction (the bound
1e-4*sqrt(B*N) of a gradWeight product is 6 % for the first AlexNet layer).  These can: the shapes reach the tiled
MFMA kernels with the reduction batched over images (gradWeight), with per-image reduction lengths N that are not
multiples of the 16-wide reduction step (169, 729, 3025: the last step of every image is partial and is moved
back, its already-covered part masked), with row and column counts ragged against every tile, unsplit and split,
on the column route and on the gathered route.  The per-kernel timing labels say which kernel, tile and split ran.
"""
import functools
import zlib

import numpy as np
import pytest

from helpers import rng_for, uniform

pytestmark = pytest.mark.gpu

import oracle  # noqa: E402

TILES = {"128x128": (128, 128), "192x128": (192, 128), "64x256": (64, 256), "128x256": (128, 256),
         "256x128": (256, 128), "64x64": (64, 64), "64x128": (64, 128), "96x128": (96, 128)}

SHAPES = {
    # name: B, C, H, W, M, kH, kW, pH, pW, sH, sW
    "first_layer_N3025": (4, 3, 224, 224, 64, 11, 11, 2, 2, 4, 4),     # N = 3025 = 189*16 + 1, K = 363, M = 64
    "second_layer_N729": (3, 64, 27, 27, 192, 5, 5, 2, 2, 1, 1),      # N = 729 = 45*16 + 9, K = 1600
    "third_layer_N169": (5, 192, 13, 13, 384, 3, 3, 1, 1, 1, 1),      # N = 169 = 10*16 + 9, K = 1728
    "ragged_M200_K630_N195": (3, 70, 15, 13, 200, 3, 3, 1, 1, 1, 1),  # nothing a multiple of any tile
    "ragged_M130_K1188_N100": (7, 132, 12, 12, 130, 3, 3, 0, 0, 1, 1),
    "strided_M257_K588_N221": (2, 12, 40, 51, 257, 7, 7, 3, 3, 3, 3),
    "first_layer_M96_N225": (3, 3, 70, 70, 96, 11, 11, 0, 0, 4, 4),    # 96 rows: the tile of 96 to 127 rows
    "ragged_M110_K225_N144": (2, 25, 14, 14, 110, 3, 3, 0, 0, 1, 1),   # ... with an edge tile shifted back
}


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


@functools.lru_cache(maxsize=None)
def case(name):
    """Integer-valued inputs of a shape and the oracle's results (the host BLAS does the oracle's sgemm: on these
    inputs every order of summation gives the same floats, so it is the plain loops' result too)."""
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = SHAPES[name]
    K = C * kH * kW
    rng = rng_for(zlib.crc32(name.encode()) % 1000 + 81)
    ints = lambda lo, hi, shape: rng.integers(lo, hi + 1, size=shape).astype(np.float32)
    x, w, b = ints(-2, 2, (B, C, H, W)), ints(-2, 2, (M, K)), ints(-3, 3, (M,))
    geo = (kH, kW, pH, pW, sH, sW)
    oracle.use_blas(True)
    try:
        out, finput = oracle.conv_updateOutput(x, w, b, *geo)
        go = ints(-2, 2, out.shape)
        gi, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
        gw0, gb0 = ints(-5, 5, (M, K)), ints(-5, 5, (M,))
        gw, gb = gw0.copy(), gb0.copy()
        oracle.conv_accGradParameters(go, finput, gw, gb, 2.0)
    finally:
        oracle.use_blas(False)
    # the products are integers below 2^24 in magnitude: exact in fp32, so the oracle's own rounding plays no part
    assert max(np.abs(out).max(), np.abs(gi).max(), np.abs(gw).max(), np.abs(gb).max()) < 2 ** 24
    n0 = 3
    assert np.array_equal(out[0, :n0].astype(np.int64), brute_output(x[0], w[:n0], b[:n0], geo))
    return x, w, b, go, gw0, gb0, out, gi, gw, gb


def brute_output(x, w, b, geo):
    """The first output planes of one image from the convolution's definition, in int64 (independent of the oracle)."""
    kH, kW, pH, pW, sH, sW = geo
    C, H, W = x.shape
    xp = np.pad(x.astype(np.int64), [(0, 0), (pH, pH), (pW, pW)])
    Ho, Wo = (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1
    wk = w.astype(np.int64).reshape(w.shape[0], C, kH, kW)
    out = np.zeros((w.shape[0], Ho, Wo), np.int64)
    for kh in range(kH):
        for kw in range(kW):
            patch = xp[:, kh:kh + (Ho - 1) * sH + 1:sH, kw:kw + (Wo - 1) * sW + 1:sW]
            out += np.einsum("mc,chw->mhw", wk[:, :, kh, kw], patch)
    return out + b.astype(np.int64)[:, None, None]


def run(gt, name, mode):
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = SHAPES[name]
    x, w, b, go, gw0, gb0, out, gi, gw, gb = case(name)
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0
    try:
        m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
        m._assign("weight", w)
        m._assign("bias", b)
        m.gradWeight[...] = gw0
        m.gradBias[...] = gb0
        m.gpu()
        dx, dgo = dev(gt, x), dev(gt, go)
        gt.gputorch.synchronize()
        gt.gputorch.prof_reset()
        gt.gputorch.prof_enable(True)
        try:
            got_out = m.forward(dx).float()
            got_gi = m.updateGradInput(dx, dgo).float()
            m.accGradParameters(dx, dgo, 2.0)
            gt.gputorch.synchronize()
            labels = sorted(k for k in gt.gputorch.prof_report() if k.startswith("gemm_conv"))
        finally:
            gt.gputorch.prof_enable(False)
            gt.gputorch.prof_reset()
        got_gw, got_gb = m.gradWeight.float(), m.gradBias.float()
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0
    assert np.array_equal(got_out, out), "output"
    assert np.array_equal(got_gi, gi), "gradInput"
    assert np.array_equal(got_gw, gw), "gradWeight"
    assert np.array_equal(got_gb, gb), "gradBias"
    return {l.split(" ")[0]: l for l in labels}


@pytest.mark.parametrize("mode", [0, 2], ids=["columns", "gathered"])
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_integer_conv_exact_library_choice(gt, name, mode):
    labels = run(gt, name, mode)
    print(name, mode, labels, flush=True)
    assert "generic" not in labels["gemm_conv_gradweight"], labels   # these shapes are meant for the tiled kernels


@pytest.mark.parametrize("split", [1, 2, 5])
@pytest.mark.parametrize("tile", sorted(TILES))
@pytest.mark.parametrize("mode", [0, 2], ids=["columns", "gathered"])
@pytest.mark.parametrize("name", sorted(SHAPES))
def test_integer_conv_exact_every_tile_and_split(gt, name, mode, tile, split, switches):
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = SHAPES[name]
    K = C * kH * kW
    bm, bn = TILES[tile]
    if M < bm or K < bn:
        pytest.skip("the gradWeight product (%d x %d) is smaller than the tile" % (M, K))
    switches("gemm_tile", tile)
    switches("gemm_split", split)
    labels = run(gt, name, mode)
    gw_label = labels["gemm_conv_gradweight"]
    assert "tile=%s " % tile in gw_label, labels          # the reduction-batched kernel of this tile ran
    N = ((H + 2 * pH - kH) // sH + 1) * ((W + 2 * pW - kW) // sW + 1)
    max_split = max(1, min(256, B * ((N + 15) // 16) // 8))
    ran = int(gw_label.split("split=")[1])
    assert ran == min(split, max_split), labels


@pytest.mark.parametrize("mode", [0, 2], ids=["columns", "gathered"])
def test_products_of_96_rows_take_the_96_row_tile(gt, mode):
    """Products of 96 to 127 rows whose first operand lies along the reduction (forward and gradWeight on either
    route) run on the 96 x 128 tile rather than on two 64-row tiles with a third of the work repeated: the
    library's choice at the size of the reference benchmark's first layer (gpunn/test/benchmark.lua:73-80; the
    results of this tile are checked on the small shapes above)."""
    B, C, H, W, M, k = 16, 3, 128, 128, 96, 11
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0
    try:
        m = gt.nn.SpatialConvolutionMM(C, M, k, k).gpu()
        rng = rng_for(85)
        dx = dev(gt, uniform(rng, (B, C, H, W)))
        dgo = dev(gt, uniform(rng, (B, M, H - k + 1, W - k + 1)))
        gt.gputorch.synchronize()
        gt.gputorch.prof_reset()
        gt.gputorch.prof_enable(True)
        try:
            m.forward(dx)
            m.accGradParameters(dx, dgo, 1.0)
            gt.gputorch.synchronize()
            labels = {k2.split(" ")[0]: k2 for k2 in gt.gputorch.prof_report() if k2.startswith("gemm_conv")}
        finally:
            gt.gputorch.prof_enable(False)
            gt.gputorch.prof_reset()
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0
    assert "tile=96x128 " in labels["gemm_conv_fwd"], labels
    assert "tile=96x128 " in labels["gemm_conv_gradweight"], labels


@pytest.mark.parametrize("mode", [0, 2], ids=["columns", "gathered"])
@pytest.mark.parametrize("name", ["second_layer_N729", "ragged_M130_K1188_N100", "first_layer_M96_N225"])
def test_bias_gradient_rides_on_the_gradweight_product(gt, name, mode, switches):
    """gradBias is the row sums of the gradWeight product's first operand (gpunn-impl/SpatialConvolutionMM.cpp:413-417
    computes it with a gemv against ones): the tiled reduction-batched kernels sum it on the side and the reduction
    launch finishes it, so no bias-gradient kernel of its own runs; the gradbias_separate switch brings the two-stage
    sum back.  Both are exact on integers (checked inside run())."""
    def kernels(separate):
        switches("gradbias_separate", "1" if separate else None)
        B, C, H, W, M, kH, kW, pH, pW, sH, sW = SHAPES[name]
        x, w, b, go, gw0, gb0, out, gi, gw, gb = case(name)
        lib = gt._lib.lib
        before = lib.thgpu_conv_get_mode()
        assert lib.thgpu_conv_set_mode(mode) == 0
        try:
            m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
            m._assign("weight", w)
            m._assign("bias", b)
            m.gradWeight[...] = gw0
            m.gradBias[...] = gb0
            m.gpu()
            dx, dgo = dev(gt, x), dev(gt, go)
            m.forward(dx)
            gt.gputorch.synchronize()
            gt.gputorch.prof_reset()
            gt.gputorch.prof_enable(True)
            try:
                m.accGradParameters(dx, dgo, 2.0)
                gt.gputorch.synchronize()
                labels = sorted(gt.gputorch.prof_report())
            finally:
                gt.gputorch.prof_enable(False)
                gt.gputorch.prof_reset()
            assert np.array_equal(m.gradBias.float(), gb) and np.array_equal(m.gradWeight.float(), gw)
        finally:
            assert lib.thgpu_conv_set_mode(before) == 0
        return labels

    fused, separate = kernels(False), kernels(True)
    assert not any(l.startswith("gradbias") for l in fused), fused
    assert any(l.startswith("gemm_split_reduce") for l in fused), fused
    assert any(l.startswith("gradbias") for l in separate), separate


def random_layers(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    out = []
    for _ in range(n):
        kH, kW = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        sH, sW = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        pH, pW = int(rng.integers(0, kH)), int(rng.integers(0, kW))
        H, W = int(rng.integers(max(kH, 8), 90)), int(rng.integers(max(kW, 8), 90))
        B = int(rng.integers(1, 9))
        C = int(rng.choice([1, 2, 3, 4, 6, 12, 16, 33, 64, 70]))
        M = int(rng.choice([8, 24, 48, 64, 96, 100, 110, 127, 128, 130, 192]))
        out.append((B, C, H, W, M, kH, kW, pH, pW, sH, sW))
    return out


@pytest.mark.parametrize("cfg", random_layers(60, 4242))
def test_random_layers_integer_exact_on_every_route(gt, cfg):
    """Seeded random layers (plane counts around the tile heights, kernels up to 11, strides up to 4) on integer data:
    output, gradInput, gradWeight and gradBias equal the oracle's bit for bit on the column route, on the library's
    choice and with everything gathered that can be."""
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    K = C * kH * kW
    geo = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(zlib.crc32(repr(cfg).encode()) % 100000)
    ints = lambda lo, hi, shape: rng.integers(lo, hi + 1, size=shape).astype(np.float32)
    x, w, b = ints(-2, 2, (B, C, H, W)), ints(-2, 2, (M, K)), ints(-3, 3, (M,))
    oracle.use_blas(True)
    try:
        out, finput = oracle.conv_updateOutput(x, w, b, *geo)
        go = ints(-2, 2, out.shape)
        gi, _ = oracle.conv_updateGradInput(go, w, x.shape, *geo)
        gw0, gb0 = ints(-5, 5, (M, K)), ints(-5, 5, (M,))
        gw, gb = gw0.copy(), gb0.copy()
        oracle.conv_accGradParameters(go, finput, gw, gb, 2.0)
    finally:
        oracle.use_blas(False)
    assert max(np.abs(out).max(), np.abs(gi).max(), np.abs(gw).max(), np.abs(gb).max()) < 2 ** 24
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    try:
        for mode in (0, 1, 2):
            assert lib.thgpu_conv_set_mode(mode) == 0
            print("layer", cfg, "mode", mode, flush=True)
            m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
            m._assign("weight", w)
            m._assign("bias", b)
            m.gradWeight[...] = gw0
            m.gradBias[...] = gb0
            m.gpu()
            dx, dgo = dev(gt, x), dev(gt, go)
            assert np.array_equal(m.forward(dx).float(), out), "output, mode %d" % mode
            assert np.array_equal(m.updateGradInput(dx, dgo).float(), gi), "gradInput, mode %d" % mode
            m.accGradParameters(dx, dgo, 2.0)
            assert np.array_equal(m.gradWeight.float(), gw), "gradWeight, mode %d" % mode
            assert np.array_equal(m.gradBias.float(), gb), "gradBias, mode %d" % mode
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0

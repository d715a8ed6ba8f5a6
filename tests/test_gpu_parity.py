"""GPU parity tests: the HIP library, called through its C ABI (ctypes), against
the CPU oracle on identical seeded inputs.

Bars: bit-exact for im2col / col2im buffers, max-pool outputs, argmax indices
and gradients, threshold; fp32 GEMM-backed results within a norm-wise relative
error of 1e-4*sqrt(reduction length).
"""
import ctypes
import itertools

import numpy as np
import pytest

from helpers import (check_close, check_digest, gemm_tol, kat_conv_inputs, kat_pool_inputs, load_kat, oracle_stack, rel_err, both_rel_err,
                     rng_for, uniform)

# These tests check the column buffers too, so they pin the column route.
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("columns_route")]

import oracle  # noqa: E402


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def f32p(t, gt):
    return gt._lib.lib.THGPUTensor_data(t._p)


GEOMS = [
    # B, C, H, W, kH, kW, pH, pW, sH, sW
    (2, 2, 6, 7, 3, 3, 0, 0, 1, 1),
    (3, 3, 7, 5, 3, 2, 1, 1, 1, 1),
    (2, 1, 9, 8, 3, 2, 1, 2, 2, 3),
    (2, 2, 8, 9, 2, 4, 0, 3, 3, 2),
    (2, 3, 23, 23, 11, 11, 2, 2, 4, 4),
    (1, 2, 5, 5, 1, 1, 0, 0, 1, 1),
    (5, 3, 101, 77, 5, 5, 0, 0, 3, 3),      # odd sizes of the edge sweep (d)
    (2, 3, 128, 96, 7, 3, 3, 1, 2, 1),      # non-square kernel/stride/pad of the edge sweep (b)
    (2, 3, 128, 96, 3, 7, 1, 3, 1, 2),
    (4, 16, 27, 27, 5, 5, 2, 2, 1, 1),
    (3, 8, 13, 13, 3, 3, 1, 1, 1, 1),
    (2, 5, 56, 56, 3, 3, 1, 1, 1, 1),
    (3, 2, 24, 28, 5, 5, 0, 0, 1, 1),
    (300, 2, 3, 4, 3, 3, 2, 2, 1, 1),       # planes much smaller than a workgroup
    (2, 3, 9, 7, 5, 5, 4, 4, 1, 1),         # padding as large as the window allows
    (2, 3, 224, 224, 11, 11, 2, 2, 4, 4),   # first layer of the AlexNet-style stack
    (1, 2, 70, 90, 5, 7, 2, 3, 2, 3),
    (2, 2, 65, 131, 4, 6, 0, 5, 3, 2),
]


@pytest.fixture(params=[None, "unit", "strip", "direct"])
def im2col_kernel(request, switches):
    """Runs a test with the library's own kernel choice, then with each im2col kernel forced
    (a forced kernel that does not apply to a geometry falls through to the next)."""
    switches("im2col_kernel", request.param)
    return request.param


@pytest.mark.parametrize("geo", GEOMS)
def test_im2col_bit_exact(gt, geo, im2col_kernel):
    B, C, H, W, kH, kW, pH, pW, sH, sW = geo
    im = uniform(rng_for(21), (B, C, H, W))
    ref = oracle.im2col(im, kH, kW, pH, pW, sH, sW)
    d_im = dev(gt, im)
    d_col = gt.GPUTensor(*ref.shape)
    d_col.fill(np.nan)
    rc = gt._lib.lib.thgpu_im2col(f32p(d_im, gt), B, C, H, W, kH, kW, pH, pW, sH, sW, f32p(d_col, gt))
    gt._lib.check_status(rc)
    assert np.array_equal(bits(d_col.float()), bits(ref))


def test_im2col_unaligned_destination(gt, im2col_kernel):
    B, C, H, W, kH, kW, pH, pW, sH, sW = 2, 3, 9, 11, 3, 3, 1, 1, 2, 1
    im = uniform(rng_for(22), (B, C, H, W))
    ref = oracle.im2col(im, kH, kW, pH, pW, sH, sW)
    d_im = dev(gt, im)
    buf = gt.GPUTensor(ref.size + 1)
    buf.fill(7.0)
    view = buf.narrow(0, 1, ref.size)     # 4-byte aligned only
    rc = gt._lib.lib.thgpu_im2col(f32p(d_im, gt), B, C, H, W, kH, kW, pH, pW, sH, sW, f32p(view, gt))
    gt._lib.check_status(rc)
    host = buf.float()
    assert host[0] == 7.0
    assert np.array_equal(bits(host[1:]), bits(ref.ravel()))


@pytest.fixture(params=[None, "1"], ids=["auto", "generic"])
def col2im_kernel(request, switches):
    """Runs a test with the library's own col2im kernel choice, then with the general kernel forced."""
    switches("col2im_generic", request.param)
    return request.param


@pytest.mark.parametrize("geo", GEOMS)
def test_col2im_bit_exact(gt, geo, col2im_kernel):
    B, C, H, W, kH, kW, pH, pW, sH, sW = geo
    Ho, Wo = oracle.conv_out_size(H, W, kH, kW, pH, pW, sH, sW)
    col = uniform(rng_for(23), (B, C * kH * kW, Ho * Wo))
    ref = oracle.col2im(col, C, H, W, kH, kW, pH, pW, sH, sW)
    d_col = dev(gt, col)
    d_im = gt.GPUTensor(B, C, H, W)
    d_im.fill(np.nan)
    rc = gt._lib.lib.thgpu_col2im(f32p(d_col, gt), B, C, H, W, kH, kW, pH, pW, sH, sW, f32p(d_im, gt))
    gt._lib.check_status(rc)
    assert np.array_equal(bits(d_im.float()), bits(ref))


def _run_conv(gt, x, w, b, go, geo, scale=1.0, gw0=None, gb0=None):
    kH, kW, pH, pW, sH, sW = geo
    M, K = w.shape
    C = x.shape[-3]
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gradWeight[...] = 0 if gw0 is None else gw0
    m.gradBias[...] = 0 if gb0 is None else gb0
    m.gpu()
    dx, dgo = dev(gt, x), dev(gt, go)
    out = m.forward(dx).float()
    gi = m.backward(dx, dgo, scale).float()
    return dict(output=out, finput=m.finput.float(), fgradInput=m.fgradInput.float(), gradInput=gi,
                gradWeight=m.gradWeight.float(), gradBias=m.gradBias.float())


@pytest.mark.parametrize("name", ["conv_stride1", "conv_strided"])
def test_conv_reference_known_answers_exact(gt, name):
    cfg = load_kat()[name]
    x, w, b, go = kat_conv_inputs(cfg)
    geo = (cfg["kH"], cfg["kW"], cfg["pH"], cfg["pW"], cfg["sH"], cfg["sW"])
    got = _run_conv(gt, x, w, b, go, geo, cfg["scale"])
    for key in ("finput", "output", "fgradInput", "gradInput", "gradWeight", "gradBias"):
        if key in cfg:
            check_digest(got[key], cfg[key])


CONVS = [
    # B, C, H, W, M, kH, kW, pH, pW, sH, sW
    (2, 3, 12, 10, 5, 3, 3, 1, 1, 1, 1),
    (3, 4, 13, 17, 6, 5, 3, 2, 0, 2, 3),
    (16, 3, 224, 224, 64, 11, 11, 2, 2, 4, 4),   # first benchmark configuration, full size
    (1, 384, 13, 13, 256, 3, 3, 1, 1, 1, 1),     # edge (a): batch 1
    (4, 64, 27, 27, 192, 5, 5, 2, 2, 1, 1),      # AlexNet conv2 shape
    # edge (b) at its stated batch of 32: kernel 7x3, stride 2x1, pad 3x1 on 128x96 maps.  The configuration's text
    # names both 3 and 64 input planes, and Torch's argument order (kW, kH) leaves the orientation open: all four.
    (32, 3, 128, 96, 128, 7, 3, 3, 1, 2, 1),
    (32, 3, 128, 96, 128, 3, 7, 1, 3, 1, 2),
    (32, 64, 128, 96, 128, 7, 3, 3, 1, 2, 1),
    (32, 64, 128, 96, 128, 3, 7, 1, 3, 1, 2),
    (5, 3, 101, 77, 37, 5, 5, 0, 0, 3, 3),       # edge (d): nothing a multiple of the MFMA tile
    (3, 130, 9, 9, 70, 3, 3, 1, 1, 1, 1),
]


@pytest.mark.parametrize("cfg", CONVS)
def test_conv_fwd_bwd_parity(gt, cfg):
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    geo = (kH, kW, pH, pW, sH, sW)
    K = C * kH * kW
    rng = rng_for(31)
    s = 1.0 / np.sqrt(K)
    x = uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (M, K), -s, s), uniform(rng, (M,), -s, s)
    # the oracle's plain sgemm loops for what they finish in seconds, the host BLAS above that (pinned against
    # those loops in tests/test_oracle_math.py)
    big = 6.0 * B * M * K * ((H + 2 * pH - kH) // sH + 1) * ((W + 2 * pW - kW) // sW + 1) > 2e10
    oracle.use_blas(big)
    try:
        out_ref, finput_ref = oracle.conv_updateOutput(x, w, b, *geo)
        go = uniform(rng, out_ref.shape)
        gi_ref, fgi_ref = oracle.conv_updateGradInput(go, w, x.shape, *geo)
        gw0, gb0 = uniform(rng, (M, K)), uniform(rng, (M,))
        gw_ref, gb_ref = gw0.copy(), gb0.copy()
        scale = 0.5
        oracle.conv_accGradParameters(go, finput_ref, gw_ref, gb_ref, scale)
    finally:
        oracle.use_blas(False)
    got = _run_conv(gt, x, w, b, go, geo, scale, gw0, gb0)
    N = out_ref.shape[2] * out_ref.shape[3]
    tag = "conv b%d %d->%d %dx%d k%dx%d p%dx%d s%dx%d columns " % (B, C, M, H, W, kH, kW, pH, pW, sH, sW)
    assert np.array_equal(bits(got["finput"]), bits(finput_ref))
    check_close(tag + "output", got["output"], out_ref, K)
    check_close(tag + "fgradInput", got["fgradInput"], fgi_ref, M)
    check_close(tag + "gradInput", got["gradInput"], gi_ref, M)
    check_close(tag + "gradWeight", got["gradWeight"], gw_ref, B * N)
    check_close(tag + "gradBias", got["gradBias"], gb_ref, B * N)


def test_conv_non_batch_input_and_rerun_is_identical(gt):
    C, H, W, M, kH, kW = 3, 14, 15, 8, 3, 5
    rng = rng_for(32)
    x, w, b = uniform(rng, (C, H, W)), uniform(rng, (M, C * kH * kW)), uniform(rng, (M,))
    ref, _ = oracle.conv_updateOutput(x[None], w, b, kH, kW, 1, 2, 1, 1)
    go = uniform(rng, ref.shape[1:])
    a = _run_conv(gt, x, w, b, go, (kH, kW, 1, 2, 1, 1))
    b2 = _run_conv(gt, x, w, b, go, (kH, kW, 1, 2, 1, 1))
    assert a["output"].shape == ref.shape[1:] and a["gradInput"].shape == x.shape
    assert both_rel_err(a["output"], ref[0]) < gemm_tol(C * kH * kW)
    for k in a:
        assert np.array_equal(bits(a[k]), bits(b2[k])), k   # deterministic: no atomics anywhere


@pytest.mark.parametrize("ta,tb", list(itertools.product("nt", "nt")))
@pytest.mark.parametrize("mnk", [(7, 5, 11), (130, 70, 33), (64, 256, 100), (1, 9, 300), (257, 129, 17)])
def test_blas_gemm_all_transposes(gt, ta, tb, mnk):
    m, n, k = mnk
    rng = rng_for(41)
    lda = (m if ta == "n" else k) + 3
    ldb = (k if tb == "n" else n) + 2
    ldc = m + 1
    a = uniform(rng, (lda * (k if ta == "n" else m),))
    b = uniform(rng, (ldb * (n if tb == "n" else k),))
    c0 = uniform(rng, (ldc * n,))
    ref = c0.copy()
    oracle.sgemm(ta, tb, m, n, k, 0.5, a, lda, b, ldb, 2.0, ref, ldc)
    da, db, dc = dev(gt, a), dev(gt, b), dev(gt, c0)
    gt.gputorch.gemm(ta, tb, m, n, k, 0.5, da, lda, db, ldb, 2.0, dc, ldc)
    got = dc.float()
    assert both_rel_err(got.reshape(n, ldc)[:, :m], ref.reshape(n, ldc)[:, :m]) < gemm_tol(k)
    assert np.array_equal(got.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])


def test_blas_gemm_integer_exact_beta0_ignores_nan_and_quick_returns(gt):
    rng = rng_for(42)
    m, n, k = 70, 45, 129
    a = rng.integers(-3, 4, size=(k, m)).astype(np.float32)
    b = rng.integers(-3, 4, size=(n, k)).astype(np.float32)
    c = np.full((n, m), np.nan, np.float32)
    da, db, dc = dev(gt, a), dev(gt, b), dev(gt, c)
    gt.gputorch.gemm("n", "n", m, n, k, 1.0, da, m, db, k, 0.0, dc, m)
    assert np.array_equal(dc.float(), (b.astype(np.int64) @ a.astype(np.int64)).astype(np.float32))
    before = dc.float()
    gt.gputorch.gemm("n", "n", m, n, k, 0.0, da, m, db, k, 1.0, dc, m)   # alpha 0, beta 1: untouched
    gt.gputorch.gemm("n", "n", m, n, 0, 1.0, da, m, db, k, 1.0, dc, m)   # k 0, beta 1: untouched
    assert np.array_equal(dc.float(), before)
    gt.gputorch.gemm("n", "n", m, n, k, 0.0, da, m, db, k, 3.0, dc, m)   # alpha 0: C *= beta
    assert np.array_equal(dc.float(), before * 3.0)


GEMM_TILES = ["128x128", "192x128", "64x256", "128x256", "256x128", "64x64", "64x128", "96x128"]


@pytest.mark.parametrize("split", [1, 3])
@pytest.mark.parametrize("ta,tb", list(itertools.product("nt", "nt")))
@pytest.mark.parametrize("tile", GEMM_TILES)
def test_blas_gemm_every_tile_configuration_exact(gt, tile, ta, tb, split, switches):
    """Every tile configuration of the fast kernel is forced in turn on a ragged problem (edge tiles shifted back in
    both directions, a partial last reduction step) with small integers, where any summation order is exact.  The
    profiler label tells which kernel ran."""
    switches("gemm_tile", tile)
    switches("gemm_split", split)
    rng = rng_for(43)
    m, n, k = 300, 421, 601
    lda = (m if ta == "n" else k) + 1
    ldb = (k if tb == "n" else n) + 3
    ldc = m + 2
    a = rng.integers(-3, 4, size=(lda * (k if ta == "n" else m),)).astype(np.float32)
    b = rng.integers(-3, 4, size=(ldb * (n if tb == "n" else k),)).astype(np.float32)
    c0 = rng.integers(-3, 4, size=(ldc * n,)).astype(np.float32)
    A = a.reshape(-1, lda)[:, :(m if ta == "n" else k)].astype(np.int64)      # column-major: [col][row]
    Bm = b.reshape(-1, ldb)[:, :(k if tb == "n" else n)].astype(np.int64)
    opA = A.T if ta == "n" else A                                              # m x k
    opB = Bm.T if tb == "n" else Bm                                            # k x n
    ref = c0.reshape(n, ldc).copy()
    ref[:, :m] = (2 * (opA @ opB).T + 3 * ref[:, :m].astype(np.int64)).astype(np.float32)
    da, db, dc = dev(gt, a), dev(gt, b), dev(gt, c0)
    gt.gputorch.synchronize()
    gt.gputorch.prof_reset()
    gt.gputorch.prof_enable(True)
    try:
        gt.gputorch.gemm(ta, tb, m, n, k, 2.0, da, lda, db, ldb, 3.0, dc, ldc)
        gt.gputorch.synchronize()
        labels = [key for key in gt.gputorch.prof_report() if "tile=" in key]
    finally:
        gt.gputorch.prof_enable(False)
        gt.gputorch.prof_reset()
    assert np.array_equal(dc.float().reshape(n, ldc), ref)
    assert len(labels) == 1
    ran = labels[0].split("tile=")[1].split(" ")[0]
    # the 96-row tile loads its first operand along the reduction only: op(B) = B, in BLAS terms
    expect = "generic" if tile == "96x128" and tb == "t" else tile
    assert ran == expect, labels
    assert ("split=%d" % split) in labels[0] or ran == "generic", labels


POOLS = [(2, 3, 7, 7, 3, 3, 2, 2), (3, 2, 9, 8, 2, 2, 2, 2), (2, 2, 10, 11, 3, 2, 1, 3), (1, 1, 6, 6, 4, 4, 1, 1),
         (4, 16, 55, 55, 3, 3, 2, 2), (2, 8, 13, 13, 3, 3, 2, 2), (2, 4, 24, 24, 2, 2, 2, 2),
         (2, 3, 11, 12, 2, 2, 3, 3),       # windows smaller than the stride: uncovered pixels
         (1, 2, 224, 224, 2, 2, 2, 2), (3, 5, 14, 9, 3, 3, 2, 2), (2, 2, 10, 10, 3, 3, 3, 3), (1, 1, 3, 300, 3, 3, 2, 2),
         (37, 3, 13, 13, 3, 3, 2, 2),      # more planes than one workgroup groups, a ragged last group
         (2, 3, 30, 31, 5, 4, 1, 1),       # dense overlap: 5 x 4 windows cover a pixel, 20 scatter phases
         (1, 2, 9, 70, 3, 3, 2, 2),        # rows wider than a wavefront: column chunks
         (2, 1, 120, 130, 4, 7, 3, 5),     # row strips and column chunks, stride below the window
         (3, 2, 40, 64, 3, 3, 1, 2), (2, 2, 33, 33, 2, 2, 1, 1), (1, 1, 64, 64, 64, 64, 1, 1)]


@pytest.fixture(params=["auto", "direct", "tile", "cell", "staged", "staged_small_share"])
def pool_bwd_kernel(request, switches):
    """Runs a test with the library's own forward and backward kernel choice (direct forward; for 3x3 / 2x2 windows at
    stride 2 the cell backward kernel on small launches and the staged one on large, else the LDS tile kernel), then
    with the wavefront-level tile forward and the direct backward kernel forced, then with each of the LDS tile, cell
    and staged backward kernels forced (the staged one with its full workgroup share and with a small one, so that
    strips of rows and ragged last groups occur on small planes too)."""
    switches("pool_fwd_wave", "1" if request.param == "direct" else None)
    switches("pool_bwd_direct", "1" if request.param == "direct" else None)
    switches("pool_bwd_tile", "1" if request.param == "tile" else None)
    switches("pool_bwd_cell", "1" if request.param == "cell" else None)
    switches("pool_bwd_pixels", {"staged": "4096", "staged_small_share": "300"}.get(request.param))
    return request.param


@pytest.mark.parametrize("cfg", POOLS)
@pytest.mark.parametrize("ties", [False, True])
def test_maxpool_fwd_bwd_bit_exact(gt, cfg, ties, pool_bwd_kernel):
    B, C, H, W, kH, kW, dH, dW = cfg
    rng = rng_for(51)
    x = rng.integers(0, 8, size=(B, C, H, W)).astype(np.float32) if ties else uniform(rng, (B, C, H, W))
    out_ref, ind_ref = oracle.maxpool_updateOutput(x, kH, kW, dH, dW)
    go = uniform(rng, out_ref.shape)
    gi_ref = oracle.maxpool_updateGradInput(go, ind_ref, x.shape, dH, dW)
    m = gt.nn.SpatialMaxPooling(kW, kH, dW, dH).gpu()
    dx = dev(gt, x)
    out = m.forward(dx).float()
    gi = m.backward(dx, dev(gt, go)).float()
    assert np.array_equal(bits(out), bits(out_ref))
    assert np.array_equal(bits(m.indices.float()), bits(ind_ref))
    assert np.array_equal(bits(gi), bits(gi_ref))


def test_maxpool_reference_known_answers_and_3d_input(gt):
    cfg = load_kat()["maxpool_overlap_ties"]
    x, go = kat_pool_inputs(cfg)
    m = gt.nn.SpatialMaxPooling(cfg["kW"], cfg["kH"], cfg["dW"], cfg["dH"]).gpu()
    dx = dev(gt, x[0])                       # 3D input, non-batch mode
    out = m.forward(dx).float()
    assert out.shape == (2, 3, 3) and np.all(out == cfg["output_all"])
    ind = m.indices.float()
    assert ind.shape == (2, 2, 3, 3)
    assert ind[0].ravel().tolist() == [float(v) for v in cfg["indices_y"]]
    assert ind[1].ravel().tolist() == [float(v) for v in cfg["indices_x"]]
    gi = m.backward(dx, dev(gt, go[0])).float()
    assert np.array_equal(gi, np.array(cfg["gradInput"], np.float32))


def test_maxpool_edge_c_tied_integers_large(gt, pool_bwd_kernel):
    # edge sweep (c) at its stated size: overlapping 3x3 s2 on a 128x256x27x27 input of integers 0..7
    rng = rng_for(52)
    x = rng.integers(0, 8, size=(128, 256, 27, 27)).astype(np.float32)
    out_ref, ind_ref = oracle.maxpool_updateOutput(x, 3, 3, 2, 2)
    go = rng.integers(-4, 5, size=out_ref.shape).astype(np.float32)
    gi_ref = oracle.maxpool_updateGradInput(go, ind_ref, x.shape, 2, 2)
    m = gt.nn.SpatialMaxPooling(3, 3, 2, 2).gpu()
    dx = dev(gt, x)
    assert np.array_equal(bits(m.forward(dx).float()), bits(out_ref))
    assert np.array_equal(bits(m.indices.float()), bits(ind_ref))
    gi = m.backward(dx, dev(gt, go)).float()
    assert np.array_equal(bits(gi), bits(gi_ref))
    assert gi.sum() == go.sum()


@pytest.mark.parametrize("n", [1, 3, 4, 1023, 4096, 100003])
def test_threshold_exact(gt, n):
    rng = rng_for(61)
    x, g = uniform(rng, (n,)), uniform(rng, (n,))
    x[::7] = 0.0
    m = gt.nn.ReLU().gpu()
    dx = dev(gt, x)
    assert np.array_equal(bits(m.forward(dx).float()), bits(oracle.threshold_updateOutput(x)))
    assert np.array_equal(bits(m.backward(dx, dev(gt, g)).float()), bits(oracle.threshold_updateGradInput(x, g)))
    m2 = gt.nn.Threshold(0.25, -3.0).gpu()
    assert np.array_equal(bits(m2.forward(dx).float()), bits(oracle.threshold_updateOutput(x, 0.25, -3.0)))


def test_small_alexnet_stack_matches_oracle(gt):
    stacks = gt.stacks
    name, B = "alexnet", 2
    layers = stacks.STACKS[name]["layers"]
    net = stacks.build(name, seed_base=2000)
    params = [(np.array(m.weight), np.array(m.bias)) if hasattr(m, "weight") else None for m in net.modules]
    x = stacks.make_input(name, B, seed=2000)
    go = uniform(rng_for(2003), stacks.output_shape(name, B))
    outs, gins, grads = oracle_stack(layers, params, x, go)
    net.gpu()
    dx = dev(gt, x)
    out = net.forward(dx).float()
    gi = net.backward(dx, dev(gt, go)).float()
    assert rel_err(out, outs[-1]) < 1e-3
    assert rel_err(gi, gins[0]) < 5e-3
    for m, g in zip(net.modules, grads):
        if g is not None:
            assert rel_err(m.gradWeight.float(), g[0]) < 5e-3
            assert rel_err(m.gradBias.float(), g[1]) < 5e-3

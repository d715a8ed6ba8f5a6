"""Seeded random geometries against the CPU oracle, through the C ABI: the fixed lists of the other test files name the
cases somebody thought of; these draw kernel sizes, strides, paddings and plane shapes at random (same seed every run),
so every kernel's index arithmetic meets shapes nobody chose.

Bars as elsewhere: im2col / col2im buffers, max-pool outputs, indices and gradInput, average-pooling and sub-sampling
outputs and gradInput bit-exact; convolution outputs and gradients within 1e-4 * sqrt(reduction length).
"""
import ctypes

import numpy as np
import pytest

import oracle
from helpers import gemm_tol, rel_err, both_rel_err, uniform

# These tests check the column buffers too, so they pin the column route.
pytestmark = [pytest.mark.gpu, pytest.mark.usefixtures("columns_route")]


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def f32p(t, gt):
    return gt._lib.lib.THGPUTensor_data(t._p)


def conv_geometries(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    out = []
    while len(out) < n:
        kH, kW = int(rng.integers(1, 8)), int(rng.integers(1, 8))
        sH, sW = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        pH, pW = int(rng.integers(0, kH)), int(rng.integers(0, kW))
        H, W = int(rng.integers(1, 70)), int(rng.integers(1, 90))
        if H + 2 * pH < kH or W + 2 * pW < kW:
            continue
        out.append((int(rng.integers(1, 4)), int(rng.integers(1, 6)), H, W, kH, kW, pH, pW, sH, sW))
    return out


def pool_geometries(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    out = []
    while len(out) < n:
        kH, kW = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        dH, dW = int(rng.integers(1, 5)), int(rng.integers(1, 5))
        H, W = int(rng.integers(kH, 60)), int(rng.integers(kW, 80))
        out.append((int(rng.integers(1, 4)), int(rng.integers(1, 6)), H, W, kH, kW, dH, dW))
    return out


@pytest.mark.parametrize("geo", conv_geometries(40, 2001))
def test_im2col_col2im_random_geometry_bit_exact(gt, geo):
    B, C, H, W, kH, kW, pH, pW, sH, sW = geo
    lib = gt._lib.lib
    rng = np.random.Generator(np.random.PCG64(hash(geo) % (1 << 32)))
    im = uniform(rng, (B, C, H, W))
    ref = oracle.im2col(im, kH, kW, pH, pW, sH, sW)
    d_im, d_col = dev(gt, im), gt.GPUTensor(*ref.shape)
    d_col.fill(np.nan)
    gt._lib.check_status(lib.thgpu_im2col(f32p(d_im, gt), B, C, H, W, kH, kW, pH, pW, sH, sW, f32p(d_col, gt)))
    assert np.array_equal(bits(d_col.float()), bits(ref))
    col = uniform(rng, ref.shape)
    back = oracle.col2im(col, C, H, W, kH, kW, pH, pW, sH, sW)
    d_col, d_back = dev(gt, col), gt.GPUTensor(B, C, H, W)
    d_back.fill(np.nan)
    gt._lib.check_status(lib.thgpu_col2im(f32p(d_col, gt), B, C, H, W, kH, kW, pH, pW, sH, sW, f32p(d_back, gt)))
    assert np.array_equal(bits(d_back.float()), bits(back))


@pytest.mark.parametrize("geo", conv_geometries(24, 2002))
def test_convolution_random_geometry(gt, geo):
    B, C, H, W, kH, kW, pH, pW, sH, sW = geo
    rng = np.random.Generator(np.random.PCG64(hash(geo) % (1 << 32)))
    M = int(rng.integers(1, 40))
    K = C * kH * kW
    x, w, b = uniform(rng, (B, C, H, W)), uniform(rng, (M, K)), uniform(rng, (M,))
    out_ref, finput = oracle.conv_updateOutput(x, w, b, kH, kW, pH, pW, sH, sW)
    go = uniform(rng, out_ref.shape)
    gi_ref, _ = oracle.conv_updateGradInput(go, w, x.shape, kH, kW, pH, pW, sH, sW)
    gw_ref, gb_ref = np.zeros_like(w), np.zeros_like(b)
    oracle.conv_accGradParameters(go, finput, gw_ref, gb_ref, 0.5)
    m = gt.nn.SpatialConvolutionMM(C, M, kW, kH, sW, sH, 0, padW=pW, padH=pH)
    m._assign("weight", w)
    m._assign("bias", b)
    m.gpu()
    m.zeroGradParameters()
    dx, dgo = dev(gt, x), dev(gt, go)
    out = m.forward(dx).float()
    gi = m.backward(dx, dgo, 0.5).float()
    N = out_ref.shape[2] * out_ref.shape[3]
    assert np.array_equal(bits(m.finput.float()), bits(finput))
    assert both_rel_err(out, out_ref) < gemm_tol(K)
    assert both_rel_err(gi, gi_ref) < gemm_tol(M)
    assert both_rel_err(m.gradWeight.float(), gw_ref) < gemm_tol(B * N)
    assert both_rel_err(m.gradBias.float(), gb_ref) < gemm_tol(B * N)


@pytest.mark.parametrize("geo", pool_geometries(40, 2003))
def test_pooling_random_geometry_bit_exact(gt, geo):
    B, C, H, W, kH, kW, dH, dW = geo
    lib = gt._lib.lib
    rng = np.random.Generator(np.random.PCG64(hash(geo) % (1 << 32)))
    x = rng.integers(0, 6, size=(B, C, H, W)).astype(np.float32) if (H + W) % 2 else uniform(rng, (B, C, H, W))
    dx = dev(gt, x)
    # max pooling: output, both index planes, gradInput (ties included when the input is integer valued)
    ref, ind = oracle.maxpool_updateOutput(x, kH, kW, dH, dW)
    go = uniform(rng, ref.shape)
    out, dind, dgo, gi = gt.GPUTensor(), gt.GPUTensor(), dev(gt, go), gt.GPUTensor()
    gt._lib.check_status(lib.thgpu_SpatialMaxPooling_updateOutput(dx._p, out._p, dind._p, kW, kH, dW, dH))
    assert np.array_equal(bits(out.float()), bits(ref)) and np.array_equal(dind.float(), ind)
    gt._lib.check_status(lib.thgpu_SpatialMaxPooling_updateGradInput(dx._p, dgo._p, gi._p, dind._p, kW, kH, dW, dH))
    assert np.array_equal(bits(gi.float()), bits(oracle.maxpool_updateGradInput(go, ind, x.shape, dH, dW)))
    # window sums and per-plane sub-sampling
    w, b = uniform(rng, (C,)), uniform(rng, (C,))
    dw, db = dev(gt, w), dev(gt, b)
    gt._lib.check_status(lib.thgpu_SpatialAveragePooling_updateOutput(dx._p, out._p, kW, kH, dW, dH))
    assert np.array_equal(bits(out.float()), bits(oracle.subsample_updateOutput(x, None, None, kH, kW, dH, dW)))
    gt._lib.check_status(lib.thgpu_SpatialAveragePooling_updateGradInput(dx._p, dgo._p, gi._p, kW, kH, dW, dH))
    assert np.array_equal(bits(gi.float()), bits(oracle.subsample_updateGradInput(go, None, x.shape, kH, kW, dH, dW)))
    gt._lib.check_status(lib.thgpu_SpatialSubSampling_updateOutput(dx._p, dw._p, db._p, out._p, kW, kH, dW, dH))
    assert np.array_equal(bits(out.float()), bits(oracle.subsample_updateOutput(x, w, b, kH, kW, dH, dW)))
    gt._lib.check_status(lib.thgpu_SpatialSubSampling_updateGradInput(dx._p, dgo._p, dw._p, gi._p, kW, kH, dW, dH))
    assert np.array_equal(bits(gi.float()), bits(oracle.subsample_updateGradInput(go, w, x.shape, kH, kW, dH, dW)))


def gemm_cases(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    out = []
    for _ in range(n):
        big = rng.integers(0, 3) == 0
        hi = 700 if big else 90
        m, nn_, k = int(rng.integers(1, hi)), int(rng.integers(1, hi)), int(rng.integers(1, hi))
        out.append(("nt"[rng.integers(0, 2)], "nt"[rng.integers(0, 2)], m, nn_, k, int(rng.integers(0, 4)),
                    int(rng.integers(0, 4)), int(rng.integers(0, 4)), float(rng.choice([1.0, 0.5, -2.0])),
                    float(rng.choice([0.0, 1.0, 0.25]))))
    return out


@pytest.mark.parametrize("case", gemm_cases(48, 2004))
def test_blas_gemm_random_shapes(gt, case):
    ta, tb, m, n, k, pa, pb, pc, alpha, beta = case
    rng = np.random.Generator(np.random.PCG64(hash(case[:8]) % (1 << 32)))
    lda = (m if ta == "n" else k) + pa
    ldb = (k if tb == "n" else n) + pb
    ldc = m + pc
    integer = (m + n + k) % 2 == 0                 # half of the cases on small integers: any summation order is exact
    draw = (lambda size: rng.integers(-3, 4, size=size).astype(np.float32)) if integer else (lambda size: uniform(rng, size))
    a = draw((lda * (k if ta == "n" else m),))
    b = draw((ldb * (n if tb == "n" else k),))
    c0 = draw((ldc * n,))
    ref = c0.copy()
    oracle.sgemm(ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, ref, ldc)
    da, db, dc = dev(gt, a), dev(gt, b), dev(gt, c0)
    gt.gputorch.gemm(ta, tb, m, n, k, alpha, da, lda, db, ldb, beta, dc, ldc)
    got = dc.float().reshape(n, ldc)
    ref = ref.reshape(n, ldc)
    if integer:
        assert np.array_equal(got, ref)
    else:
        assert both_rel_err(got[:, :m], ref[:, :m]) < gemm_tol(k)
        assert np.array_equal(got[:, m:], c0.reshape(n, ldc)[:, m:])       # the padding of C is never written

"""Pins the CPU oracle with what the mathematics fixes: brute force from the
closed-form index maps, the im2col/col2im adjoint identity, exact integer
GEMMs, and torch's CPU conv2d / max_pool2d as an independent library routine.
CPU only."""
import itertools

import numpy as np
import pytest

import oracle
from helpers import (brute_col2im, brute_im2col, brute_maxpool, brute_maxpool_bwd, gemm_tol, rel_err, rng_for,
                     uniform)

GEOMS = [
    # C, H, W, kH, kW, pH, pW, sH, sW
    (2, 6, 7, 3, 3, 0, 0, 1, 1),
    (3, 7, 5, 3, 2, 1, 1, 1, 1),
    (1, 9, 8, 3, 2, 1, 2, 2, 3),
    (2, 8, 9, 2, 4, 0, 3, 3, 2),
    (3, 11, 11, 5, 5, 2, 2, 4, 4),
    (2, 5, 5, 1, 1, 0, 0, 1, 1),
    (1, 4, 6, 4, 6, 0, 0, 1, 1),
    (2, 7, 7, 7, 3, 3, 1, 2, 1),
]


@pytest.mark.parametrize("geo", GEOMS)
def test_im2col_equals_bruteforce(geo):
    C, H, W, *g = geo
    im = uniform(rng_for(1), (2, C, H, W))
    assert np.array_equal(oracle.im2col(im, *g), brute_im2col(im, *g))


def test_im2col_arange_is_self_describing_and_pads_with_positive_zero():
    C, H, W = 2, 5, 4
    im = (np.arange(C * H * W, dtype=np.float32) + 1).reshape(1, C, H, W)
    col = oracle.im2col(im, 3, 3, 1, 1, 1, 1)
    # centre tap (kh=1,kw=1) of channel c reproduces the channel itself
    for c in range(C):
        assert np.array_equal(col[0, (c * 3 + 1) * 3 + 1].reshape(H, W), im[0, c])
    zeros = col[col == 0]
    assert zeros.size > 0 and not np.any(np.signbit(zeros))


@pytest.mark.parametrize("k,pad", [(3, 0), (3, 1), (3, 2), (5, 2), (5, 4), (4, 3), (2, 1), (3, 4), (1, 2)])
def test_unfold_edges_against_padding_by_hand(k, pad):
    """The left / right and top / bottom edge handling of the unfold (lpad / rpad in
    mcw_nn/generic/SpatialConvolutionMM.c:35-37,81-85), pinned independently of any index formula: pad the image by
    hand with numpy, then column row (c, kh, kw) is the padded plane shifted by (kh, kw) and cut to the output size.
    Paddings from 0 through k-1 and above (a whole tap row or column outside the image); fold is held to the adjoint
    identity on the same geometries, with integer data so that every sum is exact."""
    rng = rng_for(40 + 7 * k + pad)
    B, C, H, W = 2, 2, 6, 7
    Ho, Wo = H + 2 * pad - k + 1, W + 2 * pad - k + 1
    if Ho < 1 or Wo < 1:
        pytest.skip("kernel larger than the padded image")
    im = rng.integers(-4, 5, (B, C, H, W)).astype(np.float32)
    padded = np.pad(im, [(0, 0), (0, 0), (pad, pad), (pad, pad)])
    col = oracle.im2col(im, k, k, pad, pad, 1, 1)
    assert col.shape == (B, C * k * k, Ho * Wo)
    for c in range(C):
        for kh in range(k):
            for kw in range(k):
                want = padded[:, c, kh:kh + Ho, kw:kw + Wo].reshape(B, Ho * Wo)
                assert np.array_equal(col[:, (c * k + kh) * k + kw], want), (c, kh, kw)
    assert not np.any(np.signbit(col[col == 0]))          # padding is +0.0f
    y = rng.integers(-4, 5, col.shape).astype(np.float32)
    back = oracle.col2im(y, C, H, W, k, k, pad, pad, 1, 1)
    assert float(np.sum(col.astype(np.float64) * y)) == float(np.sum(im.astype(np.float64) * back))
    # fold by hand: every column row added back at its shift, cropped to the image
    acc = np.zeros_like(padded, dtype=np.float64)
    for c in range(C):
        for kh in range(k):
            for kw in range(k):
                acc[:, c, kh:kh + Ho, kw:kw + Wo] += y[:, (c * k + kh) * k + kw].reshape(B, Ho, Wo)
    assert np.array_equal(back, acc[:, :, pad:pad + H, pad:pad + W].astype(np.float32))


@pytest.mark.parametrize("geo", GEOMS)
def test_col2im_equals_ordered_bruteforce_bit_exact(geo):
    C, H, W, kH, kW, pH, pW, sH, sW = geo
    Ho, Wo = oracle.conv_out_size(H, W, kH, kW, pH, pW, sH, sW)
    col = uniform(rng_for(2), (2, C * kH * kW, Ho * Wo))
    got = oracle.col2im(col, C, H, W, kH, kW, pH, pW, sH, sW)
    ref = brute_col2im(col, C, H, W, kH, kW, pH, pW, sH, sW)
    assert np.array_equal(got.view(np.uint32), ref.view(np.uint32))


def test_col2im_add_order_is_kh_then_kw_ascending():
    # Values chosen so that float32 addition order changes the result:
    # (1e8 + 1) - 1e8 depends on which pair is added first.
    C, H, W, kH, kW = 1, 1, 3, 1, 3
    Ho, Wo = oracle.conv_out_size(H, W, kH, kW, 0, 1, 1, 1)
    col = np.zeros((1, 3, Ho * Wo), np.float32)
    # pixel x=1 receives kw=0 from wo=2, kw=1 from wo=1, kw=2 from wo=0
    col[0, 0, 2], col[0, 1, 1], col[0, 2, 0] = 1.0, 1e8, -1e8
    got = oracle.col2im(col, C, H, W, kH, kW, 0, 1, 1, 1)
    asc = np.float32(np.float32(np.float32(0) + np.float32(1.0)) + np.float32(1e8)) + np.float32(-1e8)
    desc = np.float32(np.float32(np.float32(0) + np.float32(-1e8)) + np.float32(1e8)) + np.float32(1.0)
    assert asc != desc
    assert got[0, 0, 0, 1] == asc


@pytest.mark.parametrize("geo", GEOMS)
def test_adjoint_identity_and_window_multiplicity(geo):
    C, H, W, kH, kW, pH, pW, sH, sW = geo
    g = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(3)
    x = rng.integers(-4, 5, size=(2, C, H, W)).astype(np.float32)
    Ho, Wo = oracle.conv_out_size(H, W, *g)
    y = rng.integers(-4, 5, size=(2, C * kH * kW, Ho * Wo)).astype(np.float32)
    lhs = np.sum(oracle.im2col(x, *g).astype(np.float64) * y)
    rhs = np.sum(x.astype(np.float64) * oracle.col2im(y, C, H, W, *g))
    assert lhs == rhs
    counts = oracle.col2im(np.ones_like(y), C, H, W, *g)
    assert counts.sum() == np.count_nonzero(oracle.im2col(np.ones_like(x), *g))


@pytest.mark.parametrize("ta,tb", list(itertools.product("nt", "nt")))
def test_sgemm_loops_all_transposes_ragged_ld(ta, tb):
    rng = rng_for(4)
    m, n, k = 7, 5, 11
    lda = (m if ta == "n" else k) + 3
    ldb = (k if tb == "n" else n) + 2
    ldc = m + 1
    a = uniform(rng, (lda * (k if ta == "n" else m),))
    b = uniform(rng, (ldb * (n if tb == "n" else k),))
    c0 = uniform(rng, (ldc * n,))
    A = a.reshape(-1, lda).T[:m, :k] if ta == "n" else a.reshape(-1, lda)[:m, :k]
    Bm = b.reshape(-1, ldb).T[:k, :n] if tb == "n" else b.reshape(-1, ldb)[:k, :n]
    c = c0.copy()
    oracle.sgemm(ta, tb, m, n, k, 0.5, a, lda, b, ldb, 2.0, c, ldc)
    ref = 2.0 * c0.reshape(n, ldc)[:, :m].T.astype(np.float64) + 0.5 * (A.astype(np.float64) @ Bm.astype(np.float64))
    assert rel_err(c.reshape(n, ldc)[:, :m].T, ref) < 1e-6
    assert np.array_equal(c.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])  # padding rows untouched


def test_sgemm_loops_exact_on_small_integers_and_beta_zero_ignores_c():
    rng = rng_for(5)
    m, n, k = 9, 6, 33
    a = rng.integers(-3, 4, size=(k, m)).astype(np.float32)   # column-major m x k
    b = rng.integers(-3, 4, size=(n, k)).astype(np.float32)   # column-major k x n
    c = np.full((n, m), np.nan, np.float32)
    oracle.sgemm("n", "n", m, n, k, 1.0, a.ravel(), m, b.ravel(), k, 0.0, c.ravel(), m)
    assert np.array_equal(c, (b.astype(np.int64) @ a.astype(np.int64)).astype(np.float32))


def test_sgemm_blas_backend_agrees_with_loops_within_tolerance():
    name = oracle.use_blas(True)
    try:
        if name == "th-fallback-loops":
            pytest.skip("no optimised BLAS found")
        rng = rng_for(6)
        m, n, k = 65, 33, 300
        a, b = uniform(rng, (k * m,)), uniform(rng, (n * k,))
        c1, c2 = np.zeros(n * m, np.float32), np.zeros(n * m, np.float32)
        oracle.sgemm("n", "n", m, n, k, 1.0, a, m, b, k, 0.0, c1, m)
        oracle.use_blas(False)
        oracle.sgemm("n", "n", m, n, k, 1.0, a, m, b, k, 0.0, c2, m)
        assert rel_err(c1, c2) < gemm_tol(k)
    finally:
        oracle.use_blas(False)


TORCH_GEOMS = [
    # B, C, H, W, M, kH, kW, pH, pW, sH, sW
    (3, 3, 12, 10, 5, 3, 3, 1, 1, 1, 1),
    (2, 4, 13, 17, 6, 5, 3, 2, 0, 2, 3),
    (2, 3, 23, 23, 8, 11, 11, 2, 2, 4, 4),
    (1, 5, 9, 9, 7, 7, 3, 3, 1, 2, 1),
]


@pytest.mark.parametrize("cfg", TORCH_GEOMS)
def test_conv_fwd_bwd_against_torch_cpu_float64(cfg):
    torch = pytest.importorskip("torch")
    B, C, H, W, M, kH, kW, pH, pW, sH, sW = cfg
    g = (kH, kW, pH, pW, sH, sW)
    rng = rng_for(7)
    K = C * kH * kW
    x, w, bias = uniform(rng, (B, C, H, W)), uniform(rng, (M, K)), uniform(rng, (M,))
    out, finput = oracle.conv_updateOutput(x, w, bias, *g)
    go = uniform(rng, out.shape)
    gi, _ = oracle.conv_updateGradInput(go, w, x.shape, *g)
    gw0, gb0 = uniform(rng, (M, K)), uniform(rng, (M,))
    gw, gb = gw0.copy(), gb0.copy()
    scale = 0.75
    oracle.conv_accGradParameters(go, finput, gw, gb, scale)

    xt = torch.tensor(x, dtype=torch.float64, requires_grad=True)
    wt = torch.tensor(w.reshape(M, C, kH, kW), dtype=torch.float64, requires_grad=True)
    bt = torch.tensor(bias, dtype=torch.float64, requires_grad=True)
    ot = torch.nn.functional.conv2d(xt, wt, bt, stride=(sH, sW), padding=(pH, pW))
    ot.backward(torch.tensor(go, dtype=torch.float64))
    N = out.shape[2] * out.shape[3]
    assert rel_err(out, ot.detach().numpy()) < gemm_tol(K)
    assert rel_err(gi, xt.grad.numpy()) < gemm_tol(M)
    assert rel_err(gw - gw0, scale * wt.grad.numpy().reshape(M, K)) < gemm_tol(B * N)
    assert rel_err(gb - gb0, scale * bt.grad.numpy()) < gemm_tol(B * N)


def test_conv_identity_weight_is_a_shifted_copy():
    # one-hot weight row selecting tap (c=1,kh=0,kw=2) turns the conv into a crop of channel 1
    rng = rng_for(8)
    x = uniform(rng, (2, 2, 6, 6))
    w = np.zeros((1, 2 * 3 * 3), np.float32)
    w[0, (1 * 3 + 0) * 3 + 2] = 1.0
    out, _ = oracle.conv_updateOutput(x, w, np.zeros(1, np.float32), 3, 3, 0, 0, 1, 1)
    assert np.array_equal(out[:, 0], x[:, 1, 0:4, 2:6])


def test_gradbias_is_rowsum_in_ascending_order():
    B, M, N, K = 3, 2, 1000, 4
    go = uniform(rng_for(9), (B, M, 25, 40))
    finput = np.zeros((B, K, N), np.float32)
    gw, gb = np.zeros((M, K), np.float32), np.zeros(M, np.float32)
    oracle.conv_accGradParameters(go, finput, gw, gb, 0.5)
    ref = np.zeros(M, np.float32)
    for b in range(B):
        for m in range(M):
            s = np.float32(0)
            for v in go[b, m].ravel():
                s = np.float32(s + v)
            ref[m] = np.float32(ref[m] + np.float32(np.float32(0.5) * s))
    assert np.array_equal(gb, ref)
    assert not gw.any()


POOLS = [(2, 3, 7, 7, 3, 3, 2, 2), (1, 2, 9, 8, 2, 2, 2, 2), (2, 2, 10, 11, 3, 2, 1, 3), (1, 1, 6, 6, 4, 4, 1, 1)]


@pytest.mark.parametrize("cfg", POOLS)
def test_maxpool_equals_bruteforce_with_ties(cfg):
    B, C, H, W, kH, kW, dH, dW = cfg
    rng = rng_for(10)
    x = rng.integers(0, 4, size=(B, C, H, W)).astype(np.float32)
    out, ind = oracle.maxpool_updateOutput(x, kH, kW, dH, dW)
    bout, bind = brute_maxpool(x, kH, kW, dH, dW)
    assert np.array_equal(out, bout) and np.array_equal(ind, bind)
    go = rng.integers(-5, 6, size=out.shape).astype(np.float32)
    gi = oracle.maxpool_updateGradInput(go, ind, x.shape, dH, dW)
    assert np.array_equal(gi, brute_maxpool_bwd(go, ind, x.shape, dH, dW))
    assert gi.sum() == go.sum()


def test_maxpool_constant_image_picks_first_element_and_matches_torch():
    torch = pytest.importorskip("torch")
    x = np.full((1, 2, 8, 8), 2.5, np.float32)
    out, ind = oracle.maxpool_updateOutput(x, 3, 3, 2, 2)
    assert np.all(ind == 1.0) and np.all(out == 2.5)
    rng = rng_for(11)
    x = uniform(rng, (2, 3, 13, 13))
    out, ind = oracle.maxpool_updateOutput(x, 3, 3, 2, 2)
    to, ti = torch.nn.functional.max_pool2d(torch.tensor(x), 3, 2, return_indices=True)
    assert np.array_equal(out, to.numpy())
    Ho, Wo = out.shape[2:]
    i, j = np.ogrid[:Ho, :Wo]
    flat = ((ind[0] - 1 + i * 2) * 13 + (ind[1] - 1 + j * 2)).astype(np.int64)
    assert np.array_equal(flat, ti.numpy())


def test_maxpool_backward_float_add_order():
    # two overlapping windows hit the same pixel; order (i,j) ascending is visible in float32
    x = np.zeros((1, 1, 3, 5), np.float32)
    x[0, 0, 1, 2] = 9.0
    out, ind = oracle.maxpool_updateOutput(x, 3, 3, 1, 1)   # Wo = 3, all windows pick pixel (1,2)
    go = np.array([1.0, 1e8, -1e8], np.float32).reshape(1, 1, 1, 3)
    gi = oracle.maxpool_updateGradInput(go, ind, x.shape, 1, 1)
    expect = np.float32(np.float32(np.float32(0) + np.float32(1.0)) + np.float32(1e8)) + np.float32(-1e8)
    reverse = np.float32(np.float32(np.float32(0) + np.float32(-1e8)) + np.float32(1e8)) + np.float32(1.0)
    assert expect != reverse
    assert gi[0, 0, 1, 2] == expect


def test_threshold_closed_form():
    x = np.array([-1.0, -0.0, 0.0, 1e-30, 2.0, np.inf, -np.inf], np.float32)
    g = np.arange(1, 8, dtype=np.float32)
    assert np.array_equal(oracle.threshold_updateOutput(x), np.array([0, 0, 0, 1e-30, 2, np.inf, 0], np.float32))
    assert np.array_equal(oracle.threshold_updateGradInput(x, g), np.array([0, 0, 0, 4, 5, 6, 0], np.float32))
    assert np.array_equal(oracle.threshold_updateOutput(x, 1.0, -7.0), np.array([-7, -7, -7, -7, 2, np.inf, -7], np.float32))


# ---- THTensor addmm / addmv / addr and nn.Linear (the classifier after a conv stack) -----------------
def test_oracle_addmm_addmv_addr_exact_on_small_integers():
    rng = rng_for(71)
    m1 = rng.integers(-3, 4, (5, 7)).astype(np.float32)
    m2 = rng.integers(-3, 4, (7, 4)).astype(np.float32)
    t = rng.integers(-3, 4, (5, 4)).astype(np.float32)
    assert np.array_equal(oracle.addmm(2.0, t, 3.0, m1, m2), 2 * t + 3 * (m1 @ m2))
    assert np.array_equal(oracle.addmm(0.0, np.full_like(t, np.nan), 1.0, m1, m2), m1 @ m2)   # beta 0 ignores t
    v7, v5, v4 = (rng.integers(-3, 4, n).astype(np.float32) for n in (7, 5, 4))
    assert np.array_equal(oracle.addmv(2.0, v5, 3.0, m1, v7), 2 * v5 + 3 * (m1 @ v7))
    assert np.array_equal(oracle.addmv_t(2.0, v7, 3.0, m1, v5), 2 * v7 + 3 * (m1.T @ v5))
    assert np.array_equal(oracle.addr(2.0, t, 3.0, v5, v4), 2 * t + 3 * np.outer(v5, v4))


def test_oracle_gemv_orders_follow_the_th_loops():
    # 't' (row-major mat @ vec): one accumulator, j ascending -> (1*1 + 1e8) - 1e8 = 0 in fp32, not 1
    mat = np.array([[1.0, 1e8, -1e8]], np.float32)
    assert oracle.addmv(0.0, np.zeros(1, np.float32), 1.0, mat, np.ones(3, np.float32))[0] == 0.0
    mat = np.array([[1e8, -1e8, 1.0]], np.float32)
    assert oracle.addmv(0.0, np.zeros(1, np.float32), 1.0, mat, np.ones(3, np.float32))[0] == 1.0
    # 'n' (mat.T @ vec): columns added j ascending into y
    mat = np.array([[1.0], [1e8], [-1e8]], np.float32)
    assert oracle.addmv_t(1.0, np.zeros(1, np.float32), 1.0, mat, np.ones(3, np.float32))[0] == 0.0


def test_oracle_linear_matches_torch_linear_and_autograd():
    torch = pytest.importorskip("torch")
    rng = rng_for(72)
    B, I, O = 6, 11, 5
    x, w, b, go = uniform(rng, (B, I)), uniform(rng, (O, I)), uniform(rng, (O,)), uniform(rng, (B, O))
    tx, tw, tb = (torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (x, w, b))
    out = torch.nn.functional.linear(tx, tw, tb)
    out.backward(torch.tensor(go, dtype=torch.float64))
    assert rel_err(oracle.linear_updateOutput(x, w, b), out.detach().numpy()) < 1e-6
    assert rel_err(oracle.linear_updateGradInput(go, w), tx.grad.numpy()) < 1e-6
    gw, gb = np.zeros_like(w), np.zeros_like(b)
    oracle.linear_accGradParameters(x, go, gw, gb, 0.5)
    assert rel_err(gw, 0.5 * tw.grad.numpy()) < 1e-6
    assert rel_err(gb, 0.5 * tb.grad.numpy()) < 1e-6

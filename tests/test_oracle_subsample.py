"""Pins the oracle's nn.SpatialSubSampling / nn.SpatialAveragePooling restatements (CPU only).

What pins them: a brute-force restatement written from the loop structure of
mcw_nn/generic/SpatialSubSampling.c:58-96,151-181,236-270 in pure Python (same float32 operation order, so equality is
bit-for-bit); torch's CPU avg_pool2d and grouped conv2d with autograd as an independent library routine (tolerance);
and closed forms on integer data: a plane of ones must give kH*kW everywhere -- the reference module returns the window
SUM, it never divides (mcw_nn/generic/SpatialAveragePooling.c:75-86).
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle
from helpers import rel_err, rng_for, uniform

GEOMS = [  # B, C, H, W, kH, kW, dH, dW
    (2, 3, 6, 6, 2, 2, 2, 2),      # the usual non-overlapping case
    (1, 2, 7, 8, 3, 2, 1, 1),      # overlapping, the Lua default stride
    (2, 2, 9, 7, 3, 3, 2, 2),      # overlapping with stride 2
    (1, 3, 8, 9, 2, 2, 3, 4),      # stride above the window: uncovered pixels
    (2, 1, 5, 5, 5, 5, 1, 1),      # one window
    (1, 2, 10, 4, 1, 1, 1, 1),     # 1x1 windows
]
f32 = np.float32


def brute_forward(x, w, b, kH, kW, dH, dW):
    B, C, H, W = x.shape
    Ho, Wo = (H - kH) // dH + 1, (W - kW) // dW + 1
    out = np.empty((B, C, Ho, Wo), f32)
    for p in range(B):
        for k in range(C):
            for yy in range(Ho):
                for xx in range(Wo):
                    s = f32(0)
                    for ky in range(kH):
                        for kx in range(kW):
                            s = f32(s + x[p, k, yy * dH + ky, xx * dW + kx])
                    if w is None:
                        out[p, k, yy, xx] = f32(f32(0) + s)
                    else:
                        out[p, k, yy, xx] = f32(b[k] + f32(w[k] * s))
    return out


def brute_backward(go, w, shape, kH, kW, dH, dW):
    B, C, H, W = shape
    gi = np.zeros(shape, f32)
    for p in range(B):
        for k in range(C):
            for yy in range(go.shape[2]):
                for xx in range(go.shape[3]):
                    z = go[p, k, yy, xx] if w is None else f32(go[p, k, yy, xx] * w[k])
                    for ky in range(kH):
                        for kx in range(kW):
                            gi[p, k, yy * dH + ky, xx * dW + kx] = f32(gi[p, k, yy * dH + ky, xx * dW + kx] + z)
    return gi


def brute_accgrad(x, go, gw, gb, kH, kW, dH, dW, scale):
    B, C = x.shape[:2]
    for k in range(C):
        for p in range(B):
            s = f32(0)
            for v in go[p, k].ravel():
                s = f32(s + v)
            gb[k] = f32(gb[k] + f32(f32(scale) * s))
            s = f32(0)
            for yy in range(go.shape[2]):
                for xx in range(go.shape[3]):
                    z = go[p, k, yy, xx]
                    for ky in range(kH):
                        for kx in range(kW):
                            s = f32(s + f32(z * x[p, k, yy * dH + ky, xx * dW + kx]))
            gw[k] = f32(gw[k] + f32(f32(scale) * s))


@pytest.mark.parametrize("geo", GEOMS)
@pytest.mark.parametrize("sub", [False, True], ids=["avgpool", "subsample"])
def test_forward_backward_equal_the_loop_restatement_bit_for_bit(geo, sub):
    B, C, H, W, kH, kW, dH, dW = geo
    rng = rng_for(61)
    x = uniform(rng, (B, C, H, W))
    w, b = (uniform(rng, (C,)), uniform(rng, (C,))) if sub else (None, None)
    out = oracle.subsample_updateOutput(x, w, b, kH, kW, dH, dW)
    ref = brute_forward(x, w, b, kH, kW, dH, dW)
    assert np.array_equal(out.view(np.uint32), ref.view(np.uint32))
    go = uniform(rng, out.shape)
    gi = oracle.subsample_updateGradInput(go, w, x.shape, kH, kW, dH, dW)
    assert np.array_equal(gi.view(np.uint32), brute_backward(go, w, x.shape, kH, kW, dH, dW).view(np.uint32))


@pytest.mark.parametrize("geo", GEOMS[:4])
def test_accgradparameters_equals_the_loop_restatement_and_accumulates(geo):
    B, C, H, W, kH, kW, dH, dW = geo
    rng = rng_for(62)
    x = uniform(rng, (B, C, H, W))
    go = uniform(rng, (B, C, (H - kH) // dH + 1, (W - kW) // dW + 1))
    gw0, gb0 = uniform(rng, (C,)), uniform(rng, (C,))
    gw, gb = gw0.copy(), gb0.copy()
    oracle.subsample_accGradParameters(x, go, gw, gb, kH, kW, dH, dW, 0.5)
    rw, rb = gw0.copy(), gb0.copy()
    brute_accgrad(x, go, rw, rb, kH, kW, dH, dW, 0.5)
    assert np.array_equal(gw.view(np.uint32), rw.view(np.uint32))
    assert np.array_equal(gb.view(np.uint32), rb.view(np.uint32))


@pytest.mark.parametrize("geo", GEOMS)
def test_against_torch_avg_pool_and_grouped_conv_with_autograd(geo):
    B, C, H, W, kH, kW, dH, dW = geo
    rng = rng_for(63)
    x = uniform(rng, (B, C, H, W))
    w, b = uniform(rng, (C,)), uniform(rng, (C,))
    tx = torch.from_numpy(x).double().requires_grad_(True)
    tw = torch.from_numpy(w).double().requires_grad_(True)
    tb = torch.from_numpy(b).double().requires_grad_(True)
    # the window sum is avg_pool2d times the window size
    avg = F.avg_pool2d(tx, (kH, kW), (dH, dW)) * (kH * kW)
    out = oracle.subsample_updateOutput(x, None, None, kH, kW, dH, dW)
    assert rel_err(out, avg.detach().numpy()) < 1e-6
    go = uniform(rng, out.shape)
    avg.backward(torch.from_numpy(go).double())
    gi = oracle.subsample_updateGradInput(go, None, x.shape, kH, kW, dH, dW)
    assert rel_err(gi, tx.grad.numpy()) < 1e-6
    # sub-sampling is a depthwise convolution whose kernel is weight[k] everywhere
    tx.grad = None
    kern = tw.view(C, 1, 1, 1).expand(C, 1, kH, kW)
    sub = F.conv2d(tx, kern, tb, stride=(dH, dW), groups=C)
    out = oracle.subsample_updateOutput(x, w, b, kH, kW, dH, dW)
    assert rel_err(out, sub.detach().numpy()) < 1e-6
    sub.backward(torch.from_numpy(go).double())
    gi = oracle.subsample_updateGradInput(go, w, x.shape, kH, kW, dH, dW)
    assert rel_err(gi, tx.grad.numpy()) < 1e-6
    gw, gb = np.zeros(C, f32), np.zeros(C, f32)
    oracle.subsample_accGradParameters(x, go, gw, gb, kH, kW, dH, dW, 2.0)
    assert rel_err(gw, 2.0 * tw.grad.numpy()) < 1e-5
    assert rel_err(gb, 2.0 * tb.grad.numpy()) < 1e-5


def test_average_pooling_is_a_sum_and_uncovered_pixels_get_zero_gradient():
    x = np.ones((1, 2, 7, 9), f32)
    out = oracle.subsample_updateOutput(x, None, None, 2, 3, 3, 4)
    assert np.array_equal(out, np.full(out.shape, 6.0, f32))          # kH*kW, not 1
    gi = oracle.subsample_updateGradInput(np.ones_like(out), None, x.shape, 2, 3, 3, 4)
    cover = np.zeros((7, 9), f32)
    for yy in range(out.shape[2]):
        for xx in range(out.shape[3]):
            cover[yy * 3:yy * 3 + 2, xx * 4:xx * 4 + 3] += 1
    assert np.array_equal(gi[0, 0], cover) and np.array_equal(gi[0, 1], cover)
    assert (cover == 0).any()
    assert not np.signbit(gi).any()                                   # the zero fill is +0.0

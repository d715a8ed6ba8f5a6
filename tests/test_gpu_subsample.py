"""GPU parity of nn.SpatialAveragePooling and nn.SpatialSubSampling against the CPU oracle, through the C ABI.

Bars: output and gradInput bit-exact (the kernels add in the CPU modules' order and round product and sum separately);
gradWeight / gradBias within 1e-4 * sqrt(number of summed terms) relative, exact on small integers, reruns identical.
"""
import numpy as np
import pytest

import oracle
from helpers import rel_err, rng_for, uniform

pytestmark = pytest.mark.gpu

GEOMS = [  # B, C, H, W, kH, kW, dH, dW
    (2, 3, 6, 6, 2, 2, 2, 2),
    (1, 2, 7, 8, 3, 2, 1, 1),
    (2, 2, 9, 7, 3, 3, 2, 2),
    (1, 3, 8, 9, 2, 2, 3, 4),        # stride above the window: uncovered pixels
    (2, 1, 5, 5, 5, 5, 1, 1),
    (3, 5, 10, 4, 1, 1, 1, 1),
    (4, 16, 55, 55, 3, 3, 2, 2),
    (2, 8, 28, 28, 2, 2, 2, 2),      # LeNet-style sub-sampling
    (1, 2, 3, 300, 3, 3, 1, 2),
    (8, 64, 13, 13, 3, 3, 1, 1),
]


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def status(gt, rc):
    gt._lib.check_status(rc)


@pytest.mark.parametrize("geo", GEOMS)
def test_average_pooling_bit_exact(gt, geo):
    B, C, H, W, kH, kW, dH, dW = geo
    lib = gt._lib.lib
    rng = rng_for(71)
    x = uniform(rng, (B, C, H, W))
    ref = oracle.subsample_updateOutput(x, None, None, kH, kW, dH, dW)
    go = uniform(rng, ref.shape)
    dx, out, dgo, gi = dev(gt, x), gt.GPUTensor(), dev(gt, go), gt.GPUTensor()
    status(gt, lib.thgpu_SpatialAveragePooling_updateOutput(dx._p, out._p, kW, kH, dW, dH))
    assert out.size() == ref.shape and np.array_equal(bits(out.float()), bits(ref))
    status(gt, lib.thgpu_SpatialAveragePooling_updateGradInput(dx._p, dgo._p, gi._p, kW, kH, dW, dH))
    gref = oracle.subsample_updateGradInput(go, None, x.shape, kH, kW, dH, dW)
    assert gi.size() == x.shape and np.array_equal(bits(gi.float()), bits(gref))


@pytest.mark.parametrize("geo", GEOMS)
def test_subsampling_forward_backward_bit_exact_parameters_to_rounding(gt, geo):
    B, C, H, W, kH, kW, dH, dW = geo
    lib = gt._lib.lib
    rng = rng_for(72)
    x, w, b = uniform(rng, (B, C, H, W)), uniform(rng, (C,)), uniform(rng, (C,))
    ref = oracle.subsample_updateOutput(x, w, b, kH, kW, dH, dW)
    go = uniform(rng, ref.shape)
    dx, dw, db, out, dgo, gi = dev(gt, x), dev(gt, w), dev(gt, b), gt.GPUTensor(), dev(gt, go), gt.GPUTensor()
    status(gt, lib.thgpu_SpatialSubSampling_updateOutput(dx._p, dw._p, db._p, out._p, kW, kH, dW, dH))
    assert np.array_equal(bits(out.float()), bits(ref))
    status(gt, lib.thgpu_SpatialSubSampling_updateGradInput(dx._p, dgo._p, dw._p, gi._p, kW, kH, dW, dH))
    assert np.array_equal(bits(gi.float()), bits(oracle.subsample_updateGradInput(go, w, x.shape, kH, kW, dH, dW)))
    gw0, gb0 = uniform(rng, (C,)), uniform(rng, (C,))
    gw, gb = gw0.copy(), gb0.copy()
    oracle.subsample_accGradParameters(x, go, gw, gb, kH, kW, dH, dW, 0.25)
    dgw, dgb = dev(gt, gw0), dev(gt, gb0)
    status(gt, lib.thgpu_SpatialSubSampling_accGradParameters(dx._p, dgo._p, dgw._p, dgb._p, kW, kH, dW, dH, 0.25))
    terms = B * ref.shape[2] * ref.shape[3] * kH * kW
    assert rel_err(dgw.float(), gw) < 1e-4 * np.sqrt(terms)
    assert rel_err(dgb.float(), gb) < 1e-4 * np.sqrt(terms)
    first = (dgw.float().copy(), dgb.float().copy())
    dgw, dgb = dev(gt, gw0), dev(gt, gb0)
    status(gt, lib.thgpu_SpatialSubSampling_accGradParameters(dx._p, dgo._p, dgw._p, dgb._p, kW, kH, dW, dH, 0.25))
    assert np.array_equal(bits(dgw.float()), bits(first[0])) and np.array_equal(bits(dgb.float()), bits(first[1]))


def test_subsampling_parameters_exact_on_integers_and_three_dimensional_input(gt):
    lib = gt._lib.lib
    rng = rng_for(73)
    C, H, W, kH, kW, dH, dW = 4, 12, 11, 3, 2, 2, 3
    x = rng.integers(-3, 4, size=(C, H, W)).astype(np.float32)
    w = rng.integers(-2, 3, size=(C,)).astype(np.float32)
    b = rng.integers(-2, 3, size=(C,)).astype(np.float32)
    ref = oracle.subsample_updateOutput(x[None], w, b, kH, kW, dH, dW)[0]
    go = rng.integers(-3, 4, size=ref.shape).astype(np.float32)
    dx, dw, db, out, dgo, gi = dev(gt, x), dev(gt, w), dev(gt, b), gt.GPUTensor(), dev(gt, go), gt.GPUTensor()
    status(gt, lib.thgpu_SpatialSubSampling_updateOutput(dx._p, dw._p, db._p, out._p, kW, kH, dW, dH))
    assert out.size() == ref.shape and np.array_equal(out.float(), ref)
    status(gt, lib.thgpu_SpatialSubSampling_updateGradInput(dx._p, dgo._p, dw._p, gi._p, kW, kH, dW, dH))
    assert gi.size() == x.shape
    assert np.array_equal(gi.float(), oracle.subsample_updateGradInput(go[None], w, (1,) + x.shape, kH, kW, dH, dW)[0])
    gw, gb = np.ones(C, np.float32), np.full(C, 2, np.float32)
    oracle.subsample_accGradParameters(x[None], go[None], gw, gb, kH, kW, dH, dW, 2.0)
    dgw, dgb = dev(gt, np.ones(C)), dev(gt, np.full(C, 2))
    status(gt, lib.thgpu_SpatialSubSampling_accGradParameters(dx._p, dgo._p, dgw._p, dgb._p, kW, kH, dW, dH, 2.0))
    assert np.array_equal(dgw.float(), gw) and np.array_equal(dgb.float(), gb)     # integers: any order is exact


def test_argument_errors_carry_the_reference_messages(gt):
    lib = gt._lib.lib
    x = dev(gt, np.zeros((2, 3, 4, 4)))
    out = gt.GPUTensor()
    with pytest.raises(gt.THGPUError, match="input image smaller than kernel size"):
        status(gt, lib.thgpu_SpatialAveragePooling_updateOutput(x._p, out._p, 5, 2, 1, 1))
    flat = dev(gt, np.zeros((4, 4)))               # kept in a variable: the C call borrows the tensor
    with pytest.raises(gt.THGPUError, match="3D or 4D"):
        status(gt, lib.thgpu_SpatialAveragePooling_updateOutput(flat._p, out._p, 2, 2, 1, 1))
    w4 = dev(gt, np.zeros(4))
    with pytest.raises(gt.THGPUError, match="invalid number of input planes"):
        status(gt, lib.thgpu_SpatialSubSampling_updateOutput(x._p, w4._p, w4._p, out._p, 2, 2, 2, 2))
    gi = gt.GPUTensor()
    wrong = dev(gt, np.zeros((2, 3, 3, 3)))
    with pytest.raises(gt.THGPUError, match="gradOutput size"):
        status(gt, lib.thgpu_SpatialAveragePooling_updateGradInput(x._p, wrong._p, gi._p, 2, 2, 2, 2))


def test_nn_modules_mirror_the_lua_ones(gt):
    nn = gt.nn
    rng = rng_for(74)
    x = uniform(rng, (3, 4, 9, 9))
    m = nn.SpatialAveragePooling(3, 3)                  # strides default to 1
    assert (m.dW, m.dH) == (1, 1)
    m.gpu()
    dx = dev(gt, x)
    out = m.forward(dx).float()
    assert np.array_equal(bits(out), bits(oracle.subsample_updateOutput(x, None, None, 3, 3, 1, 1)))
    go = uniform(rng, out.shape)
    gi = m.backward(dx, dev(gt, go)).float()
    assert np.array_equal(bits(gi), bits(oracle.subsample_updateGradInput(go, None, x.shape, 3, 3, 1, 1)))

    s = nn.SpatialSubSampling(4, 2, 2, 2, 2, rng=rng)
    w, b = np.array(s.weight), np.array(s.bias)
    assert w.shape == (4,) and np.all(np.abs(w) <= 0.5) and np.all(np.abs(b) <= 0.5)    # U(+-1/sqrt(kW*kH))
    s.gpu()
    s.zeroGradParameters()
    out = s.forward(dx).float()
    assert np.array_equal(bits(out), bits(oracle.subsample_updateOutput(x, w, b, 2, 2, 2, 2)))
    go = uniform(rng, out.shape)
    gi = s.backward(dx, dev(gt, go)).float()
    assert np.array_equal(bits(gi), bits(oracle.subsample_updateGradInput(go, w, x.shape, 2, 2, 2, 2)))
    gw, gb = np.zeros(4, np.float32), np.zeros(4, np.float32)
    oracle.subsample_accGradParameters(x, go, gw, gb, 2, 2, 2, 2, 1.0)
    assert rel_err(s.gradWeight.float(), gw) < 1e-4 * 10 and rel_err(s.gradBias.float(), gb) < 1e-4 * 10

"""GPU parity of nn.LogSoftMax and nn.ClassNLLCriterion against the CPU oracle, through the C ABI.

LogSoftMax computes the CPU module's arithmetic (double sums, its polynomial exp approximation); the only freedom left
is the order of the double sums, so outputs must match the oracle to the last float bit almost everywhere: the test
allows one unit in the last place and requires 99.9 % of the elements to be identical.  ClassNLLCriterion sums in double:
the loss matches to 1e-6 relative, the gradient exactly.
"""
import numpy as np
import pytest

import oracle
from helpers import rng_for

pytestmark = pytest.mark.gpu
f32 = np.float32


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def close_in_ulps(got, ref):
    got, ref = np.asarray(got, f32), np.asarray(ref, f32)
    assert got.shape == ref.shape
    same = got.view(np.uint32) == ref.view(np.uint32)
    assert same.mean() >= 0.999, same.mean()
    assert np.all(np.abs(got - ref) <= np.spacing(np.abs(ref)))


@pytest.mark.parametrize("shape", [(1,), (10,), (1000,), (1, 1), (7, 3), (128, 1000), (33, 257), (4, 5000)])
def test_logsoftmax_forward_backward(gt, shape):
    lib = gt._lib.lib
    rng = rng_for(91)
    x = (rng.normal(size=shape) * 3).astype(f32)
    ref = oracle.logsoftmax_updateOutput(x)
    go = rng.normal(size=shape).astype(f32)
    gref = oracle.logsoftmax_updateGradInput(go, ref)
    dx, out, dgo, gi = dev(gt, x), gt.GPUTensor(), dev(gt, go), gt.GPUTensor()
    gt._lib.check_status(lib.thgpu_LogSoftMax_updateOutput(dx._p, out._p))
    assert out.size() == x.shape
    close_in_ulps(out.float(), ref)
    dref = dev(gt, ref)                          # backward from the oracle's output: isolates the backward formula
    gt._lib.check_status(lib.thgpu_LogSoftMax_updateGradInput(dgo._p, dref._p, gi._p))
    assert gi.size() == x.shape
    close_in_ulps(gi.float(), gref)


def test_logsoftmax_far_entries_and_non_contiguous_input(gt):
    lib = gt._lib.lib
    far = np.array([[0.0, -13.0, -50.0], [5.0, 5.0, -100.0]], f32)
    out = gt.GPUTensor()
    dfar = dev(gt, far)
    gt._lib.check_status(lib.thgpu_LogSoftMax_updateOutput(dfar._p, out._p))
    assert np.array_equal(out.float(), oracle.logsoftmax_updateOutput(far))
    assert np.array_equal(out.float()[0], far[0])          # entries 13 or more below the maximum add exactly nothing
    rng = rng_for(92)
    x = rng.normal(size=(6, 9)).astype(f32)
    dxt = dev(gt, x).t()                                   # a transposed view: the op densifies it
    gt._lib.check_status(lib.thgpu_LogSoftMax_updateOutput(dxt._p, out._p))
    close_in_ulps(out.float(), oracle.logsoftmax_updateOutput(np.ascontiguousarray(x.T)))
    cube = dev(gt, np.zeros((2, 2, 2)))
    with pytest.raises(gt.THGPUError, match="vector or matrix expected"):
        gt._lib.check_status(lib.thgpu_LogSoftMax_updateOutput(cube._p, out._p))


@pytest.mark.parametrize("size_average", [True, False])
@pytest.mark.parametrize("shape", [(1, 5), (9, 13), (128, 1000), (300, 7)])
def test_classnll(gt, shape, size_average):
    lib = gt._lib.lib
    rng = rng_for(93)
    x = rng.normal(size=shape).astype(f32)
    target = rng.integers(1, shape[1] + 1, size=shape[0])
    dx, dt, out, gi = dev(gt, x), dev(gt, target.astype(f32)), dev(gt, np.zeros(1)), dev(gt, np.full(shape, 7.0))
    gt._lib.check_status(lib.thgpu_ClassNLLCriterion_updateOutput(dx._p, dt._p, out._p, int(size_average)))
    ref = oracle.classnll_updateOutput(x, target, size_average)
    assert abs(float(out.float()[0]) - ref) <= 1e-6 * max(abs(ref), 1.0)
    gi.zero()
    gt._lib.check_status(lib.thgpu_ClassNLLCriterion_updateGradInput(dx._p, dt._p, gi._p, int(size_average)))
    assert np.array_equal(gi.float(), oracle.classnll_updateGradInput(x, target, size_average))


def test_classnll_vector_input_skipped_targets_and_module(gt):
    lib = gt._lib.lib
    rng = rng_for(94)
    x = rng.normal(size=(11,)).astype(f32)
    dx, dt, out, gi = dev(gt, x), dev(gt, np.array([4.0])), dev(gt, np.zeros(1)), dev(gt, np.zeros(11))
    gt._lib.check_status(lib.thgpu_ClassNLLCriterion_updateOutput(dx._p, dt._p, out._p, 1))
    assert float(out.float()[0]) == -float(x[3])           # a vector is never averaged
    gt._lib.check_status(lib.thgpu_ClassNLLCriterion_updateGradInput(dx._p, dt._p, gi._p, 1))
    assert np.array_equal(gi.float(), oracle.classnll_updateGradInput(x, np.array([4])))
    # a target of 0 is skipped (gpunn-impl/ClassNLLCriterion.cpp:50-52)
    m = rng.normal(size=(3, 4)).astype(f32)
    dm, dt = dev(gt, m), dev(gt, np.array([2.0, 0.0, 4.0]))
    gt._lib.check_status(lib.thgpu_ClassNLLCriterion_updateOutput(dm._p, dt._p, out._p, 0))
    assert abs(float(out.float()[0]) + float(m[0, 1]) + float(m[2, 3])) < 1e-6
    # the Lua-mirror modules: LogSoftMax -> ClassNLLCriterion forward and backward
    nn = gt.nn
    x = rng.normal(size=(16, 10)).astype(f32)
    target = rng.integers(1, 11, size=16)
    lsm, crit = nn.LogSoftMax().gpu(), nn.ClassNLLCriterion().gpu()
    dx, dt = dev(gt, x), dev(gt, target.astype(f32))
    logp = lsm.forward(dx)
    loss = crit.forward(logp, dt)
    ref_logp = oracle.logsoftmax_updateOutput(x)
    assert abs(loss - oracle.classnll_updateOutput(ref_logp, target)) < 1e-5
    dlogp = crit.backward(logp, dt)
    gin = lsm.backward(dx, dlogp).float()
    ref_gin = oracle.logsoftmax_updateGradInput(oracle.classnll_updateGradInput(ref_logp, target), ref_logp)
    assert np.abs(gin - ref_gin).max() < 1e-6
    with pytest.raises(gt.THGPUError):
        nn.ClassNLLCriterion(weights=np.ones(10, f32))

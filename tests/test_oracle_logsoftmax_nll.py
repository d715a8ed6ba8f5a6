"""Pins the oracle's nn.LogSoftMax and nn.ClassNLLCriterion restatements (CPU only).

LogSoftMax: a pure-Python restatement of mcw_nn/generic/LogSoftMax.c:37-53,85-97 with the polynomial of
TH/THLogAdd.c:56-86 (Python floats are C doubles, so equality is bit-for-bit); the exact log-softmax of scipy bounds the
approximation the CPU module makes (a few 1e-4, the reference's own test allows 1e-2: gpunn/test/test.lua:2149); known
values of the polynomial (1 at 0, exactly 0 from 13 on); the backward pass against torch autograd of the exact function.
ClassNLLCriterion: torch's nll_loss as the independent routine.
"""
import math

import numpy as np
import pytest
import scipy.special
import torch
import torch.nn.functional as F

import oracle
from helpers import rng_for

f32 = np.float32


def approx(x):
    if x < 13.0:
        y = 1.0 + x * (0.125 + x * (0.0078125 + x * (0.00032552083 + x * 1.0172526e-5)))
        y *= y
        y *= y
        y *= y
        return 1 / y
    return 0.0


def py_forward(x):
    out = np.empty_like(x)
    for t in range(x.shape[0]):
        m = f32(-np.inf)
        for v in x[t]:
            m = m if m > v else v
        s = 0.0
        for v in x[t]:
            s += approx(float(f32(m - v)))
        logsum = float(m) + math.log(s)
        for d, v in enumerate(x[t]):
            out[t, d] = f32(float(v) - logsum)
    return out


def py_backward(go, out):
    gi = np.empty_like(out)
    for t in range(out.shape[0]):
        s = 0.0
        for v in go[t]:
            s += float(v)
        for d in range(out.shape[1]):
            gi[t, d] = f32(float(go[t, d]) - math.exp(float(out[t, d])) * s)
    return gi


@pytest.mark.parametrize("shape", [(1, 1), (3, 7), (5, 100), (2, 1000)])
def test_logsoftmax_equals_the_python_restatement_bit_for_bit(shape):
    rng = rng_for(81)
    x = (rng.normal(size=shape) * 3).astype(f32)
    out = oracle.logsoftmax_updateOutput(x)
    assert np.array_equal(out.view(np.uint32), py_forward(x).view(np.uint32))
    go = rng.normal(size=shape).astype(f32)
    gi = oracle.logsoftmax_updateGradInput(go, out)
    assert np.array_equal(gi.view(np.uint32), py_backward(go, out).view(np.uint32))
    assert np.array_equal(oracle.logsoftmax_updateOutput(x[0]), out[0])          # a vector is one frame


def test_logsoftmax_is_the_exact_function_up_to_the_modules_exp_approximation():
    rng = rng_for(82)
    x = (rng.normal(size=(16, 300)) * 2).astype(f32)
    out = oracle.logsoftmax_updateOutput(x)
    exact = scipy.special.log_softmax(x.astype(np.float64), axis=1)
    err = np.abs(out - exact).max()
    assert 1e-6 < err < 1e-2            # it IS an approximation (an exact exp would sit near 1e-7), and a close one
    assert np.all(np.argmax(out, 1) == np.argmax(x, 1))
    # the polynomial: 1 at 0, monotone, exactly zero from 13 on, within 1e-3 of exp(-x) in between (absolute)
    assert approx(0.0) == 1.0 and approx(13.0) == 0.0 and approx(12.999) > 0.0
    xs = np.linspace(0, 12.99, 500)
    assert max(abs(approx(v) - math.exp(-v)) for v in xs) < 1e-3
    # frames whose entries lie more than 13 below the maximum contribute nothing at all
    far = np.array([[0.0, -13.0, -50.0]], f32)
    assert np.array_equal(oracle.logsoftmax_updateOutput(far), far)


def test_logsoftmax_backward_against_autograd_of_the_exact_function():
    rng = rng_for(83)
    x = rng.normal(size=(6, 40)).astype(f32)
    go = rng.normal(size=(6, 40)).astype(f32)
    tx = torch.from_numpy(x).double().requires_grad_(True)
    F.log_softmax(tx, dim=1).backward(torch.from_numpy(go).double())
    out = oracle.logsoftmax_updateOutput(x)
    gi = oracle.logsoftmax_updateGradInput(go, out)
    assert np.abs(gi - tx.grad.numpy()).max() < 5e-3
    # with the exact output the formula itself is exact to float rounding
    exact_out = F.log_softmax(tx, dim=1).detach().numpy().astype(f32)
    assert np.abs(oracle.logsoftmax_updateGradInput(go, exact_out) - tx.grad.numpy()).max() < 1e-5


@pytest.mark.parametrize("size_average", [True, False])
def test_classnll_against_torch(size_average):
    rng = rng_for(84)
    x = rng.normal(size=(9, 13)).astype(f32)
    target = rng.integers(1, 14, size=9)
    tx = torch.from_numpy(x).double().requires_grad_(True)
    loss = F.nll_loss(tx, torch.from_numpy(target - 1), reduction="mean" if size_average else "sum")
    assert abs(oracle.classnll_updateOutput(x, target, size_average) - float(loss)) < 1e-12
    loss.backward()
    assert np.array_equal(oracle.classnll_updateGradInput(x, target, size_average), tx.grad.numpy().astype(f32))
    assert oracle.classnll_updateOutput(x[2], target[2:3]) == -float(x[2, target[2] - 1])      # vector input
    g = oracle.classnll_updateGradInput(x[2], target[2:3])
    assert g[target[2] - 1] == -1 and np.count_nonzero(g) == 1

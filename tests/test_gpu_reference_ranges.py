"""The reference's own GPU-vs-CPU operator tests, with its parameter ranges, run against this library.

gpunn/test/test.lua:718-920 draws nn.SpatialConvolutionMM cases from `from in [1,32]`, `to in 8*[1,8]`, kernel sides
in [3,15], output sides in [1,64], stride 1, no padding, single images and batches of 2..16, fills inputs with
randn, and accepts a max ABSOLUTE error of 1e-3 (forward) / 1e-2 (backward, gradInput / gradWeight / gradBias)
(:2-3).  :1314-1528 does the same for nn.SpatialMaxPooling (planes in [1,64], windows 2..4, output sides 1..64,
batches 4..10) and requires the argmax indices to be equal; its overlapping variant (strides 1..4 against windows
2..4) is commented out there because the reference GPU backward cannot do it -- it runs here.
The reference seeds from os.time(); here the draws are seeded, 12 per test.  Both bars are applied: the
reference's absolute ones and this repository's (1e-4*sqrt(reduction length) norm-wise; pooling bit-exact)."""
import numpy as np
import pytest

from helpers import check_close, rng_for

pytestmark = pytest.mark.gpu

import oracle  # noqa: E402

PRECISION_FORWARD, PRECISION_BACKWARD = 1e-3, 1e-2        # gpunn/test/test.lua:2-3
DRAWS = 12


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def draw_conv(rng, batch):
    frm, to = int(rng.integers(1, 33)), int(rng.integers(1, 9)) * 8
    ki, kj = int(rng.integers(3, 16)), int(rng.integers(3, 16))
    outi, outj = int(rng.integers(1, 65)), int(rng.integers(1, 65))
    bs = None if not batch else int(batch(rng))
    return bs, frm, to, ki, kj, outi + ki - 1, outj + kj - 1      # ini = (outi-1)*si + ki with si = 1


def conv_case(gt, rng, cfg, mode):
    """Mirrors SpatialConvolutionMM_forward_* / _backward_*: CPU module = oracle, weights cloned to the GPU module."""
    bs, frm, to, ki, kj, ini, inj = cfg
    shape = (frm, inj, ini) if bs is None else (bs, frm, inj, ini)
    x = rng.standard_normal(shape).astype(np.float32)
    m = gt.nn.SpatialConvolutionMM(frm, to, ki, kj, 1, 1, rng=rng)           # nInputPlane, nOutputPlane, kW, kH, dW, dH
    w, b = np.array(m.weight), np.array(m.bias)
    xb = x if bs is not None else x[None]
    out_ref, cols = oracle.conv_updateOutput(xb, w, b, kj, ki, 0, 0, 1, 1)
    go = rng.standard_normal(out_ref.shape).astype(np.float32)
    gi_ref, _ = oracle.conv_updateGradInput(go, w, xb.shape, kj, ki, 0, 0, 1, 1)
    gw_ref, gb_ref = np.zeros_like(w), np.zeros_like(b)
    oracle.conv_accGradParameters(go, cols, gw_ref, gb_ref, 1.0)
    lib = gt._lib.lib
    before = lib.thgpu_conv_get_mode()
    assert lib.thgpu_conv_set_mode(mode) == 0
    try:
        m.gpu()
        dx = dev(gt, x)
        out = m.forward(dx).float()
        m.zeroGradParameters()
        gi = m.backward(dx, dev(gt, go if bs is not None else go[0])).float()
        gw, gb = m.gradWeight.float(), m.gradBias.float()
    finally:
        assert lib.thgpu_conv_set_mode(before) == 0
    if bs is None:
        out, gi = out[None], gi[None]
    # the reference's bars
    assert np.abs(out - out_ref).max() < PRECISION_FORWARD
    assert np.abs(gi - gi_ref).max() < PRECISION_BACKWARD
    assert np.abs(gw - gw_ref).max() < PRECISION_BACKWARD
    assert np.abs(gb - gb_ref).max() < PRECISION_BACKWARD
    # this repository's
    K, N, B = frm * ki * kj, out_ref.shape[2] * out_ref.shape[3], xb.shape[0]
    tag = "reference range conv b%s %d->%d k%dx%d in %dx%d mode%d " % (bs, frm, to, kj, ki, inj, ini, mode)
    check_close(tag + "output", out, out_ref, K)
    check_close(tag + "gradInput", gi, gi_ref, to * ki * kj)
    check_close(tag + "gradWeight", gw, gw_ref, B * N)
    check_close(tag + "gradBias", gb, gb_ref, B * N)


@pytest.mark.parametrize("mode", [0, 1], ids=["columns", "auto"])
@pytest.mark.parametrize("draw", range(DRAWS))
def test_conv_single_image_reference_ranges(gt, draw, mode):
    rng = rng_for(7000 + draw)
    conv_case(gt, rng, draw_conv(rng, None), mode)


@pytest.mark.parametrize("mode", [0, 1], ids=["columns", "auto"])
@pytest.mark.parametrize("draw", range(DRAWS))
def test_conv_batch_reference_ranges(gt, draw, mode):
    rng = rng_for(7100 + draw)
    # forward_batch draws bs in 2*[1,4], backward_batch in 4*[1,4] (test.lua:762,864): both, alternating
    batch = (lambda r: r.integers(1, 5) * 2) if draw % 2 == 0 else (lambda r: r.integers(1, 5) * 4)
    conv_case(gt, rng, draw_conv(rng, batch), mode)


def pool_case(gt, rng, overlapping, batch):
    frm = int(rng.integers(1, 65))
    ki, kj = int(rng.integers(2, 5)), int(rng.integers(2, 5))
    si, sj = (int(rng.integers(1, 5)), int(rng.integers(1, 5))) if overlapping else (ki, kj)
    outi, outj = int(rng.integers(1, 65)), int(rng.integers(1, 65))
    ini, inj = (outi - 1) * si + ki, (outj - 1) * sj + kj
    shape = (frm, inj, ini) if not batch else (int(rng.integers(4, 11)), frm, inj, ini)
    x = rng.standard_normal(shape).astype(np.float32)
    xb = x if batch else x[None]
    out_ref, ind_ref = oracle.maxpool_updateOutput(xb, kj, ki, sj, si)
    go = rng.standard_normal(out_ref.shape).astype(np.float32)
    gi_ref = oracle.maxpool_updateGradInput(go, ind_ref, xb.shape, sj, si)
    m = gt.nn.SpatialMaxPooling(ki, kj, si, sj).gpu()                        # kW, kH, dW, dH
    dx = dev(gt, x)
    out = m.forward(dx).float()
    ind = m.indices.float()
    gi = m.backward(dx, dev(gt, go if batch else go[0])).float()
    if not batch:
        out, gi, ind = out[None], gi[None], ind[:, None]
    assert np.abs(out - out_ref).max() < PRECISION_FORWARD and np.abs(ind - ind_ref).max() == 0    # the reference's
    assert np.abs(gi - gi_ref).max() < PRECISION_BACKWARD
    assert np.array_equal(bits(out), bits(out_ref)) and np.array_equal(bits(gi), bits(gi_ref))     # this repository's


@pytest.mark.parametrize("batch", [False, True], ids=["single", "batch"])
@pytest.mark.parametrize("overlapping", [False, True], ids=["stride=window", "strides 1..4"])
@pytest.mark.parametrize("draw", range(DRAWS))
def test_maxpool_reference_ranges(gt, draw, overlapping, batch):
    pool_case(gt, rng_for(7200 + draw), overlapping, batch)

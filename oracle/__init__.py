"""ctypes front end of the CPU oracle (oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke check and by the
cpu_baseline leg of bench.py.  Nothing in the product package imports it.

All arrays are C-contiguous float32 numpy arrays; shapes follow the reference
CPU nn path (NCHW, weight [M, C*kH*kW], finput [B, K, N], indices
[2, B, C, Ho, Wo]).
"""
import ctypes
import glob
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

_f32p = ctypes.POINTER(ctypes.c_float)
_c_long = ctypes.c_long
_c_int = ctypes.c_int
_c_float = ctypes.c_float


def build(force=False):
    """Compile liboracle.so with gcc (a few seconds)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-B", "-C", _HERE, "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _stale():
    """True when oracle.c was edited after liboracle.so was built."""
    src = os.path.join(_HERE, "oracle.c")
    return os.path.exists(src) and os.path.getmtime(src) > os.path.getmtime(_LIB_PATH)


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    elif _stale():
        build(force=True)
    lib = ctypes.CDLL(_LIB_PATH)
    ints = lambda n: [_c_int] * n
    lib.oracle_set_blas.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_set_threads.argtypes = [_c_int]
    lib.oracle_get_threads.restype = _c_int
    lib.oracle_sgemm.argtypes = [ctypes.c_char, ctypes.c_char, _c_long, _c_long, _c_long, _c_float,
                                 _f32p, _c_long, _f32p, _c_long, _c_float, _f32p, _c_long]
    lib.oracle_sgemv.argtypes = [ctypes.c_char, _c_long, _c_long, _c_float, _f32p, _c_long, _f32p, _c_long, _c_float,
                                 _f32p, _c_long]
    lib.oracle_sger.argtypes = [_c_long, _c_long, _c_float, _f32p, _c_long, _f32p, _c_long, _f32p, _c_long]
    lib.oracle_im2col.argtypes = [_f32p, _c_long] + ints(9) + [_f32p]
    lib.oracle_col2im.argtypes = [_f32p, _c_long] + ints(9) + [_f32p]
    lib.oracle_conv_updateOutput.argtypes = [_f32p, _c_long] + ints(3) + [_f32p, _f32p] + ints(7) + [_f32p, _f32p]
    lib.oracle_conv_updateGradInput.argtypes = [_f32p, _c_long] + ints(3) + [_f32p] + ints(7) + [_f32p, _f32p]
    lib.oracle_conv_accGradParameters.argtypes = [_f32p, _f32p, _c_long, _c_int, _c_long, _c_long, _c_float,
                                                  _f32p, _f32p]
    lib.oracle_maxpool_updateOutput.argtypes = [_f32p, _c_long] + ints(7) + [_f32p, _f32p]
    lib.oracle_maxpool_updateGradInput.argtypes = [_f32p, _f32p, _c_long] + ints(7) + [_f32p]
    lib.oracle_subsample_updateOutput.argtypes = [_f32p, _f32p, _f32p, _c_long] + ints(7) + [_f32p]
    lib.oracle_subsample_updateGradInput.argtypes = [_f32p, _f32p, _c_long] + ints(7) + [_f32p]
    lib.oracle_subsample_accGradParameters.argtypes = [_f32p, _f32p, _c_long] + ints(7) + [_c_float, _f32p, _f32p]
    lib.oracle_logsoftmax_updateOutput.argtypes = [_f32p, _c_long, _c_long, _f32p]
    lib.oracle_logsoftmax_updateGradInput.argtypes = [_f32p, _f32p, _c_long, _c_long, _f32p]
    lib.oracle_threshold_updateOutput.argtypes = [_f32p, _c_long, _c_float, _c_float, _f32p]
    lib.oracle_threshold_updateGradInput.argtypes = [_f32p, _f32p, _c_long, _c_float, _f32p]
    return lib


_lib = _load()
_blas_handle = None


def _p(a):
    assert a.dtype == np.float32 and a.flags["C_CONTIGUOUS"], "float32 C-contiguous array expected"
    return a.ctypes.data_as(_f32p)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def set_threads(n):
    _lib.oracle_set_threads(int(n))


def get_threads():
    return int(_lib.oracle_get_threads())


def use_blas(enable=True):
    """Route oracle_sgemm to an optimised sgemm_ found at run time (the
    reference's USE_BLAS build, TH/generic/THBlas.c:300-317) or back to the TH
    fallback loops.  Returns the backend's name."""
    global _blas_handle
    if not enable:
        _lib.oracle_set_blas(None, None)
        return "th-fallback-loops"
    try:
        import scipy
        cands = glob.glob(os.path.join(os.path.dirname(scipy.__file__), "..", "scipy.libs", "libscipy_openblas*.so*"))
    except ImportError:
        cands = []
    for path in cands:
        try:
            h = ctypes.CDLL(path)
            sg = ctypes.cast(h.scipy_sgemm_, ctypes.c_void_p)
            st = ctypes.cast(h.scipy_openblas_set_num_threads, ctypes.c_void_p)
        except (OSError, AttributeError):
            continue
        _blas_handle = h
        _lib.oracle_set_blas(sg, st)
        h.scipy_openblas_get_config.restype = ctypes.c_char_p
        return h.scipy_openblas_get_config().decode()
    _lib.oracle_set_blas(None, None)
    return "th-fallback-loops"


def conv_out_size(H, W, kH, kW, pH, pW, sH, sW):
    return (H + 2 * pH - kH) // sH + 1, (W + 2 * pW - kW) // sW + 1


def sgemm(transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    """Column-major BLAS sgemm on flat float32 arrays; c is updated in place."""
    _lib.oracle_sgemm(transa.encode(), transb.encode(), m, n, k, alpha, _p(a), lda, _p(b), ldb, beta, _p(c), ldc)
    return c


# ---- THTensor addmm / addmv / addr on row-major (C-contiguous) arrays -------------------------------
# TH sees a C-contiguous matrix as one whose SECOND dimension is contiguous, i.e. as the transpose of a
# column-major matrix; the dispatchers below make the BLAS calls TH/generic/THTensorMath.c makes for that case.
def addmm(beta, t, alpha, m1, m2):
    """r = beta*t + alpha*m1@m2 as THTensor_(addmm) (THTensorMath.c:458-561) computes it for contiguous
    operands: r has stride[1] == 1, so the operands are swapped and r^T = m2^T m1^T goes to gemm('n','n')."""
    t, m1, m2 = _f32(t), _f32(m1), _f32(m2)
    m, k = m1.shape
    k2, n = m2.shape
    assert k == k2 and t.shape == (m, n)
    r = t.copy()
    _lib.oracle_sgemm(b"n", b"n", n, m, k, alpha, _p(m2), n, _p(m1), k, beta, _p(r), n)
    return r


def addmv(beta, t, alpha, mat, vec):
    """r = beta*t + alpha*mat@vec as THTensor_(addmv) (THTensorMath.c:369-420): a C-contiguous mat has
    stride[1] == 1 and goes to gemv('t', n, m, ...)."""
    t, mat, vec = _f32(t), _f32(mat), _f32(vec)
    m, n = mat.shape
    assert vec.shape == (n,) and t.shape == (m,)
    r = t.copy()
    _lib.oracle_sgemv(b"t", n, m, alpha, _p(mat), n, _p(vec), 1, beta, _p(r), 1)
    return r


def addmv_t(beta, t, alpha, mat, vec):
    """r = beta*t + alpha*mat.T@vec for a C-contiguous mat: the transposed view has stride[0] == 1 and
    goes to gemv('n', ...) (THTensorMath.c:389-394)."""
    t, mat, vec = _f32(t), _f32(mat), _f32(vec)
    m, n = mat.shape
    assert vec.shape == (m,) and t.shape == (n,)
    r = t.copy()
    _lib.oracle_sgemv(b"n", n, m, alpha, _p(mat), n, _p(vec), 1, beta, _p(r), 1)
    return r


def addr(beta, t, alpha, vec1, vec2):
    """r = beta*t + alpha*outer(vec1, vec2) as THTensor_(addr) (THTensorMath.c:563-610): r scaled by beta
    first unless beta == 1, then ger with the vectors swapped because r has stride[1] == 1."""
    t, vec1, vec2 = _f32(t), _f32(vec1), _f32(vec2)
    m, n = vec1.shape[0], vec2.shape[0]
    assert t.shape == (m, n)
    r = t.copy()
    if beta != 1:
        r *= np.float32(beta)
    _lib.oracle_sger(n, m, alpha, _p(vec2), 1, _p(vec1), 1, _p(r), n)
    return r


# ---- nn.Linear on 2-D inputs, statement by statement (mcw_nn/Linear.lua:34-101) ------------------------
def linear_updateOutput(inp, weight, bias):
    inp, weight, bias = _f32(inp), _f32(weight), _f32(bias)
    nframe = inp.shape[0]
    out = addr(1.0, np.zeros((nframe, bias.shape[0]), np.float32), 1.0, np.ones(nframe, np.float32), bias)
    return addmm(1.0, out, 1.0, inp, np.ascontiguousarray(weight.T))


def linear_updateGradInput(gradOutput, weight):
    gradOutput, weight = _f32(gradOutput), _f32(weight)
    return addmm(0.0, np.zeros((gradOutput.shape[0], weight.shape[1]), np.float32), 1.0, gradOutput, weight)


def linear_accGradParameters(inp, gradOutput, gradWeight, gradBias, scale=1.0):
    """Accumulates into gradWeight / gradBias in place."""
    inp, gradOutput = _f32(inp), _f32(gradOutput)
    gradWeight[...] = addmm(1.0, gradWeight, scale, np.ascontiguousarray(gradOutput.T), inp)
    gradBias[...] = addmv_t(1.0, gradBias, scale, gradOutput, np.ones(inp.shape[0], np.float32))


def im2col(im, kH, kW, pH, pW, sH, sW):
    im = _f32(im)
    B, C, H, W = im.shape
    Ho, Wo = conv_out_size(H, W, kH, kW, pH, pW, sH, sW)
    col = np.empty((B, C * kH * kW, Ho * Wo), np.float32)
    _lib.oracle_im2col(_p(im), B, C, H, W, kH, kW, pH, pW, sH, sW, _p(col))
    return col


def col2im(col, C, H, W, kH, kW, pH, pW, sH, sW):
    col = _f32(col)
    B = col.shape[0]
    im = np.empty((B, C, H, W), np.float32)
    _lib.oracle_col2im(_p(col), B, C, H, W, kH, kW, pH, pW, sH, sW, _p(im))
    return im


def conv_updateOutput(inp, weight, bias, kH, kW, pH, pW, sH, sW):
    """Returns (output [B,M,Ho,Wo], finput [B,K,N])."""
    inp, weight, bias = _f32(inp), _f32(weight), _f32(bias)
    B, C, H, W = inp.shape
    M = weight.shape[0]
    assert weight.shape[1] == C * kH * kW
    Ho, Wo = conv_out_size(H, W, kH, kW, pH, pW, sH, sW)
    finput = np.empty((B, C * kH * kW, Ho * Wo), np.float32)
    out = np.empty((B, M, Ho, Wo), np.float32)
    _lib.oracle_conv_updateOutput(_p(inp), B, C, H, W, _p(weight), _p(bias), M, kH, kW, pH, pW, sH, sW,
                                  _p(finput), _p(out))
    return out, finput


def conv_updateGradInput(gradOutput, weight, in_shape, kH, kW, pH, pW, sH, sW):
    """Returns (gradInput [B,C,H,W], fgradInput [B,K,N])."""
    gradOutput, weight = _f32(gradOutput), _f32(weight)
    B, C, H, W = in_shape
    M = weight.shape[0]
    Ho, Wo = conv_out_size(H, W, kH, kW, pH, pW, sH, sW)
    assert gradOutput.shape == (B, M, Ho, Wo)
    fgi = np.zeros((B, C * kH * kW, Ho * Wo), np.float32)
    gi = np.empty((B, C, H, W), np.float32)
    _lib.oracle_conv_updateGradInput(_p(gradOutput), B, C, H, W, _p(weight), M, kH, kW, pH, pW, sH, sW,
                                     _p(fgi), _p(gi))
    return gi, fgi


def conv_accGradParameters(gradOutput, finput, gradWeight, gradBias, scale=1.0):
    """Accumulates into gradWeight [M,K] and gradBias [M] in place."""
    gradOutput, finput = _f32(gradOutput), _f32(finput)
    B, M = gradOutput.shape[:2]
    K, N = finput.shape[1:]
    assert gradWeight.shape == (M, K) and gradBias.shape == (M,)
    _lib.oracle_conv_accGradParameters(_p(gradOutput), _p(finput), B, M, K, N, scale, _p(gradWeight), _p(gradBias))
    return gradWeight, gradBias


def maxpool_updateOutput(inp, kH, kW, dH, dW):
    """Returns (output [B,C,Ho,Wo], indices [2,B,C,Ho,Wo] as float32, 1-based)."""
    inp = _f32(inp)
    B, C, H, W = inp.shape
    Ho, Wo = (H - kH) // dH + 1, (W - kW) // dW + 1
    out = np.empty((B, C, Ho, Wo), np.float32)
    ind = np.empty((2, B, C, Ho, Wo), np.float32)
    _lib.oracle_maxpool_updateOutput(_p(inp), B, C, H, W, kH, kW, dH, dW, _p(out), _p(ind))
    return out, ind


def maxpool_updateGradInput(gradOutput, indices, in_shape, dH, dW):
    gradOutput, indices = _f32(gradOutput), _f32(indices)
    B, C, H, W = in_shape
    Ho, Wo = gradOutput.shape[2:]
    gi = np.empty((B, C, H, W), np.float32)
    _lib.oracle_maxpool_updateGradInput(_p(gradOutput), _p(indices), B, C, H, W, Ho, Wo, dH, dW, _p(gi))
    return gi


def subsample_updateOutput(inp, weight, bias, kH, kW, dH, dW):
    """nn.SpatialSubSampling forward; weight=None gives nn.SpatialAveragePooling (a window sum)."""
    inp = _f32(inp)
    B, C, H, W = inp.shape
    Ho, Wo = (H - kH) // dH + 1, (W - kW) // dW + 1
    out = np.empty((B, C, Ho, Wo), np.float32)
    w = None if weight is None else _f32(weight)
    b = None if weight is None else _f32(bias)
    _lib.oracle_subsample_updateOutput(_p(inp), None if w is None else _p(w), None if b is None else _p(b),
                                       B, C, H, W, kH, kW, dH, dW, _p(out))
    return out


def subsample_updateGradInput(gradOutput, weight, in_shape, kH, kW, dH, dW):
    gradOutput = _f32(gradOutput)
    B, C, H, W = in_shape
    gi = np.empty((B, C, H, W), np.float32)
    w = None if weight is None else _f32(weight)
    _lib.oracle_subsample_updateGradInput(_p(gradOutput), None if w is None else _p(w), B, C, H, W, kH, kW, dH, dW,
                                          _p(gi))
    return gi


def subsample_accGradParameters(inp, gradOutput, gradWeight, gradBias, kH, kW, dH, dW, scale=1.0):
    """Accumulates into gradWeight / gradBias (float32 vectors of C elements) in place."""
    inp, gradOutput = _f32(inp), _f32(gradOutput)
    B, C, H, W = inp.shape
    assert gradWeight.dtype == np.float32 and gradBias.dtype == np.float32
    _lib.oracle_subsample_accGradParameters(_p(inp), _p(gradOutput), B, C, H, W, kH, kW, dH, dW, scale,
                                            _p(gradWeight), _p(gradBias))


def logsoftmax_updateOutput(inp):
    """nn.LogSoftMax forward on a vector or a matrix of frames."""
    inp = _f32(inp)
    assert inp.ndim in (1, 2)
    nframe, dim = (1, inp.shape[0]) if inp.ndim == 1 else inp.shape
    out = np.empty_like(inp)
    _lib.oracle_logsoftmax_updateOutput(_p(inp), nframe, dim, _p(out))
    return out


def logsoftmax_updateGradInput(gradOutput, output):
    gradOutput, output = _f32(gradOutput), _f32(output)
    nframe, dim = (1, output.shape[0]) if output.ndim == 1 else output.shape
    gi = np.empty_like(output)
    _lib.oracle_logsoftmax_updateGradInput(_p(gradOutput), _p(output), nframe, dim, _p(gi))
    return gi


def classnll_updateOutput(inp, target, sizeAverage=True):
    """nn.ClassNLLCriterion forward as the Lua module computes it on CPU tensors without class weights
    (mcw_nn/ClassNLLCriterion.lua:21-41): a Lua number (a double) accumulated frame after frame; target holds
    1-based class numbers."""
    inp = _f32(inp)
    target = np.asarray(target)
    if inp.ndim == 1:
        return -float(inp[int(target.ravel()[0]) - 1])
    output = 0.0
    for i in range(inp.shape[0]):
        output = output - float(inp[i, int(target[i]) - 1])
    if sizeAverage:
        output = output / inp.shape[0]
    return output


def classnll_updateGradInput(inp, target, sizeAverage=True):
    """mcw_nn/ClassNLLCriterion.lua:43-71: zeros with -1 (or -1/nframe) at the target positions."""
    inp = _f32(inp)
    target = np.asarray(target)
    gi = np.zeros_like(inp)
    if inp.ndim == 1:
        gi[int(target.ravel()[0]) - 1] = -1
        return gi
    z = -1.0
    if sizeAverage:
        z = z / inp.shape[0]
    for i in range(inp.shape[0]):
        gi[i, int(target[i]) - 1] = z
    return gi


def threshold_updateOutput(inp, threshold=0.0, val=0.0):
    inp = _f32(inp)
    out = np.empty_like(inp)
    _lib.oracle_threshold_updateOutput(_p(inp), inp.size, threshold, val, _p(out))
    return out


def threshold_updateGradInput(inp, gradOutput, threshold=0.0):
    inp, gradOutput = _f32(inp), _f32(gradOutput)
    gi = np.empty_like(inp)
    _lib.oracle_threshold_updateGradInput(_p(inp), _p(gradOutput), inp.size, threshold, _p(gi))
    return gi

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


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = ctypes.CDLL(_LIB_PATH)
    ints = lambda n: [_c_int] * n
    lib.oracle_set_blas.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
    lib.oracle_set_threads.argtypes = [_c_int]
    lib.oracle_get_threads.restype = _c_int
    lib.oracle_sgemm.argtypes = [ctypes.c_char, ctypes.c_char, _c_long, _c_long, _c_long, _c_float,
                                 _f32p, _c_long, _f32p, _c_long, _c_float, _f32p, _c_long]
    lib.oracle_im2col.argtypes = [_f32p, _c_long] + ints(9) + [_f32p]
    lib.oracle_col2im.argtypes = [_f32p, _c_long] + ints(9) + [_f32p]
    lib.oracle_conv_updateOutput.argtypes = [_f32p, _c_long] + ints(3) + [_f32p, _f32p] + ints(7) + [_f32p, _f32p]
    lib.oracle_conv_updateGradInput.argtypes = [_f32p, _c_long] + ints(3) + [_f32p] + ints(7) + [_f32p, _f32p]
    lib.oracle_conv_accGradParameters.argtypes = [_f32p, _f32p, _c_long, _c_int, _c_long, _c_long, _c_float,
                                                  _f32p, _f32p]
    lib.oracle_maxpool_updateOutput.argtypes = [_f32p, _c_long] + ints(7) + [_f32p, _f32p]
    lib.oracle_maxpool_updateGradInput.argtypes = [_f32p, _f32p, _c_long] + ints(7) + [_f32p]
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

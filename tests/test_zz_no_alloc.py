"""thgpu_gemm_noalloc, the entry point for callers that cannot allocate device memory, against THGPUBlas_gemm.

Both go through the C ABI on device pointers.  The shapes have few output tiles and a long reduction, so the
reduction is split and the partial sums go through the fixed device array (the per-kernel timing label says so).
Integer-valued operands make every fp32 sum exact: the two entry points must agree bit for bit with each other and
with the int64 product, whatever split either chose.  Float operands: within 1e-4*sqrt(k) of the fp64 product, the
bar every GEMM-backed result is held to.  Two calls in a row, the second on a smaller problem (the array still holds
the first call's partial sums), then the limits.
"""
import ctypes

import numpy as np
import pytest

from helpers import gemm_tol, rel_err, rng_for, uniform

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def ptr(gt, t):
    return gt._lib.lib.THGPUTensor_data(t._p)


def run_both(gt, ta, tb, m, n, k, alpha, a, lda, b, ldb, beta, c0, ldc):
    """Returns (THGPUBlas_gemm result, thgpu_gemm_noalloc result, timing labels of the no-alloc call)."""
    lib = gt._lib.lib
    da, db = dev(gt, a), dev(gt, b)
    c_ref, c_new = dev(gt, c0), dev(gt, c0)
    gt.gputorch.gemm(ta, tb, m, n, k, alpha, da, lda, db, ldb, beta, c_ref, ldc)
    gt.gputorch.synchronize()
    gt.gputorch.prof_reset()
    gt.gputorch.prof_enable(True)
    try:
        # the property the entry point exists for: no hipMalloc / hipFree by the library during the call, the block
        # cache untouched (the counter covers storage blocks, the growing split workspace and the offset tables)
        allocs, cached = lib.thgpu_device_alloc_calls(), lib.thgpu_cached_bytes()
        rc = lib.thgpu_gemm_noalloc(ta.encode(), tb.encode(), m, n, k, alpha, ptr(gt, da), lda, ptr(gt, db), ldb, beta,
                                    ptr(gt, c_new), ldc)
        gt._lib.check_status(rc)
        assert lib.thgpu_device_alloc_calls() == allocs and lib.thgpu_cached_bytes() == cached
        gt.gputorch.synchronize()
        labels = [key for key in gt.gputorch.prof_report() if key.startswith("gemm_blas_noalloc")]
    finally:
        gt.gputorch.prof_enable(False)
        gt.gputorch.prof_reset()
    return c_ref.float(), c_new.float(), labels


def problem(rng, ta, tb, m, n, k, integer):
    lda = (m if ta == "n" else k) + 1
    ldb = (k if tb == "n" else n) + 2
    ldc = m + 3
    draw = (lambda size: rng.integers(-3, 4, size=size).astype(np.float32)) if integer else (lambda size: uniform(rng, size))
    a = draw((lda * (k if ta == "n" else m),))
    b = draw((ldb * (n if tb == "n" else k),))
    c0 = draw((ldc * n,))
    A = a.reshape(-1, lda)[:, :(m if ta == "n" else k)].astype(np.float64)   # column-major: [col][row]
    B = b.reshape(-1, ldb)[:, :(k if tb == "n" else n)].astype(np.float64)
    opA = A.T if ta == "n" else A                                             # m x k
    opB = B.T if tb == "n" else B                                             # k x n
    return a, lda, b, ldb, c0, ldc, (opA @ opB).T                             # product as [n][m], like c


def split_of(labels):
    assert len(labels) == 1, labels
    return int(labels[0].split("split=")[1].split(" ")[0])


@pytest.mark.parametrize("ta,tb", [("n", "n"), ("t", "n"), ("n", "t"), ("t", "t")])
def test_noalloc_matches_blas_gemm_twice_second_smaller(gt, ta, tb):
    rng = rng_for(71)
    # (m, n, k): 16 and then 4 output tiles of 128 x 128 against 256 CUs -> the reduction is split
    for (m, n, k), integer in (((512, 521, 6000), True), ((300, 257, 4100), True), ((512, 521, 6000), False),
                               ((300, 257, 4100), False)):
        a, lda, b, ldb, c0, ldc, prod = problem(rng, ta, tb, m, n, k, integer)
        ref, got, labels = run_both(gt, ta, tb, m, n, k, 2.0, a, lda, b, ldb, 3.0, c0, ldc)
        assert split_of(labels) > 1, labels          # the fixed array was used
        want = c0.reshape(n, ldc).astype(np.float64).copy()
        want[:, :m] = 2.0 * prod + 3.0 * want[:, :m]
        if integer:
            assert np.array_equal(got, ref)
            assert np.array_equal(got.reshape(n, ldc), want.astype(np.float32))
        else:
            assert rel_err(got.reshape(n, ldc)[:, :m], want[:, :m]) < gemm_tol(k)
            assert rel_err(got.reshape(n, ldc)[:, :m], ref.reshape(n, ldc)[:, :m]) < gemm_tol(k)
            assert np.array_equal(got.reshape(n, ldc)[:, m:], c0.reshape(n, ldc)[:, m:])   # padding untouched


def test_noalloc_unsplit_and_small_problems(gt):
    rng = rng_for(72)
    for m, n, k in ((1024, 2048, 64), (7, 5, 11), (70, 45, 129)):       # many tiles: no split; below a tile: generic kernel
        a, lda, b, ldb, c0, ldc, prod = problem(rng, "n", "n", m, n, k, True)
        ref, got, labels = run_both(gt, "n", "n", m, n, k, 1.0, a, lda, b, ldb, 0.0, c0, ldc)
        assert np.array_equal(got, ref)
        assert np.array_equal(got.reshape(n, ldc)[:, :m], prod.astype(np.float32))


def test_noalloc_limits_and_quick_returns(gt):
    lib = gt._lib.lib
    d = dev(gt, np.zeros(16, np.float32))
    p = ptr(gt, d)
    cap = 16 << 20
    rc = lib.thgpu_gemm_noalloc(b"n", b"n", 8192, cap // 8192 + 1, 4, 1.0, p, 8192, p, 4, 0.0, p, 8192)
    assert rc != 0 and b"exceeds the limit" in lib.thgpu_last_error()
    assert d.float().tolist() == [0.0] * 16                  # rejected before anything was launched
    # the reference dispatcher's quick returns: nothing to do, status 0
    assert lib.thgpu_gemm_noalloc(b"n", b"n", 0, 4, 4, 1.0, p, 1, p, 4, 0.0, p, 1) == 0
    assert lib.thgpu_gemm_noalloc(b"n", b"n", 2, 2, 2, 0.0, p, 2, p, 2, 1.0, p, 2) == 0

"""GPU parity of the tensor math behind nn.Linear (THGPUTensor_addmm / addmv / addr / add / mul / div / cadd)
and of nn.Linear itself, through the C ABI, against the CPU oracle.

Bars: exact on small-integer data (every product and sum is exact in fp32, so any summation order must give
the same bits); otherwise max error relative to the largest reference magnitude below 1e-4*sqrt(reduction
length).
"""
import numpy as np
import pytest

from helpers import gemm_tol, rel_err, both_rel_err, rng_for, uniform

pytestmark = pytest.mark.gpu

import oracle  # noqa: E402


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def ints(rng, shape):
    return rng.integers(-3, 4, shape).astype(np.float32)


def view_of(gt, a, kind):
    """A device tensor with the values of `a` laid out as `kind`: dense, the transpose of a dense transposed
    copy (first dimension contiguous), or a window of a larger buffer (neither dimension contiguous... the
    column window keeps stride[1] == 1 but a row pitch larger than the row)."""
    if kind == "dense":
        return dev(gt, a)
    if kind == "transposed":
        return dev(gt, a.T).t()
    if kind == "window":
        big = np.full((a.shape[0] + 2, a.shape[1] + 3), 7.0, np.float32)
        big[1:1 + a.shape[0], 2:2 + a.shape[1]] = a
        return dev(gt, big).narrow(0, 1, a.shape[0]).narrow(1, 2, a.shape[1])
    if kind == "strided":            # every second column of a wider buffer: no dimension contiguous
        big = np.full((a.shape[0], 2 * a.shape[1]), 7.0, np.float32)
        big[:, ::2] = a
        wide = dev(gt, big)
        t = gt.GPUTensor(_ptr=gt._lib.lib.THGPUTensor_newWithStorage2d(
            gt._lib.lib.THGPUTensor_storage(wide._p), 0, a.shape[0], 2 * a.shape[1], a.shape[1], 2))
        t._keep = wide
        return t
    raise ValueError(kind)


KINDS = ["dense", "transposed", "window", "strided"]


@pytest.mark.parametrize("kr", KINDS)
@pytest.mark.parametrize("k1", KINDS)
@pytest.mark.parametrize("k2", ["dense", "transposed", "strided"])
def test_addmm_every_view_combination_exact(gt, kr, k1, k2):
    rng = rng_for(81)
    m, k, n = 9, 13, 7
    t, m1, m2 = ints(rng, (m, n)), ints(rng, (m, k)), ints(rng, (k, n))
    r = view_of(gt, t, kr)
    r.addmm(2.0, 3.0, view_of(gt, m1, k1), view_of(gt, m2, k2))
    assert np.array_equal(r.float(), 2 * t + 3 * (m1 @ m2))


@pytest.mark.parametrize("mnk", [(130, 70, 300), (64, 256, 100), (1, 9, 33), (257, 1, 17), (128, 4096, 1024)])
def test_addmm_tolerance_and_separate_result(gt, mnk):
    m, n, k = mnk
    rng = rng_for(82)
    t, m1, m2 = uniform(rng, (m, n)), uniform(rng, (m, k)), uniform(rng, (k, n))
    r = gt.GPUTensor()
    r.addmm(0.5, dev(gt, t), 1.5, dev(gt, m1), dev(gt, m2))          # r is resized to t and takes its values
    assert r.size() == (m, n)
    ref = 0.5 * t.astype(np.float64) + 1.5 * (m1.astype(np.float64) @ m2.astype(np.float64))
    assert both_rel_err(r.float(), ref) < gemm_tol(k)
    oracle.use_blas(k >= 1024)
    try:
        assert both_rel_err(r.float(), oracle.addmm(0.5, t, 1.5, m1, m2)) < gemm_tol(k)
    finally:
        oracle.use_blas(False)


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("vstride", [1, 3])
def test_addmv_views_exact(gt, kind, vstride):
    rng = rng_for(83)
    m, n = 11, 6
    mat, vec, t = ints(rng, (m, n)), ints(rng, (n,)), ints(rng, (m,))
    buf = np.full(n * vstride, 9.0, np.float32)
    buf[::vstride] = vec
    dvec = dev(gt, buf)
    if vstride != 1:
        v = gt.GPUTensor(_ptr=gt._lib.lib.THGPUTensor_newWithStorage1d(
            gt._lib.lib.THGPUTensor_storage(dvec._p), 0, n, vstride))
    else:
        v = dvec
    r = dev(gt, t)
    r.addmv(2.0, 3.0, view_of(gt, mat, kind), v)
    assert np.array_equal(r.float(), 2 * t + 3 * (mat @ vec))
    assert np.array_equal(r.float(), oracle.addmv(2.0, t, 3.0, mat, vec))


@pytest.mark.parametrize("kind", KINDS)
def test_addr_views_exact(gt, kind):
    rng = rng_for(84)
    m, n = 8, 5
    t, v1, v2 = ints(rng, (m, n)), ints(rng, (m,)), ints(rng, (n,))
    r = view_of(gt, t, kind)
    r.addr(2.0, 3.0, dev(gt, v1), dev(gt, v2))
    assert np.array_equal(r.float(), 2 * t + 3 * np.outer(v1, v2))
    assert np.array_equal(r.float(), oracle.addr(2.0, t, 3.0, v1, v2))


def test_scalar_ops_and_cadd_exact(gt):
    rng = rng_for(85)
    a, b = uniform(rng, (7, 33)), uniform(rng, (7, 33))
    x = dev(gt, a)
    assert np.array_equal(x.add(0.25).float(), a + np.float32(0.25))
    assert np.array_equal(x.mul(3.0).float(), (a + np.float32(0.25)) * np.float32(3.0))
    assert np.array_equal(x.div(7.0).float(), ((a + np.float32(0.25)) * np.float32(3.0)) / np.float32(7.0))
    y = dev(gt, a)
    y.add(0.5, dev(gt, b))
    assert np.array_equal(y.float(), a + np.float32(0.5) * b)        # a + value*b, one rounding each (no fma)
    z = view_of(gt, a, "transposed")
    z.add(dev(gt, b))
    assert np.array_equal(z.float(), a + b)


def test_math_argument_errors(gt):
    a, b = dev(gt, np.zeros((3, 4), np.float32)), dev(gt, np.zeros((5, 6), np.float32))
    with pytest.raises(gt.THGPUError, match="size mismatch"):
        dev(gt, np.zeros((3, 6), np.float32)).addmm(a, b)
    with pytest.raises(gt.THGPUError, match="matrix and vector expected"):
        dev(gt, np.zeros(3, np.float32)).addmv(a, a)
    with pytest.raises(gt.THGPUError, match="vector and vector expected"):
        a.addr(a, a)


@pytest.mark.parametrize("shape", [(6, 11, 5), (128, 300, 64), (3, 20, 1)])
def test_linear_fwd_bwd_matches_oracle(gt, shape):
    B, I, O = shape
    rng = rng_for(86)
    m = gt.nn.Linear(I, O, rng=np.random.default_rng(5))
    w, b = np.array(m.weight), np.array(m.bias)
    x, go = uniform(rng, (B, I)), uniform(rng, (B, O))
    gw0, gb0 = uniform(rng, (O, I)), uniform(rng, (O,))
    m.gpu()
    m.gradWeight.copy(gw0)
    m.gradBias.copy(gb0)
    dx, dgo = dev(gt, x), dev(gt, go)
    out = m.forward(dx).float()
    gi = m.backward(dx, dgo, 0.5).float()
    assert both_rel_err(out, oracle.linear_updateOutput(x, w, b)) < gemm_tol(I)
    assert both_rel_err(gi, oracle.linear_updateGradInput(go, w)) < gemm_tol(O)
    gw, gb = gw0.copy(), gb0.copy()
    oracle.linear_accGradParameters(x, go, gw, gb, 0.5)
    assert both_rel_err(m.gradWeight.float(), gw) < gemm_tol(B)
    assert both_rel_err(m.gradBias.float(), gb) < gemm_tol(B)


def test_linear_vector_input(gt):
    I, O = 17, 9
    rng = rng_for(87)
    m = gt.nn.Linear(I, O, rng=np.random.default_rng(6))
    w, b = np.array(m.weight), np.array(m.bias)
    x, go = uniform(rng, (I,)), uniform(rng, (O,))
    m.gpu()
    m.zeroGradParameters()
    out = m.forward(dev(gt, x)).float()
    gi = m.backward(dev(gt, x), dev(gt, go)).float()
    assert both_rel_err(out, oracle.addmv(1.0, b, 1.0, w, x)) < gemm_tol(I)
    assert both_rel_err(gi, oracle.addmv_t(0.0, np.zeros(I, np.float32), 1.0, w, go)) < gemm_tol(O)
    assert rel_err(m.gradWeight.float(), np.outer(go, x)) < 1e-6
    assert np.array_equal(m.gradBias.float(), go)


def test_alexnet_classifier_sizes(gt):
    """The classifier that follows the AlexNet-style conv stack at batch 128: 9216 -> 4096 -> 4096 -> 1000."""
    rng = rng_for(88)
    B = 128
    x = uniform(rng, (B, 9216))
    oracle.use_blas(True)
    try:
        for I, O in ((9216, 4096), (4096, 4096), (4096, 1000)):
            m = gt.nn.Linear(I, O, rng=np.random.default_rng(I + O))
            w, b = np.array(m.weight), np.array(m.bias)
            go = uniform(rng, (B, O))
            m.gpu()
            m.zeroGradParameters()
            dx = dev(gt, x)
            out = m.forward(dx).float()
            gi = m.backward(dx, dev(gt, go)).float()
            ref = oracle.linear_updateOutput(x, w, b)
            assert both_rel_err(out, ref) < gemm_tol(I)
            assert both_rel_err(gi, oracle.linear_updateGradInput(go, w)) < gemm_tol(O)
            gw, gb = np.zeros_like(w), np.zeros_like(b)
            oracle.linear_accGradParameters(x, go, gw, gb, 1.0)
            assert both_rel_err(m.gradWeight.float(), gw) < gemm_tol(B)
            assert both_rel_err(m.gradBias.float(), gb) < gemm_tol(B)
            x = np.maximum(ref, 0)
    finally:
        oracle.use_blas(False)


def test_unfold_squeeze_setstorage_views(gt):
    rng = rng_for(89)
    a = uniform(rng, (3, 1, 10, 1))
    t = dev(gt, a)
    assert t.squeeze().size() == (3, 10) and np.array_equal(t.squeeze().float(), a.reshape(3, 10))
    assert t.squeeze(1).size() == (3, 10, 1) and t.squeeze(0).size() == (3, 1, 10, 1)
    assert dev(gt, np.ones((1, 1), np.float32)).squeeze().size() == (1,)
    v = dev(gt, np.arange(10, dtype=np.float32))
    u = v.unfold(0, 4, 3)                      # windows [0..3], [3..6], [6..9]
    assert u.size() == (3, 4) and u.stride() == (3, 1)
    assert np.array_equal(u.float(), np.array([[0, 1, 2, 3], [3, 4, 5, 6], [6, 7, 8, 9]], np.float32))
    m = dev(gt, a.reshape(3, 10))
    u2 = m.unfold(1, 2, 4)                     # (3, 3, 2): columns {0,1}, {4,5}, {8,9}
    assert u2.size() == (3, 3, 2)
    assert np.array_equal(u2.float(), np.stack([a.reshape(3, 10)[:, [0, 1]], a.reshape(3, 10)[:, [4, 5]],
                                                a.reshape(3, 10)[:, [8, 9]]], axis=1))
    w = gt.GPUTensor()
    lib = gt._lib.lib
    lib.THGPUTensor_setStorage2d(w._p, lib.THGPUTensor_storage(m._p), 1, 3, 10, 4, 2)   # rows, every 2nd column from 1
    assert w.size() == (3, 4) and np.array_equal(w.float(), a.reshape(3, 10)[:, 1:9:2])
    with pytest.raises(gt.THGPUError, match="invalid step"):
        v.unfold(0, 2, 0)


@pytest.mark.parametrize("ta,tb", [("n", "n"), ("n", "t"), ("t", "n"), ("t", "t")])
@pytest.mark.parametrize("shared_b", [True, False])
def test_gemm_strided_batched(gt, ta, tb, shared_b):
    """Column-major C_i = beta*C_i + alpha*op(A_i)*op(B_i) for a batch; a shared B with op(A) = A takes the
    single-launch path of the convolution products, everything else one launch per problem."""
    rng = rng_for(90)
    m, n, k, batch = 70, 33, 129, 5
    A = ints(rng, (batch, k, m) if ta == "n" else (batch, m, k))       # column-major m x k (or k x m) per problem
    B = ints(rng, (1 if shared_b else batch, n, k) if tb == "n" else (1 if shared_b else batch, k, n))
    C = ints(rng, (batch, n, m))                                       # column-major m x n per problem
    dA, dB, dC = dev(gt, A), dev(gt, B), dev(gt, C)
    lib = gt._lib.lib
    rc = lib.thgpu_gemm_strided_batched(ta.encode(), tb.encode(), m, n, k, 2.0, lib.THGPUTensor_data(dA._p),
                                        m if ta == "n" else k, A[0].size, lib.THGPUTensor_data(dB._p),
                                        k if tb == "n" else n, 0 if shared_b else B[0].size, 3.0,
                                        lib.THGPUTensor_data(dC._p), m, m * n, batch)
    gt._lib.check_status(rc)
    got = dC.float()
    for i in range(batch):
        opA = A[i].T if ta == "n" else A[i]                            # m x k
        Bi = B[0 if shared_b else i]
        opB = Bi.T if tb == "n" else Bi                                # k x n
        assert np.array_equal(got[i].T, 3 * C[i].T + 2 * (opA @ opB)), i


def _ref_gemv(trans, m, n, alpha, a, lda, x, incx, beta, y, incy):
    """TH's fallback loops (TH/generic/THBlas.c:216-240) in float32, for the bit-for-bit comparisons."""
    a, x, y = a.copy(), x.copy(), y.copy()
    f = np.float32
    if trans == "t":
        for i in range(n):
            s = f(0)
            for j in range(m):
                s = f(s + f(x[j * incx] * a[j + i * lda]))
            y[i * incy] = f(f(beta * y[i * incy]) + f(alpha * s))
    else:
        if beta != 1:
            for i in range(m):
                y[i * incy] = f(beta * y[i * incy])
        for j in range(n):
            z = f(f(alpha) * x[j * incx])
            for i in range(m):
                y[i * incy] = f(y[i * incy] + f(z * a[i + j * lda]))
    return y


@pytest.mark.parametrize("trans", ["n", "t"])
@pytest.mark.parametrize("shape", [(1, 1), (5, 3), (70, 130), (257, 64), (3, 1), (1, 9)])
def test_blas_gemv_strided(gt, trans, shape):
    """THGPUBlas_gemv with padded leading dimension and strided vectors: 'n' bit for bit with TH's loop order,
    't' within 1e-4*sqrt(m) (its column sums are trees), both exact on integers."""
    m, n = shape
    rng = rng_for(71)
    lda, incx, incy = m + 3, 2, 3
    nx, ny = (n, m) if trans == "n" else (m, n)
    for integers in (False, True):
        draw = (lambda shp: rng.integers(-3, 4, size=shp).astype(np.float32)) if integers else (lambda shp: uniform(rng, shp))
        a, x, y = draw((lda * n,)), draw((nx * incx,)), draw((ny * incy,))
        alpha, beta = (2.0, -1.0) if integers else (0.75, 0.5)
        da, dx, dy = dev(gt, a), dev(gt, x), dev(gt, y)
        gt.gputorch.gemv(trans, m, n, alpha, da, lda, dx, incx, beta, dy, incy)
        got = dy.float()
        ref = _ref_gemv(trans, m, n, np.float32(alpha), a, lda if n != 1 else m, x, incx, np.float32(beta), y, incy)
        if trans == "n" or integers:
            assert np.array_equal(got, ref)
        else:
            assert np.max(np.abs(got - ref)) <= 1e-4 * np.sqrt(m) * max(1.0, np.max(np.abs(ref)))
        # elements between the strided ones are untouched
        mask = np.ones(ny * incy, bool)
        mask[::incy] = False
        assert np.array_equal(got[mask], y[mask])


def test_blas_ger_and_axpy(gt):
    rng = rng_for(72)
    m, n, lda, incx, incy = 37, 21, 40, 2, 3
    a, x, y = uniform(rng, (lda * n,)), uniform(rng, (m * incx,)), uniform(rng, (n * incy,))
    da = dev(gt, a)
    gt.gputorch.ger(m, n, 0.5, dev(gt, x), incx, dev(gt, y), incy, da, lda)
    ref = a.copy()
    f = np.float32
    for j in range(n):
        z = f(f(0.5) * y[j * incy])
        ref[j * lda:j * lda + m] = ref[j * lda:j * lda + m] + z * x[:m * incx:incx]
    assert np.array_equal(da.float(), ref)
    k = 1000
    u, v = uniform(rng, (k * 2,)), uniform(rng, (k * 3,))
    dv = dev(gt, v)
    gt.gputorch.axpy(k, 1.5, dev(gt, u), 2, dv, 3)
    ref = v.copy()
    ref[::3] = ref[::3] + f(1.5) * u[::2]
    assert np.array_equal(dv.float(), ref)


# ---- dot and the index operations (what Torch's generic tensor binding calls besides the above) ------------------
@pytest.mark.parametrize("n", [1, 5, 255, 4096, 4097, 100003, 5000000])
def test_dot_against_float64_and_exact_on_integers(gt, n):
    rng = rng_for(300 + n % 97)
    a, b = uniform(rng, (n,)), uniform(rng, (n,))
    ref = float(np.dot(a.astype(np.float64), b.astype(np.float64)))
    got = dev(gt, a).dot(dev(gt, b))
    scale = float(np.sum(np.abs(a.astype(np.float64) * b)))
    assert abs(got - ref) <= 1e-6 * scale + 1e-30
    assert dev(gt, a).dot(dev(gt, b)) == got                       # fixed summation shape: reruns are bit-identical
    ia, ib = ints(rng, (n,)), ints(rng, (n,))
    assert dev(gt, ia).dot(dev(gt, ib)) == float(np.dot(ia.astype(np.float64), ib))
    # a strided view and a matrix of the same element count (newContiguous on both sides)
    if n == 4096:
        m = uniform(rng, (64, 128))
        assert abs(dev(gt, m).t().dot(dev(gt, m.T.copy())) - float(np.sum(m.astype(np.float64) ** 2))) < 1e-3
    with pytest.raises(gt.THGPUError, match="size do not match"):
        dev(gt, a).dot(dev(gt, np.zeros(n + 1, np.float32)))


@pytest.mark.parametrize("shape,dim", [((7,), 0), ((5, 9), 0), ((5, 9), 1), ((3, 4, 6), 1), ((2, 3, 4, 5), 3)])
def test_index_select_copy_fill_bit_exact(gt, shape, dim):
    rng = rng_for(310 + len(shape) * 7 + dim)
    x = uniform(rng, shape)
    n = shape[dim]
    idx = rng.integers(1, n + 1, size=n + 2)                       # 1-based, repeats allowed
    got = dev(gt, x).index(dim, idx).float()
    assert np.array_equal(got, np.take(x, idx - 1, axis=dim))
    # a non-contiguous source
    if len(shape) == 2:
        got_t = dev(gt, x.T.copy()).t().index(dim, idx).float()
        assert np.array_equal(got_t, np.take(x, idx - 1, axis=dim))
    # indexCopy: distinct targets, slices of src in order
    perm = rng.permutation(n)[:max(1, n // 2)] + 1
    src_shape = list(shape)
    src_shape[dim] = len(perm)
    src = uniform(rng, src_shape)
    ref = x.copy()
    sl = [slice(None)] * len(shape)
    for k, p in enumerate(perm):
        sl[dim] = p - 1
        ss = list(sl)
        ss[dim] = k
        ref[tuple(sl)] = src[tuple(ss)]
    d = dev(gt, x)
    assert np.array_equal(d.indexCopy(dim, perm, dev(gt, src)).float(), ref)
    # indexFill
    ref2 = x.copy()
    for p in perm:
        sl[dim] = p - 1
        ref2[tuple(sl)] = 2.5
    assert np.array_equal(dev(gt, x).indexFill(dim, perm, 2.5).float(), ref2)
    with pytest.raises(gt.THGPUError, match="out of range"):
        dev(gt, x).index(dim, [n + 1])
    with pytest.raises(gt.THGPUError, match="out of bounds"):
        dev(gt, x).index(len(shape), [1])


def test_raw_memcpy_entry_points_round_trip(gt):
    import ctypes
    lib = gt._lib.lib
    x = uniform(rng_for(320), (1000,))
    d = gt.GPUTensor(1000)
    f32p = ctypes.POINTER(ctypes.c_float)
    assert lib.thgpu_memcpy_h2d(lib.THGPUTensor_data(d._p), x.ctypes.data_as(f32p), 1000) == 0
    back = np.zeros(1000, np.float32)
    assert lib.thgpu_memcpy_d2h(back.ctypes.data_as(f32p), lib.THGPUTensor_data(d._p), 1000) == 0
    assert np.array_equal(back, x) and np.array_equal(d.float(), x)
    assert lib.thgpu_memcpy_d2h(back.ctypes.data_as(f32p), None, 4) != 0 and b"null" in lib.thgpu_last_error()
    assert lib.thgpu_memcpy_h2d(None, x.ctypes.data_as(f32p), 0) == 0

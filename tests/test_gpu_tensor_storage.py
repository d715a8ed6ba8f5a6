"""GPU tests of THGPUStorage, THGPUTensor and the host<->device copies, through the C ABI.

What is pinned (all bit-exact: these are data-movement and bookkeeping functions):
  * storage: sizes, fill/get/set, resize keeps min(old, new) elements (gputorch/lib/THC/THCStorage.cpp:178-197),
    newWithData copies from a HOST pointer (:99-110), device-to-device and typed host copies;
  * tensor: the view algebra of TH/generic/THTensor.c (narrow / select / transpose / unfold / squeeze share the
    storage), resize never shrinks the storage (THCTensor.cpp:682-683), newContiguous hands back the same tensor
    when it already is contiguous (:186-195), fill/zero/copy through non-contiguous views, element get/set;
  * copies: :gpu() / :float() round trips of every host type, from and to non-contiguous host tensors
    (THCTensorCopy.cpp:20-80).
"""
import ctypes

import numpy as np
import pytest

from helpers import rng_for, uniform

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gt():
    import mcw_cppamp_torch_amd as pkg
    assert pkg._lib.lib.thgpu_init() == 0, pkg._lib.lib.thgpu_last_error()
    return pkg


def dev(gt, a):
    return gt.GPUTensor.from_numpy(np.ascontiguousarray(a, np.float32))


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


# ---- storage ---------------------------------------------------------------------------------------------------
def test_storage_basics_and_resize_keeps_prefix(gt):
    S = gt.gputorch.GPUStorage
    assert S().size() == 0 and S(0).size() == 0
    s = S(10).fill(2.5)
    assert s.size() == 10 and np.array_equal(s.float(), np.full(10, 2.5, np.float32))
    s[3] = -1.0
    assert s[3] == -1.0 and s[2] == 2.5
    host = np.arange(7, dtype=np.float32)
    t = S(host)                                   # newWithData: a host pointer, copied
    host[:] = 99
    assert np.array_equal(t.float(), np.arange(7, dtype=np.float32))
    t.resize(12)                                  # grow: the old 7 elements survive
    assert t.size() == 12 and np.array_equal(t.float()[:7], np.arange(7, dtype=np.float32))
    t.resize(4)                                   # shrink: the first 4 survive
    assert t.size() == 4 and np.array_equal(t.float(), np.arange(4, dtype=np.float32))
    t.resize(0)
    assert t.size() == 0 and t.float().size == 0
    with pytest.raises(gt.THGPUError):
        s[10]                                     # out of range
    with pytest.raises(gt.THGPUError):
        s[-1] = 0.0


def test_storage_copies_device_and_every_host_type(gt):
    S = gt.gputorch.GPUStorage
    rng = rng_for(101)
    a = S(uniform(rng, (33,)))
    b = S(33).copy(a)
    assert np.array_equal(bits(b.float()), bits(a.float()))
    with pytest.raises(gt.THGPUError):
        S(5).copy(a)                              # sizes must match
    for dtype in (np.uint8, np.int8, np.int16, np.int32, np.int64, np.float32, np.float64):
        src = rng.integers(0, 100, 33).astype(dtype)
        s = S(33).copy(src)
        assert np.array_equal(s.float(), src.astype(np.float32)), dtype
    # the reverse direction: every TH<Type>Storage_copyGPU
    lib = gt._lib.lib
    vals = np.arange(-5, 28, dtype=np.float32)
    s = S(vals)
    for kind, dtype in (("Byte", np.uint8), ("Char", np.int8), ("Short", np.int16), ("Int", np.int32),
                        ("Long", np.int64), ("Float", np.float32), ("Double", np.float64)):
        out = np.zeros(33, dtype)
        st = gt._lib.HostStorage[kind]()
        st.data = ctypes.cast(out.ctypes.data, ctypes.POINTER(gt._lib.HOST_TYPES[kind]))
        st.size = out.size
        getattr(lib, "TH%sStorage_copyGPU" % kind)(ctypes.byref(st), s._p)
        gt._lib.check()
        ref = vals.astype(dtype) if kind != "Byte" else vals.astype(np.int64).astype(np.uint8)
        assert np.array_equal(out, ref), kind


# ---- tensor bookkeeping ------------------------------------------------------------------------------------------
def test_tensor_resize_semantics(gt):
    t = gt.GPUTensor(4, 6)
    assert t.size() == (4, 6) and t.stride() == (6, 1) and t.isContiguous() and t.nElement() == 24
    st = t.storage()
    assert st.size() == 24
    t.fill(1.5)
    t.resize(2, 3)                                # smaller: the storage is kept as it is
    assert t.size() == (2, 3) and t.storage().size() == 24
    assert np.array_equal(t.float(), np.full((2, 3), 1.5, np.float32))
    t.resize(5, 5, 2)                             # larger: the storage grows and keeps its prefix
    assert t.size() == (5, 5, 2) and t.storage().size() == 50
    assert np.array_equal(t.float().ravel()[:24], np.full(24, 1.5, np.float32))
    t.resize(2, 3, 4, 5, 6)
    assert t.size() == (2, 3, 4, 5, 6) and t.stride() == (360, 120, 30, 6, 1)
    t.resize(1, 2, 1, 2, 1, 3)                    # six dimensions go through the LongStorage form
    assert t.size() == (1, 2, 1, 2, 1, 3)
    e = gt.GPUTensor()
    assert e.dim() == 0 and e.nElement() == 0 and e.storage() is None
    assert e.resizeAs(gt.GPUTensor(3, 2)).size() == (3, 2)


def test_views_share_storage_and_follow_th_algebra(gt):
    rng = rng_for(102)
    a = uniform(rng, (4, 5, 6))
    t = dev(gt, a)
    n = t.narrow(1, 1, 3)
    assert n.size() == (4, 3, 6) and n.stride() == (30, 6, 1) and n.storageOffset() == 6 and not n.isContiguous()
    assert np.array_equal(bits(n.float()), bits(a[:, 1:4, :]))
    s = t.select(2, 4)
    assert s.size() == (4, 5) and s.stride() == (30, 6) and s.storageOffset() == 4
    assert np.array_equal(bits(s.float()), bits(a[:, :, 4]))
    tr = t.transpose(0, 2)
    assert tr.size() == (6, 5, 4) and tr.stride() == (1, 6, 30)
    assert np.array_equal(bits(tr.float()), bits(a.transpose(2, 1, 0)))
    assert n.data_ptr() == t.data_ptr() + 6 * 4   # views alias the storage
    n.fill(7.0)                                   # fill through a non-contiguous view touches only the view
    back = t.float()
    ref = a.copy()
    ref[:, 1:4, :] = 7.0
    assert np.array_equal(bits(back), bits(ref))
    tr.select(0, 0).zero()
    ref[:, :, 0] = 0.0
    assert np.array_equal(bits(t.float()), bits(ref))
    with pytest.raises(gt.THGPUError):
        t.narrow(1, 3, 3)                         # runs past the dimension
    with pytest.raises(gt.THGPUError):
        t.select(3, 0)
    with pytest.raises(gt.THGPUError):
        dev(gt, a[0, 0]).select(0, 0)             # cannot select on a vector


def test_contiguous_clone_set_and_refcounts(gt):
    rng = rng_for(103)
    a = uniform(rng, (3, 7))
    t = dev(gt, a)
    c = t.contiguous()
    assert c._p and ctypes.addressof(c._p.contents) == ctypes.addressof(t._p.contents)   # same tensor, retained
    tt = t.t()
    cc = tt.contiguous()
    assert cc.isContiguous() and cc.data_ptr() != t.data_ptr()
    assert np.array_equal(bits(cc.float()), bits(a.T))
    cl = t.clone()
    assert cl.data_ptr() != t.data_ptr() and np.array_equal(bits(cl.float()), bits(a))
    v = gt.GPUTensor().set(tt)
    assert v.size() == (7, 3) and v.stride() == (1, 7) and v.data_ptr() == t.data_ptr()
    # a view keeps the storage alive after the tensor it came from is gone
    keep = dev(gt, a).narrow(0, 1, 2)
    import gc
    gc.collect()
    assert np.array_equal(bits(keep.float()), bits(a[1:3]))


def test_copy_between_views_and_shapes(gt):
    rng = rng_for(104)
    a, b = uniform(rng, (6, 8)), uniform(rng, (8, 6))
    dst = dev(gt, a)
    dst.copy(dev(gt, b).t())                      # strided source, same shape
    assert np.array_equal(bits(dst.float()), bits(b.T))
    dst = dev(gt, a)
    dst.t().copy(dev(gt, b))                      # strided destination
    assert np.array_equal(bits(dst.float()), bits(b.T))
    dst = dev(gt, a)
    dst.narrow(1, 2, 4).copy(dev(gt, b).narrow(0, 1, 6).narrow(1, 0, 4))     # both windows
    ref = a.copy()
    ref[:, 2:6] = b[1:7, 0:4]
    assert np.array_equal(bits(dst.float()), bits(ref))
    flat = gt.GPUTensor(48).copy(dev(gt, a))      # same element count, different shape: element order
    assert np.array_equal(bits(flat.float()), bits(a.ravel()))
    flat2 = gt.GPUTensor(48).copy(dev(gt, b).t())  # different shape and a strided source
    assert np.array_equal(bits(flat2.float()), bits(b.T.ravel()))
    win = dev(gt, np.zeros((10, 6), np.float32))
    win.narrow(0, 2, 8).copy(gt.GPUTensor(48).copy(dev(gt, a)))             # strided destination, other shape
    ref = np.zeros((10, 6), np.float32)
    ref[2:10] = a.reshape(8, 6)
    assert np.array_equal(bits(win.float()), bits(ref))
    with pytest.raises(gt.THGPUError):
        gt.GPUTensor(5).copy(dev(gt, a))
    # eight dimensions through the strided kernel
    big = uniform(rng, (2, 3, 2, 2, 3, 2, 2, 2))
    d8 = dev(gt, big).transpose(0, 7).transpose(2, 5)
    assert np.array_equal(bits(d8.contiguous().float()), bits(big.transpose(7, 1, 5, 3, 4, 2, 6, 0)))


def test_element_access(gt):
    a = np.arange(2 * 3 * 4 * 5, dtype=np.float32).reshape(2, 3, 4, 5)
    t = dev(gt, a)
    assert t[1, 2, 3, 4] == a[1, 2, 3, 4] and t[0, 0, 0, 0] == 0.0
    t[1, 0, 2, 1] = -3.5
    assert t.float()[1, 0, 2, 1] == -3.5
    v = t.select(0, 1).select(0, 2)               # 2-D view
    assert v[3, 4] == a[1, 2, 3, 4]
    v[0, 0] = 123.0
    assert t[1, 2, 0, 0] == 123.0
    with pytest.raises(gt.THGPUError):
        t[2, 0, 0, 0]
    with pytest.raises(gt.THGPUError):
        t[0, 0]                                   # wrong number of indices


# ---- host <-> device copies --------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [np.uint8, np.int8, np.int16, np.int32, np.int64, np.float32, np.float64])
def test_host_round_trip_every_type(gt, dtype):
    rng = rng_for(105)
    src = rng.integers(0, 120, (5, 7, 3)).astype(dtype)
    t = gt.GPUTensor(5, 7, 3).copy(src)
    assert np.array_equal(t.float(), src.astype(np.float32))
    out = np.empty((5, 7, 3), dtype)
    kind, th, keep = gt.gputorch._host_tensor_struct(out)
    getattr(gt._lib.lib, "TH%sTensor_copyGPU" % kind)(ctypes.byref(th), t._p)
    gt._lib.check()
    assert np.array_equal(out, src)


def test_float_round_trip_is_bit_exact_including_specials(gt):
    vals = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 3.4028235e38, 1.17549435e-38],
                    np.float32)
    big = np.random.default_rng(7).integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32).view(np.float32)
    for a in (vals, big):
        assert np.array_equal(bits(dev(gt, a).float()), bits(a))


def test_copies_with_non_contiguous_host_and_device_tensors(gt):
    rng = rng_for(106)
    base = uniform(rng, (9, 10))
    host_view = base[1:8:2, ::3]                  # strided host tensor (4 x 4)
    t = gt.GPUTensor(4, 4).copy(host_view)
    assert np.array_equal(bits(t.float()), bits(host_view))
    d = dev(gt, base)
    out = np.zeros((10, 9), np.float32)
    kind, th, keep = gt.gputorch._host_tensor_struct(out.T)     # strided host destination
    gt._lib.lib.THFloatTensor_copyGPU(ctypes.byref(th), d._p)
    gt._lib.check()
    assert np.array_equal(bits(out.T), bits(base))
    dv = d.narrow(0, 2, 5).t()                    # strided device source (10 x 5)
    assert np.array_equal(bits(dv.float()), bits(base[2:7].T))
    fresh = uniform(rng, (10, 5))
    dv.copy(fresh)                                # strided device destination from the host
    ref = base.copy()
    ref[2:7] = fresh.T
    assert np.array_equal(bits(d.float()), bits(ref))
    with pytest.raises(gt.THGPUError):
        gt.GPUTensor(3, 3).copy(base)             # sizes do not match
    assert d.double().dtype == np.float64 and np.array_equal(d.double(), ref.astype(np.float64))


def test_allocation_failure_is_reported_and_leaves_the_library_usable(gt):
    S = gt.gputorch.GPUStorage
    with pytest.raises(gt.THGPUError, match="hipMalloc"):
        S(1 << 46)                                # 256 TiB
    s = S(8).fill(1.0)
    with pytest.raises(gt.THGPUError, match="hipMalloc"):
        s.resize(1 << 46)
    assert s.size() == 8 and np.array_equal(s.float(), np.ones(8, np.float32))      # unchanged by the failed resize
    t = gt.GPUTensor(3, 3).fill(2.0)              # kernels still launch and check clean
    assert np.array_equal(t.float(), np.full((3, 3), 2.0, np.float32))
    with pytest.raises(gt.THGPUError):
        gt.GPUTensor(1 << 23, 1 << 23)


def test_storage_write_read_binary_and_ascii_known_answers(gt):
    """storage:write / :read (gputorch/torch/generic/Storage.c:180-201 over gputorch/Storage.cpp:14-31) against
    byte strings written out by hand from THDiskFile's formats: a native long and raw floats, or "%ld" / "%.9g"
    text with single spaces and a newline after each non-empty array."""
    import io
    import struct
    vals = [1.0, 2.5, -1.0 / 3.0, 1e-7, 16777216.0]
    st = gt.gputorch.GPUStorage(vals)
    f = io.BytesIO()
    st.write(f)
    assert f.getvalue() == struct.pack("<q", 5) + struct.pack("<5f", *vals)
    f = io.BytesIO()
    st.write(f, binary=False)
    assert f.getvalue() == b"5\n1 2.5 -0.333333343 1.00000001e-07 16777216\n"
    for binary in (True, False):
        f = io.BytesIO()
        st.write(f, binary=binary)
        gt.gputorch.GPUStorage().write(f, binary=binary)          # an empty storage after it
        gt.gputorch.GPUStorage([7.0]).write(f, binary=binary)
        f.seek(0)
        back = gt.gputorch.GPUStorage(3).read(f, binary=binary)
        assert back.size() == 5 and np.array_equal(back.float(), np.array(vals, np.float32))
        assert gt.gputorch.GPUStorage(2).read(f, binary=binary).size() == 0
        assert gt.gputorch.GPUStorage().read(f, binary=binary).float().tolist() == [7.0]
        assert f.read() == b""
    with pytest.raises(gt._lib.THGPUError):
        gt.gputorch.GPUStorage().read(io.BytesIO(struct.pack("<q", 4) + b"\0" * 8))
    with pytest.raises(gt._lib.THGPUError):
        gt.gputorch.GPUStorage().read(io.BytesIO(b"3\n1 2\n"), binary=False)


def test_fill_many_fills_every_tensor_in_one_call_and_rejects_views(gt):
    import ctypes
    L = gt._lib
    sizes = [(3, 5), (1,), (0,), (129, 7), (64, 363), (4097,)] + [(i + 1,) for i in range(40)]     # more than one launch's 32
    tensors = [gt.GPUTensor(*s) if s != (0,) else gt.GPUTensor() for s in sizes]
    for t in tensors:
        t.fill(7.0)
    guard = gt.GPUTensor(16)
    guard.fill(3.0)
    arr = (L.TensorP * len(tensors))(*[t._p for t in tensors])
    L.check_status(L.lib.thgpu_fill_many(arr, len(tensors), -1.5))
    for s, t in zip(sizes, tensors):
        if s != (0,):
            assert np.array_equal(t.float(), np.full(s, -1.5, np.float32)), s
    assert np.array_equal(guard.float(), np.full(16, 3.0, np.float32))
    view = tensors[3].narrow(1, 1, 3)                       # not contiguous: rejected before anything is written
    arr2 = (L.TensorP * 2)(tensors[0]._p, view._p)
    assert L.lib.thgpu_fill_many(arr2, 2, 9.0) != 0 and b"not contiguous" in L.lib.thgpu_last_error()
    assert np.array_equal(tensors[0].float(), np.full((3, 5), -1.5, np.float32))
    # nn.Sequential:zeroGradParameters goes through it
    nn = gt.nn
    net = nn.Sequential().add(nn.SpatialConvolutionMM(3, 4, 3, 3)).add(nn.ReLU()).add(nn.SpatialConvolutionMM(4, 5, 3, 3)).gpu()
    for m in (net.get(0), net.get(2)):
        m.gradWeight.fill(2.0)
        m.gradBias.fill(2.0)
    net.zeroGradParameters()
    for m in (net.get(0), net.get(2)):
        assert not m.gradWeight.float().any() and not m.gradBias.float().any()


def test_released_blocks_are_reused_without_a_device_free(gt):
    """A released storage buffer is handed to the next request of the same size (same device address, contents of
    the new owner intact although the old owner's work was still queued), other sizes get other blocks, and
    thgpu_empty_cache returns everything to the device."""
    lib = gt._lib.lib
    assert lib.thgpu_empty_cache() == 0 and lib.thgpu_cached_bytes() == 0
    n = 1 << 20
    a = gt.GPUTensor(n).fill(1.5)
    addr = lib.THGPUTensor_data(a._p)
    addr = ctypes_addr(addr)
    del a
    import gc
    gc.collect()
    assert lib.thgpu_cached_bytes() == 4 * n
    b = gt.GPUTensor(n // 2).fill(2.5)          # another size: a fresh block
    assert ctypes_addr(lib.THGPUTensor_data(b._p)) != addr
    c = gt.GPUTensor(n).fill(3.5)               # the same size: the kept block, ordered after the old owner's fill
    assert ctypes_addr(lib.THGPUTensor_data(c._p)) == addr and lib.thgpu_cached_bytes() == 0
    assert np.all(c.float() == 3.5) and np.all(b.float() == 2.5)
    c.resize(n + 7)                             # a resize keeps the prefix and releases the old block
    assert np.all(c.float()[:n] == 3.5) and lib.thgpu_cached_bytes() == 4 * n
    assert lib.thgpu_empty_cache() == 0 and lib.thgpu_cached_bytes() == 0


def ctypes_addr(p):
    import ctypes
    return ctypes.cast(p, ctypes.c_void_p).value

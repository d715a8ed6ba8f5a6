"""Host-side mirror of the `gputorch` package: torch.GPUStorage / torch.GPUTensor
objects over the C ABI, with the :gpu() / :float() / :double() conversions of
gputorch/Tensor.lua:7-40 and the copy dispatch of gputorch/Tensor.cpp:38-65.

Host tensors (torch.FloatTensor / torch.DoubleTensor in the reference) are
numpy arrays here; `FloatTensor` is an ndarray subclass that adds .gpu().
"""
import ctypes
import json

import numpy as np

from . import _lib
from ._lib import THGPUError, lib

_NP_TO_TH = {
    np.dtype(np.uint8): "Byte", np.dtype(np.int8): "Char", np.dtype(np.int16): "Short",
    np.dtype(np.int32): "Int", np.dtype(np.int64): "Long", np.dtype(np.float32): "Float",
    np.dtype(np.float64): "Double",
}


class FloatTensor(np.ndarray):
    """numpy float32 array with the reference's conversion methods."""

    def __new__(cls, *shape):
        if len(shape) == 1 and not np.isscalar(shape[0]):
            return np.ascontiguousarray(shape[0], dtype=np.float32).view(cls)
        return np.zeros(shape, np.float32).view(cls)

    def gpu(self):
        return GPUTensor.from_numpy(self)

    def float(self):
        return self

    def double(self):
        return np.asarray(self, np.float64)


def _host_tensor_struct(arr):
    """Builds a TH<Type>Tensor view (strides in elements) over a numpy array.
    Returns (struct, keepalive)."""
    kind = _NP_TO_TH.get(arr.dtype)
    if kind is None:
        raise TypeError("unsupported host dtype %s" % arr.dtype)
    St, Te = _lib.HostStorage[kind], _lib.HostTensor[kind]
    nd = arr.ndim
    if any(s % arr.itemsize for s in arr.strides) or any(s < 0 for s in arr.strides):
        arr = np.ascontiguousarray(arr)
    sizes = (ctypes.c_long * max(nd, 1))(*arr.shape)
    strides = (ctypes.c_long * max(nd, 1))(*[s // arr.itemsize for s in arr.strides])
    # A storage that spans the addressed range, starting at element 0 of the view.
    span = 1 + sum((n - 1) * (s // arr.itemsize) for n, s in zip(arr.shape, arr.strides)) if arr.size else 0
    storage = St()
    storage.data = ctypes.cast(arr.ctypes.data, ctypes.POINTER(_lib.HOST_TYPES[kind]))
    storage.size = span
    storage.refcount = 1
    storage.flag = 0
    tensor = Te()
    tensor.size = ctypes.cast(sizes, _lib.longp)
    tensor.stride = ctypes.cast(strides, _lib.longp)
    tensor.nDimension = nd if arr.size else 0
    tensor.storage = ctypes.pointer(storage)
    tensor.storageOffset = 0
    tensor.refcount = 1
    tensor.flag = 0
    return kind, tensor, (arr, sizes, strides, storage)


def _ascii_tokens(f, n):
    """Reads n whitespace-separated tokens from a byte stream, then the newline that follows a non-empty array
    (the auto-spacing of THDiskFile's ASCII mode, mcw_torch7_core/lib/TH/THDiskFile.c:55-68)."""
    out = []
    while len(out) < n:
        tok = b""
        while True:
            c = f.read(1)
            if not c:
                break
            if c.isspace():
                if tok:
                    break
                continue
            tok += c
        if not tok:
            raise _lib.THGPUError("read error: read %d blocks instead of %d" % (len(out), n))
        out.append(tok)
        last = c
    if n > 0 and last not in (b"\n", b""):
        f.seek(-1, 1)   # only a newline right after the last element belongs to the array
    return out


class GPUStorage(object):
    """torch.GPUStorage (gputorch/Storage.cpp, gputorch/lib/THC/THCStorage.cpp)."""

    def __init__(self, arg=None, _ptr=None):
        if _ptr is not None:
            self._p = _ptr
        elif arg is None:
            self._p = lib.THGPUStorage_new()
        elif np.isscalar(arg):
            self._p = lib.THGPUStorage_newWithSize(int(arg))
        else:
            host = np.ascontiguousarray(arg, dtype=np.float32).ravel()
            self._p = lib.THGPUStorage_newWithData(host.ctypes.data_as(_lib.f32p), host.size)
        _lib.check()

    def __del__(self):
        p, self._p = getattr(self, "_p", None), None
        if p:
            lib.THGPUStorage_free(p)

    def size(self):
        return int(lib.THGPUStorage_size(self._p))

    __len__ = size

    def resize(self, n):
        lib.THGPUStorage_resize(self._p, int(n))
        _lib.check()
        return self

    def fill(self, v):
        lib.THGPUStorage_fill(self._p, float(v))
        _lib.check()
        return self

    def __getitem__(self, i):  # 0-based, unlike Lua
        v = lib.THGPUStorage_get(self._p, int(i))
        _lib.check()
        return float(v)

    def __setitem__(self, i, v):
        lib.THGPUStorage_set(self._p, int(i), float(v))
        _lib.check()

    def copy(self, src):
        if isinstance(src, GPUStorage):
            lib.THGPUStorage_copy(self._p, src._p)
        else:
            host = np.ascontiguousarray(src).ravel()
            kind = _NP_TO_TH.get(host.dtype)
            if kind is None:
                raise TypeError("unsupported host dtype %s" % host.dtype)
            st = _lib.HostStorage[kind]()
            st.data = ctypes.cast(host.ctypes.data, ctypes.POINTER(_lib.HOST_TYPES[kind]))
            st.size = host.size
            getattr(lib, "THGPUStorage_copy%s" % kind)(self._p, ctypes.byref(st))
        _lib.check()
        return self

    def write(self, f, binary=True):
        """storage:write(file): the element count as a long, then the floats staged through host memory
        (gputorch/torch/generic/Storage.c:180-189 with the THFile_writeRealRaw of gputorch/Storage.cpp:23-31), in
        the disk file's native binary encoding or its ASCII mode ("%ld", "%.9g", elements separated by one space, a
        newline after each non-empty array: mcw_torch7_core/lib/TH/THDiskFile.c:88-130,304-310).  `f` is a file
        object opened for writing bytes."""
        host = self.float()
        if binary:
            f.write(np.int64(host.size).tobytes())
            f.write(host.tobytes())
        else:
            f.write(b"%d\n" % host.size)
            if host.size:
                f.write(" ".join("%.9g" % float(v) for v in host).encode("ascii") + b"\n")
        return self

    def read(self, f, binary=True):
        """storage:read(file): the inverse of write (gputorch/torch/generic/Storage.c:191-201,
        gputorch/Storage.cpp:14-21); resizes the storage to the stored element count."""
        if binary:
            head = f.read(8)
            if len(head) != 8:
                raise _lib.THGPUError("read error: read 0 blocks instead of 1")
            n = int(np.frombuffer(head, np.int64)[0])
            raw = f.read(4 * n)
            if n < 0 or len(raw) != 4 * n:
                raise _lib.THGPUError("read error: read %d blocks instead of %d" % (len(raw) // 4, n))
            host = np.frombuffer(raw, np.float32)
        else:
            n = int(_ascii_tokens(f, 1)[0])
            host = np.array([float(t) for t in _ascii_tokens(f, n)], np.float32)
        self.resize(n)
        if n:
            self.copy(host)
        return self

    def float(self):
        out = np.empty(self.size(), np.float32)
        st = _lib.HostStorage["Float"]()
        st.data = out.ctypes.data_as(_lib.f32p)
        st.size = out.size
        lib.THFloatStorage_copyGPU(ctypes.byref(st), self._p)
        _lib.check()
        return out


class GPUTensor(object):
    """torch.GPUTensor (gputorch/Tensor.cpp, gputorch/lib/THC/THCTensor.cpp)."""

    def __init__(self, *sizes, **kw):
        ptr = kw.pop("_ptr", None)
        if ptr is not None:
            self._p = ptr
        else:
            self._p = lib.THGPUTensor_new()
            _lib.check()
            if len(sizes) == 1 and not np.isscalar(sizes[0]):
                sizes = tuple(sizes[0])
            if sizes:
                self.resize(*sizes)

    def __del__(self):
        p, self._p = getattr(self, "_p", None), None
        if p:
            lib.THGPUTensor_free(p)

    # ---- construction / conversion ------------------------------------------
    @classmethod
    def from_numpy(cls, arr):
        arr = np.asarray(arr)
        t = cls()
        if arr.size:
            t.resize(*arr.shape)
            t.copy(arr)
        return t

    def gpu(self):
        return self

    def float(self):
        """Blocking device-to-host copy into a float32 array (Tensor:float())."""
        return self._to_host(np.float32)

    def double(self):
        return self._to_host(np.float64)

    def _to_host(self, dtype):
        out = np.empty(self.size(), dtype)
        if out.size:
            kind, th, keep = _host_tensor_struct(out)
            getattr(lib, "TH%sTensor_copyGPU" % kind)(ctypes.byref(th), self._p)
            _lib.check()
        return out.view(FloatTensor) if dtype == np.float32 else out

    def type(self, name=None):
        if name is None:
            return "torch.GPUTensor"
        if name == "torch.GPUTensor":
            return self
        if name == "torch.FloatTensor":
            return self.float()
        if name == "torch.DoubleTensor":
            return self.double()
        raise THGPUError("unknown tensor type %s" % name)

    # ---- shape ----------------------------------------------------------------
    def dim(self):
        return int(self._p.contents.nDimension)

    nDimension = dim

    def size(self, d=None):
        c = self._p.contents
        if d is None:
            return tuple(int(c.size[i]) for i in range(c.nDimension))
        v = lib.THGPUTensor_size(self._p, int(d))
        _lib.check()
        return int(v)

    def stride(self, d=None):
        c = self._p.contents
        if d is None:
            return tuple(int(c.stride[i]) for i in range(c.nDimension))
        v = lib.THGPUTensor_stride(self._p, int(d))
        _lib.check()
        return int(v)

    @property
    def shape(self):
        return self.size()

    def nElement(self):
        return int(lib.THGPUTensor_nElement(self._p))

    def isContiguous(self):
        return bool(lib.THGPUTensor_isContiguous(self._p))

    def storageOffset(self):
        return int(lib.THGPUTensor_storageOffset(self._p))

    def storage(self):
        sp = lib.THGPUTensor_storage(self._p)
        if not sp:
            return None
        lib.THGPUStorage_retain(sp)
        return GPUStorage(_ptr=sp)

    def data_ptr(self):
        p = lib.THGPUTensor_data(self._p)
        return ctypes.cast(p, ctypes.c_void_p).value or 0

    def resize(self, *sizes):
        if len(sizes) == 1 and not np.isscalar(sizes[0]):
            sizes = tuple(sizes[0])
        n = len(sizes)
        if n == 0:
            return self
        if n <= 5:
            getattr(lib, "THGPUTensor_resize%dd" % n)(self._p, *[int(s) for s in sizes])
        else:
            arr = (ctypes.c_long * n)(*sizes)
            st = _lib.THLongStorage()
            st.data = ctypes.cast(arr, _lib.longp)
            st.size = n
            lib.THGPUTensor_resize(self._p, ctypes.byref(st), None)
        _lib.check()
        return self

    def resizeAs(self, other):
        lib.THGPUTensor_resizeAs(self._p, other._p)
        _lib.check()
        return self

    def _view(self, ptr):
        _lib.check()
        return GPUTensor(_ptr=ptr)

    def select(self, dim, index):
        return self._view(lib.THGPUTensor_newSelect(self._p, int(dim), int(index)))

    def narrow(self, dim, first, size):
        return self._view(lib.THGPUTensor_newNarrow(self._p, int(dim), int(first), int(size)))

    def transpose(self, d1, d2):
        return self._view(lib.THGPUTensor_newTranspose(self._p, int(d1), int(d2)))

    def unfold(self, dim, size, step):
        return self._view(lib.THGPUTensor_newUnfold(self._p, int(dim), int(size), int(step)))

    def squeeze(self, dim=None):
        t = self._view(lib.THGPUTensor_newWithTensor(self._p))
        if dim is None:
            lib.THGPUTensor_squeeze(t._p, None)
        else:
            lib.THGPUTensor_squeeze1d(t._p, None, int(dim))
        _lib.check()
        return t

    def view(self, *sizes):
        """tensor:view(sizes) (mcw_torch7_core/Tensor.lua: a new tensor on the same storage; the tensor must be
        contiguous and the element count must match)."""
        if len(sizes) == 1 and not np.isscalar(sizes[0]):
            sizes = tuple(sizes[0])
        sizes = [int(v) for v in sizes]
        if sizes.count(-1) == 1:                  # one dimension may be left for view to work out
            known = int(np.prod([v for v in sizes if v != -1], dtype=np.int64))
            if known > 0 and self.nElement() % known == 0:
                sizes[sizes.index(-1)] = self.nElement() // known
        if not self.isContiguous():
            raise THGPUError("expecting a contiguous tensor")
        if int(np.prod(sizes, dtype=np.int64)) != self.nElement():
            raise THGPUError("Wrong size for view. Input size: %d. Output size: %s" % (self.nElement(), "x".join(map(str, sizes))))
        arr = (ctypes.c_long * len(sizes))(*sizes)
        st = _lib.THLongStorage()
        st.data = ctypes.cast(arr, _lib.longp)
        st.size = len(sizes)
        return self._view(lib.THGPUTensor_newWithStorage(lib.THGPUTensor_storage(self._p), self.storageOffset(),
                                                         ctypes.byref(st), None))

    def viewAs(self, other):
        return self.view(*other.size())

    def contiguous(self):
        return self._view(lib.THGPUTensor_newContiguous(self._p))

    def clone(self):
        return self._view(lib.THGPUTensor_newClone(self._p))

    def set(self, other):
        lib.THGPUTensor_set(self._p, other._p)
        _lib.check()
        return self

    # ---- content --------------------------------------------------------------
    def fill(self, v):
        lib.THGPUTensor_fill(self._p, float(v))
        _lib.check()
        return self

    def zero(self):
        lib.THGPUTensor_zero(self._p)
        _lib.check()
        return self

    def copy(self, src):
        """Tensor:copy(src) with the type dispatch of gputorch/Tensor.cpp:38-65."""
        if isinstance(src, GPUTensor):
            lib.THGPUTensor_copy(self._p, src._p)
        else:
            src = np.asarray(src)
            if src.dtype not in _NP_TO_TH:
                src = src.astype(np.float32)
            kind, th, keep = _host_tensor_struct(src)
            getattr(lib, "THGPUTensor_copy%s" % kind)(self._p, ctypes.byref(th))
        _lib.check()
        return self

    # ---- math (the overloads of the Lua methods, gputorch/TensorMath.cpp wrap of THCTensorMath.h) ----
    def t(self):
        assert self.dim() == 2, "t() expects a matrix"
        return self.transpose(0, 1)

    def add(self, *args):
        """x:add(value) | x:add(y) | x:add(value, y)  (value defaults to 1)."""
        if len(args) == 1 and not isinstance(args[0], GPUTensor):
            lib.THGPUTensor_add(self._p, self._p, float(args[0]))
        else:
            value, other = (1.0, args[0]) if len(args) == 1 else (float(args[0]), args[1])
            lib.THGPUTensor_cadd(self._p, self._p, value, other._p)
        _lib.check()
        return self

    def mul(self, value):
        lib.THGPUTensor_mul(self._p, self._p, float(value))
        _lib.check()
        return self

    def div(self, value):
        lib.THGPUTensor_div(self._p, self._p, float(value))
        _lib.check()
        return self

    @staticmethod
    def _blas_args(args, ntensors):
        """([beta,] [alpha,] [t,] a, b) -> beta, alpha, t-or-None, a, b as the Lua methods accept them."""
        nums = [float(a) for a in args if not isinstance(a, GPUTensor)]
        tens = [a for a in args if isinstance(a, GPUTensor)]
        assert len(nums) <= 2 and len(tens) in (ntensors, ntensors + 1), "bad arguments"
        beta, alpha = (1.0, 1.0) if not nums else (1.0, nums[0]) if len(nums) == 1 else (nums[0], nums[1])
        t = tens[0] if len(tens) == ntensors + 1 else None
        return beta, alpha, t, tens[-2], tens[-1]

    def addmm(self, *args):
        beta, alpha, t, m1, m2 = self._blas_args(args, 2)
        lib.THGPUTensor_addmm(self._p, beta, (t or self)._p, alpha, m1._p, m2._p)
        _lib.check()
        return self

    def addmv(self, *args):
        beta, alpha, t, mat, vec = self._blas_args(args, 2)
        lib.THGPUTensor_addmv(self._p, beta, (t or self)._p, alpha, mat._p, vec._p)
        _lib.check()
        return self

    def addr(self, *args):
        beta, alpha, t, v1, v2 = self._blas_args(args, 2)
        lib.THGPUTensor_addr(self._p, beta, (t or self)._p, alpha, v1._p, v2._p)
        _lib.check()
        return self

    def dot(self, other):
        """torch.dot / the `*` of two vectors (gputorch/torch/generic/TensorOperator.c:120)."""
        v = lib.THGPUTensor_dot(self._p, other._p)
        _lib.check()
        return float(v)

    @staticmethod
    def _index_vector(index):
        # a host LongTensor of 1-based indices, as the Lua methods take (gputorch/torch/generic/Tensor.c:393-456)
        arr = np.ascontiguousarray(np.asarray(index, np.int64).reshape(-1))
        return _host_tensor_struct(arr)

    def index(self, dim, index):
        """tensor:index(dim, index): a new tensor of the slices `index` names along `dim` (0-based here, entries of
        `index` 1-based as in Lua)."""
        _, th, keep = self._index_vector(index)
        out = GPUTensor()
        lib.THGPUTensor_indexSelect(out._p, self._p, dim, ctypes.byref(th))
        _lib.check()
        return out

    def indexCopy(self, dim, index, src):
        _, th, keep = self._index_vector(index)
        lib.THGPUTensor_indexCopy(self._p, dim, ctypes.byref(th), src._p)
        _lib.check()
        return self

    def indexFill(self, dim, index, value):
        _, th, keep = self._index_vector(index)
        lib.THGPUTensor_indexFill(self._p, dim, ctypes.byref(th), float(value))
        _lib.check()
        return self

    def __getitem__(self, idx):  # 0-based element access (slow, blocking)
        if np.isscalar(idx):
            idx = (idx,)
        fn = getattr(lib, "THGPUTensor_get%dd" % len(idx))
        v = fn(self._p, *[int(i) for i in idx])
        _lib.check()
        return float(v)

    def __setitem__(self, idx, value):
        if np.isscalar(idx):
            idx = (idx,)
        getattr(lib, "THGPUTensor_set%dd" % len(idx))(self._p, *([int(i) for i in idx] + [float(value)]))
        _lib.check()

    def __repr__(self):
        return "GPUTensor(size=%s)" % (self.size(),)


# ---- package-level functions (gputorch/init.cpp:10-94) -------------------------
def synchronize():
    _lib.check_status(lib.thgpu_synchronize())


def getDeviceCount():
    return 1 if lib.thgpu_init() == 0 else 0


def getDeviceProperties():
    name = ctypes.create_string_buffer(256)
    cus = ctypes.c_int(0)
    mem = ctypes.c_long(0)
    _lib.check_status(lib.thgpu_device_info(name, 256, ctypes.byref(cus), ctypes.byref(mem)))
    return {"name": name.value.decode(), "multiProcessorCount": cus.value, "totalGlobalMem": mem.value}


def gemm(transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc):
    """THGPUBlas_gemm on GPUTensor operands (column-major BLAS semantics)."""
    lib.THGPUBlas_gemm(transa.encode(), transb.encode(), m, n, k, alpha, lib.THGPUTensor_data(a._p), lda,
                       lib.THGPUTensor_data(b._p), ldb, beta, lib.THGPUTensor_data(c._p), ldc)
    _lib.check()


def gemv(trans, m, n, alpha, a, lda, x, incx, beta, y, incy):
    """THGPUBlas_gemv on GPUTensor operands (column-major, strided vectors)."""
    lib.THGPUBlas_gemv(trans.encode(), m, n, alpha, lib.THGPUTensor_data(a._p), lda, lib.THGPUTensor_data(x._p), incx,
                       beta, lib.THGPUTensor_data(y._p), incy)
    _lib.check()


def ger(m, n, alpha, x, incx, y, incy, a, lda):
    """THGPUBlas_ger: a += alpha * x y^T on a column-major m x n matrix."""
    lib.THGPUBlas_ger(m, n, alpha, lib.THGPUTensor_data(x._p), incx, lib.THGPUTensor_data(y._p), incy,
                      lib.THGPUTensor_data(a._p), lda)
    _lib.check()


def axpy(n, a, x, incx, y, incy):
    """THGPUBlas_axpy: y += a * x."""
    lib.THGPUBlas_axpy(n, a, lib.THGPUTensor_data(x._p), incx, lib.THGPUTensor_data(y._p), incy)
    _lib.check()


class Event(object):
    """HIP event on the library stream."""

    def __init__(self):
        self.h = lib.thgpu_event_create()
        if self.h < 0:
            _lib.check_status(1)

    def record(self):
        _lib.check_status(lib.thgpu_event_record(self.h))
        return self

    def elapsed_ms(self, stop):
        ms = ctypes.c_float(0)
        _lib.check_status(lib.thgpu_event_elapsed_ms(self.h, stop.h, ctypes.byref(ms)))
        return float(ms.value)


def prof_enable(on=True):
    lib.thgpu_prof_enable(1 if on else 0)


def prof_reset():
    lib.thgpu_prof_reset()


def prof_report():
    n = lib.thgpu_prof_report(None, 0)
    buf = ctypes.create_string_buffer(int(n) + 16)
    lib.thgpu_prof_report(buf, len(buf))
    return json.loads(buf.value.decode() or "{}")

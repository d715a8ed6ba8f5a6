"""ctypes binding of libthgpu.so (the C ABI declared in include/thgpu.h).

The library is the product; there is no fallback.  If it has not been built
the import fails with instructions instead of degrading to a CPU path.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libthgpu.so")

c_long, c_int, c_float, c_char = ctypes.c_long, ctypes.c_int, ctypes.c_float, ctypes.c_char
c_void_p, c_char_p = ctypes.c_void_p, ctypes.c_char_p
f32p = ctypes.POINTER(c_float)
longp = ctypes.POINTER(c_long)


def _storage_struct(name, ctype):
    return type(name, (ctypes.Structure,), {"_fields_": [
        ("data", ctypes.POINTER(ctype)), ("size", c_long), ("refcount", c_int), ("flag", c_char),
        ("allocator", c_void_p), ("allocatorContext", c_void_p)]})


def _tensor_struct(name, storage):
    return type(name, (ctypes.Structure,), {"_fields_": [
        ("size", longp), ("stride", longp), ("nDimension", c_int), ("storage", ctypes.POINTER(storage)),
        ("storageOffset", c_long), ("refcount", c_int), ("flag", c_char)]})


# Layouts of gputorch/FFI.lua:5-29 and TH/generic/THStorage.h:23-31.
THGPUStorage = _storage_struct("THGPUStorage", c_float)
THGPUTensor = _tensor_struct("THGPUTensor", THGPUStorage)
HOST_TYPES = {
    "Byte": ctypes.c_ubyte, "Char": ctypes.c_byte, "Short": ctypes.c_short, "Int": ctypes.c_int,
    "Long": ctypes.c_long, "Float": ctypes.c_float, "Double": ctypes.c_double,
}
HostStorage = {k: _storage_struct("TH%sStorage" % k, v) for k, v in HOST_TYPES.items()}
HostTensor = {k: _tensor_struct("TH%sTensor" % k, HostStorage[k]) for k in HOST_TYPES}
THLongStorage = HostStorage["Long"]

StorageP = ctypes.POINTER(THGPUStorage)
TensorP = ctypes.POINTER(THGPUTensor)
ERROR_HANDLER = ctypes.CFUNCTYPE(None, c_char_p, c_void_p)


class THGPUError(RuntimeError):
    """Raised where the reference would raise a Lua error (luaL_argcheck / THError)."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libthgpu.so is not built (%s). Build it with `python mcw_cppamp_torch_amd/build.py` "
            "(hipcc, gfx950). There is no CPU fallback." % LIB_PATH)
    return ctypes.CDLL(LIB_PATH)


lib = _load()

_SIGNATURES = {
    # runtime
    "THGPUSetErrorHandler": (None, [ERROR_HANDLER, c_void_p]),
    "thgpu_last_error": (c_char_p, []),
    "thgpu_init": (c_int, []),
    "thgpu_synchronize": (c_int, []),
    "thgpu_empty_cache": (c_int, []),
    "thgpu_cached_bytes": (c_long, []),
    "thgpu_device_alloc_calls": (c_long, []),
    "thgpu_debug_set": (c_int, [c_char_p, c_char_p]),
    "thgpu_conv_set_mode": (c_int, [c_int]),
    "thgpu_conv_get_mode": (c_int, []),
    "thgpu_conv_set_finput_reuse": (c_int, [c_int]),
    "thgpu_conv_get_finput_reuse": (c_int, []),
    "thgpu_device_info": (c_int, [c_char_p, c_long, ctypes.POINTER(c_int), longp]),
    "thgpu_event_create": (c_int, []),
    "thgpu_event_record": (c_int, [c_int]),
    "thgpu_event_elapsed_ms": (c_int, [c_int, c_int, f32p]),
    "thgpu_prof_enable": (c_int, [c_int]),
    "thgpu_prof_reset": (c_int, []),
    "thgpu_prof_report": (c_long, [c_char_p, c_long]),
    "thgpu_selftest_index_math": (c_long, []),
    "thgpu_selftest_launch_plans": (c_long, []),
    # storage
    "THGPUStorage_data": (f32p, [StorageP]),
    "THGPUStorage_size": (c_long, [StorageP]),
    "THGPUStorage_set": (None, [StorageP, c_long, c_float]),
    "THGPUStorage_get": (c_float, [StorageP, c_long]),
    "THGPUStorage_new": (StorageP, []),
    "THGPUStorage_newWithSize": (StorageP, [c_long]),
    "THGPUStorage_newWithSize1": (StorageP, [c_float]),
    "THGPUStorage_newWithSize2": (StorageP, [c_float] * 2),
    "THGPUStorage_newWithSize3": (StorageP, [c_float] * 3),
    "THGPUStorage_newWithSize4": (StorageP, [c_float] * 4),
    "THGPUStorage_newWithMapping": (StorageP, [c_char_p, c_long, c_int]),
    "THGPUStorage_newWithData": (StorageP, [f32p, c_long]),
    "THGPUStorage_setFlag": (None, [StorageP, c_char]),
    "THGPUStorage_clearFlag": (None, [StorageP, c_char]),
    "THGPUStorage_retain": (None, [StorageP]),
    "THGPUStorage_free": (None, [StorageP]),
    "THGPUStorage_resize": (None, [StorageP, c_long]),
    "THGPUStorage_fill": (None, [StorageP, c_float]),
    "THGPUStorage_rawCopy": (None, [StorageP, f32p]),
    "THGPUStorage_copy": (None, [StorageP, StorageP]),
    "THGPUStorage_copyGPU": (None, [StorageP, StorageP]),
    # tensor
    "THGPUTensor_storage": (StorageP, [TensorP]),
    "THGPUTensor_storageOffset": (c_long, [TensorP]),
    "THGPUTensor_nDimension": (c_int, [TensorP]),
    "THGPUTensor_size": (c_long, [TensorP, c_int]),
    "THGPUTensor_stride": (c_long, [TensorP, c_int]),
    "THGPUTensor_newSizeOf": (ctypes.POINTER(THLongStorage), [TensorP]),
    "THGPUTensor_newStrideOf": (ctypes.POINTER(THLongStorage), [TensorP]),
    "THGPUTensor_data": (f32p, [TensorP]),
    "THGPUTensor_setFlag": (None, [TensorP, c_char]),
    "THGPUTensor_clearFlag": (None, [TensorP, c_char]),
    "THGPUTensor_new": (TensorP, []),
    "THGPUTensor_newWithTensor": (TensorP, [TensorP]),
    "THGPUTensor_newWithStorage": (TensorP, [StorageP, c_long, ctypes.POINTER(THLongStorage),
                                             ctypes.POINTER(THLongStorage)]),
    "THGPUTensor_newWithStorage1d": (TensorP, [StorageP, c_long] + [c_long] * 2),
    "THGPUTensor_newWithStorage2d": (TensorP, [StorageP, c_long] + [c_long] * 4),
    "THGPUTensor_newWithStorage3d": (TensorP, [StorageP, c_long] + [c_long] * 6),
    "THGPUTensor_newWithStorage4d": (TensorP, [StorageP, c_long] + [c_long] * 8),
    "THGPUTensor_newWithSize": (TensorP, [ctypes.POINTER(THLongStorage), ctypes.POINTER(THLongStorage)]),
    "THGPUTensor_newWithSize1d": (TensorP, [c_long]),
    "THGPUTensor_newWithSize2d": (TensorP, [c_long] * 2),
    "THGPUTensor_newWithSize3d": (TensorP, [c_long] * 3),
    "THGPUTensor_newWithSize4d": (TensorP, [c_long] * 4),
    "THGPUTensor_newClone": (TensorP, [TensorP]),
    "THGPUTensor_newContiguous": (TensorP, [TensorP]),
    "THGPUTensor_newSelect": (TensorP, [TensorP, c_int, c_long]),
    "THGPUTensor_newNarrow": (TensorP, [TensorP, c_int, c_long, c_long]),
    "THGPUTensor_newTranspose": (TensorP, [TensorP, c_int, c_int]),
    "THGPUTensor_newUnfold": (TensorP, [TensorP, c_int, c_long, c_long]),
    "THGPUTensor_resize": (None, [TensorP, ctypes.POINTER(THLongStorage), ctypes.POINTER(THLongStorage)]),
    "THGPUTensor_resizeAs": (None, [TensorP, TensorP]),
    "THGPUTensor_resize1d": (None, [TensorP] + [c_long]),
    "THGPUTensor_resize2d": (None, [TensorP] + [c_long] * 2),
    "THGPUTensor_resize3d": (None, [TensorP] + [c_long] * 3),
    "THGPUTensor_resize4d": (None, [TensorP] + [c_long] * 4),
    "THGPUTensor_resize5d": (None, [TensorP] + [c_long] * 5),
    "THGPUTensor_set": (None, [TensorP, TensorP]),
    "THGPUTensor_setStorage": (None, [TensorP, StorageP, c_long, ctypes.POINTER(THLongStorage),
                                      ctypes.POINTER(THLongStorage)]),
    "THGPUTensor_narrow": (None, [TensorP, TensorP, c_int, c_long, c_long]),
    "THGPUTensor_select": (None, [TensorP, TensorP, c_int, c_long]),
    "THGPUTensor_transpose": (None, [TensorP, TensorP, c_int, c_int]),
    "THGPUTensor_unfold": (None, [TensorP, TensorP, c_int, c_long, c_long]),
    "THGPUTensor_squeeze": (None, [TensorP, TensorP]),
    "THGPUTensor_squeeze1d": (None, [TensorP, TensorP, c_int]),
    "THGPUTensor_setStorage1d": (None, [TensorP, StorageP, c_long] + [c_long] * 2),
    "THGPUTensor_setStorage2d": (None, [TensorP, StorageP, c_long] + [c_long] * 4),
    "THGPUTensor_setStorage3d": (None, [TensorP, StorageP, c_long] + [c_long] * 6),
    "THGPUTensor_setStorage4d": (None, [TensorP, StorageP, c_long] + [c_long] * 8),
    "THGPUTensor_isContiguous": (c_int, [TensorP]),
    "THGPUTensor_isSameSizeAs": (c_int, [TensorP, TensorP]),
    "THGPUTensor_nElement": (c_long, [TensorP]),
    "THGPUTensor_retain": (None, [TensorP]),
    "THGPUTensor_free": (None, [TensorP]),
    "THGPUTensor_freeCopyTo": (None, [TensorP, TensorP]),
    "THGPUTensor_set1d": (None, [TensorP] + [c_long] * 1 + [c_float]),
    "THGPUTensor_set2d": (None, [TensorP] + [c_long] * 2 + [c_float]),
    "THGPUTensor_set3d": (None, [TensorP] + [c_long] * 3 + [c_float]),
    "THGPUTensor_set4d": (None, [TensorP] + [c_long] * 4 + [c_float]),
    "THGPUTensor_get1d": (c_float, [TensorP] + [c_long] * 1),
    "THGPUTensor_get2d": (c_float, [TensorP] + [c_long] * 2),
    "THGPUTensor_get3d": (c_float, [TensorP] + [c_long] * 3),
    "THGPUTensor_get4d": (c_float, [TensorP] + [c_long] * 4),
    "THGPUTensor_fill": (None, [TensorP, c_float]),
    "thgpu_fill_many": (c_int, [ctypes.POINTER(TensorP), c_int, c_float]),
    "THGPUTensor_zero": (None, [TensorP]),
    "THGPUTensor_copy": (None, [TensorP, TensorP]),
    "THGPUTensor_copyGPU": (None, [TensorP, TensorP]),
    # blas
    "THGPUTensor_add": (None, [TensorP, TensorP, c_float]),
    "THGPUTensor_mul": (None, [TensorP, TensorP, c_float]),
    "THGPUTensor_div": (None, [TensorP, TensorP, c_float]),
    "THGPUTensor_cadd": (None, [TensorP, TensorP, c_float, TensorP]),
    "THGPUTensor_addmv": (None, [TensorP, c_float, TensorP, c_float, TensorP, TensorP]),
    "THGPUTensor_addmm": (None, [TensorP, c_float, TensorP, c_float, TensorP, TensorP]),
    "THGPUTensor_addr": (None, [TensorP, c_float, TensorP, c_float, TensorP, TensorP]),
    "THGPUTensor_dot": (c_float, [TensorP, TensorP]),
    "THGPUTensor_indexSelect": (None, [TensorP, TensorP, c_int, ctypes.POINTER(HostTensor["Long"])]),
    "THGPUTensor_indexCopy": (None, [TensorP, c_int, ctypes.POINTER(HostTensor["Long"]), TensorP]),
    "THGPUTensor_indexFill": (None, [TensorP, c_int, ctypes.POINTER(HostTensor["Long"]), c_float]),
    "thgpu_memcpy_h2d": (c_int, [f32p, f32p, c_long]),
    "thgpu_memcpy_d2h": (c_int, [f32p, f32p, c_long]),
    "THGPUBlas_gemm": (None, [c_char, c_char, c_long, c_long, c_long, c_float, f32p, c_long, f32p, c_long,
                              c_float, f32p, c_long]),
    "THGPUBlas_axpy": (None, [c_long, c_float, f32p, c_long, f32p, c_long]),
    "THGPUBlas_ger": (None, [c_long, c_long, c_float, f32p, c_long, f32p, c_long, f32p, c_long]),
    "THGPUBlas_gemv": (None, [c_char, c_long, c_long, c_float, f32p, c_long, f32p, c_long, c_float, f32p, c_long]),
    "thgpu_gemm_noalloc": (c_int, [c_char, c_char, c_long, c_long, c_long, c_float, f32p, c_long, f32p, c_long,
                                   c_float, f32p, c_long]),
    "thgpu_gemm_strided_batched": (c_int, [c_char, c_char, c_long, c_long, c_long, c_float, f32p, c_long, c_long, f32p,
                                            c_long, c_long, c_float, f32p, c_long, c_long, c_long]),
    # flat operators
    "thgpu_im2col": (c_int, [f32p, c_long] + [c_int] * 9 + [f32p]),
    "thgpu_col2im": (c_int, [f32p, c_long] + [c_int] * 9 + [f32p]),
    "thgpu_SpatialConvolutionMM_updateOutput": (c_int, [TensorP] * 6 + [c_int] * 6),
    "thgpu_SpatialConvolutionMM_updateGradInput": (c_int, [TensorP] * 6 + [c_int] * 6),
    "thgpu_SpatialConvolutionMM_accGradParameters": (c_int, [TensorP] * 6 + [c_int] * 6 + [c_float]),
    "thgpu_SpatialConvolutionMM_updateOutputFused": (c_int, [TensorP] * 6 + [c_int] * 7 + [c_float] * 2),
    "thgpu_SpatialConvolutionMM_updateGradInputFused": (c_int, [TensorP] * 6 + [c_int] * 7 + [c_float]),
    "thgpu_SpatialConvolutionMM_accGradParametersFused": (c_int, [TensorP] * 6 + [c_int] * 6 + [c_float, c_int]),
    "thgpu_conv_gathers": (c_int, [c_long] + [c_int] * 10),
    "thgpu_SpatialConvolutionMM_gradOutputTwin": (c_int, [TensorP] * 4 + [c_int] * 6 + [ctypes.POINTER(c_int)]),
    "thgpu_SpatialConvolutionMM_updateGradInputTwin": (c_int, [TensorP] * 6 + [c_int] * 7 + [c_float, TensorP,
                                                               ctypes.POINTER(c_int)]),
    "thgpu_SpatialMaxPooling_updateGradInputTwin": (c_int, [TensorP] * 4 + [c_int] * 5 + [c_float, TensorP,
                                                            ctypes.POINTER(c_int)]),
    "thgpu_SpatialMaxPooling_updateGradInputMasked": (c_int, [TensorP] * 4 + [c_int] * 4 + [c_float]),
    "thgpu_SpatialMaxPooling_updateOutput": (c_int, [TensorP] * 3 + [c_int] * 4),
    "thgpu_SpatialMaxPooling_updateGradInput": (c_int, [TensorP] * 4 + [c_int] * 4),
    "thgpu_Threshold_updateOutput": (c_int, [TensorP] * 2 + [c_float] * 2),
    "thgpu_Threshold_updateGradInput": (c_int, [TensorP] * 3 + [c_float]),
    "thgpu_SpatialAveragePooling_updateOutput": (c_int, [TensorP] * 2 + [c_int] * 4),
    "thgpu_SpatialAveragePooling_updateGradInput": (c_int, [TensorP] * 3 + [c_int] * 4),
    "thgpu_SpatialSubSampling_updateOutput": (c_int, [TensorP] * 4 + [c_int] * 4),
    "thgpu_SpatialSubSampling_updateGradInput": (c_int, [TensorP] * 4 + [c_int] * 4),
    "thgpu_SpatialSubSampling_accGradParameters": (c_int, [TensorP] * 4 + [c_int] * 4 + [c_float]),
    "thgpu_LogSoftMax_updateOutput": (c_int, [TensorP] * 2),
    "thgpu_LogSoftMax_updateGradInput": (c_int, [TensorP] * 3),
    "thgpu_ClassNLLCriterion_updateOutput": (c_int, [TensorP] * 3 + [c_int]),
    "thgpu_ClassNLLCriterion_updateGradInput": (c_int, [TensorP] * 3 + [c_int]),
}
for _k in HOST_TYPES:
    _SIGNATURES["THGPUStorage_copy%s" % _k] = (None, [StorageP, ctypes.POINTER(HostStorage[_k])])
    _SIGNATURES["TH%sStorage_copyGPU" % _k] = (None, [ctypes.POINTER(HostStorage[_k]), StorageP])
    _SIGNATURES["THGPUTensor_copy%s" % _k] = (None, [TensorP, ctypes.POINTER(HostTensor[_k])])
    _SIGNATURES["TH%sTensor_copyGPU" % _k] = (None, [ctypes.POINTER(HostTensor[_k]), TensorP])

EXPORTED_SYMBOLS = sorted(_SIGNATURES)

for _name, (_res, _args) in _SIGNATURES.items():
    _fn = getattr(lib, _name)  # AttributeError here means the library lacks a declared symbol
    _fn.restype = _res
    _fn.argtypes = _args

# TH-named functions report errors through a handler; the reference's handler
# raises a Lua error (mcw_torch7_core/init.c:38-55).  Here the handler stores
# the message and the Python wrappers raise THGPUError right after the call.
_pending = []


@ERROR_HANDLER
def _handler(msg, _data):
    _pending.append(msg.decode(errors="replace") if msg else "unknown error")


lib.THGPUSetErrorHandler(_handler, None)


def check():
    """Raise if the last TH-named call reported an error."""
    if _pending:
        msg = _pending[0]
        del _pending[:]
        raise THGPUError(msg)


def check_status(rc):
    """Raise if a thgpu_* call returned a non-zero status."""
    if _pending or rc != 0:
        msg = _pending[0] if _pending else lib.thgpu_last_error().decode(errors="replace")
        del _pending[:]
        raise THGPUError(msg)

"""CPU-only checks of the product's host side: the C-ABI library loads and
exports every symbol that include/thgpu.h declares, the ctypes binding covers
them, the index arithmetic self-test passes, error paths that need no device
work report through the handler, and the stack bookkeeping reproduces the
algorithmic work of the benchmark configurations."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "thgpu.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    text = re.sub(r"#define THGPU_DECLARE_HOST_TYPES.*?TH##Name##Tensor;", "", text, flags=re.S)
    names = set(re.findall(r"\b((?:TH[A-Za-z]*|thgpu)_[A-Za-z0-9_]+)\s*\(", text))
    names |= {"THGPUSetErrorHandler"}
    return sorted(n for n in names if not n.startswith("THGPU_"))


@pytest.fixture(scope="module")
def pkg():
    import mcw_cppamp_torch_amd as p
    return p


def test_library_exports_every_declared_symbol(pkg):
    names = declared_functions()
    assert len(names) > 120
    raw = ctypes.CDLL(pkg._lib.LIB_PATH)
    missing = [n for n in names if not hasattr(raw, n)]
    assert not missing, missing


def test_ctypes_binding_covers_the_header(pkg):
    assert set(declared_functions()) == set(pkg._lib.EXPORTED_SYMBOLS)


def test_struct_layouts_match_the_header_as_a_c_compiler_sees_it(pkg, tmp_path):
    # The two structs are ABI (LuaJIT FFI reads them, gputorch/FFI.lua:5-29): compile the
    # header with gcc as plain C and compare sizes/offsets with the ctypes mirror.
    import subprocess
    src = tmp_path / "layout.c"
    src.write_text(
        '#include <stdio.h>\n#include <stddef.h>\n#include "thgpu.h"\n'
        'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n",'
        'sizeof(THGPUStorage),offsetof(THGPUStorage,size),offsetof(THGPUStorage,refcount),'
        'offsetof(THGPUStorage,flag),offsetof(THGPUStorage,allocator),offsetof(THGPUStorage,allocatorContext),'
        'sizeof(THGPUTensor),offsetof(THGPUTensor,nDimension),offsetof(THGPUTensor,storage),'
        'offsetof(THGPUTensor,storageOffset),offsetof(THGPUTensor,refcount),offsetof(THGPUTensor,flag));return 0;}\n')
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"), str(src),
                           "-o", str(exe)])
    c_view = [int(v) for v in subprocess.check_output([str(exe)]).split()]
    L = pkg._lib
    S, T = L.THGPUStorage, L.THGPUTensor
    py_view = [ctypes.sizeof(S), S.size.offset, S.refcount.offset, S.flag.offset, S.allocator.offset,
               S.allocatorContext.offset, ctypes.sizeof(T), T.nDimension.offset, T.storage.offset,
               T.storageOffset.offset, T.refcount.offset, T.flag.offset]
    assert c_view == py_view == [40, 8, 16, 20, 24, 32, 48, 16, 24, 32, 40, 44]


def test_index_math_selftest(pkg):
    assert pkg._lib.lib.thgpu_selftest_index_math() == 0


def test_launch_plan_selftest(pkg):
    # im2col strip shapes and max-pool backward tiles over a grid of geometries, checked on the host
    assert pkg._lib.lib.thgpu_selftest_launch_plans() == 0


def test_metadata_only_tensor_ops_and_error_handler(pkg):
    # Views and argument errors need no device memory.
    t = pkg.GPUTensor()
    assert t.dim() == 0 and t.nElement() == 0 and t.isContiguous()
    s = pkg.GPUStorage()
    assert s.size() == 0
    with pytest.raises(pkg.THGPUError, match="index out of bounds"):
        s[0]
    with pytest.raises(pkg.THGPUError, match="not available yet"):
        pkg._lib.lib.THGPUStorage_newWithMapping(b"x", 1, 0)
        pkg._lib.check()
    with pytest.raises(pkg.THGPUError, match="out of range"):
        t.size(0)


def test_ops_reject_bad_arguments_without_a_device(pkg):
    nn = pkg.nn
    conv = nn.SpatialConvolutionMM(3, 4, 3, 3)
    with pytest.raises(pkg.THGPUError, match="GPUTensor expected"):
        conv.forward(np.zeros((1, 3, 8, 8), np.float32))
    L = pkg._lib
    empty = [pkg.GPUTensor() for _ in range(6)]
    rc = L.lib.thgpu_SpatialConvolutionMM_updateOutput(*([e._p for e in empty] + [3, 3, 1, 1, 0, 0]))
    assert rc != 0 and b"3D or 4D" in L.lib.thgpu_last_error()
    rc = L.lib.thgpu_SpatialMaxPooling_updateOutput(empty[0]._p, empty[1]._p, empty[2]._p, 2, 2, 2, 2)
    assert rc != 0 and b"3D or 4D" in L.lib.thgpu_last_error()
    with pytest.raises(pkg.THGPUError, match="nn.Threshold"):
        nn.Threshold("a", 1)


def test_switches_are_set_by_name(pkg):
    L = pkg._lib
    assert L.lib.thgpu_debug_set(b"no_such_switch", b"1") != 0
    assert L.lib.thgpu_debug_set(b"gemm_tile", b"128x128") == 0 and L.lib.thgpu_debug_set(b"gemm_tile", None) == 0


def test_failed_resize_leaves_the_tensor_unchanged_and_operators_refuse_it(pkg):
    """A resize whose allocation fails (here: 2^46 floats, or no device at all) must not leave the tensor claiming
    the new shape over the old buffer; an operator handed such tensors returns an error before any launch."""
    L = pkg._lib
    t = pkg.GPUTensor()
    before = (t.dim(), t.nElement())
    with pytest.raises(pkg.THGPUError):
        L.lib.THGPUTensor_resize2d(t._p, 1 << 23, 1 << 23)
        L.check()
    assert (t.dim(), t.nElement()) == before
    assert t._p.contents.nDimension == 0
    st = t._p.contents.storage
    assert not st or st.contents.size == 0
    # the operator sees the old (empty) shape, not a 2^46-element claim over no memory, and refuses it
    out, ind = pkg.GPUTensor(), pkg.GPUTensor()
    assert L.lib.thgpu_SpatialMaxPooling_updateOutput(t._p, out._p, ind._p, 2, 2, 2, 2) != 0


def test_noalloc_gemm_refuses_to_run_before_init_or_beyond_its_limit(pkg):
    L = pkg._lib
    null = ctypes.POINTER(ctypes.c_float)()
    rc = L.lib.thgpu_gemm_noalloc(b"n", b"n", 4, 4, 4, 1.0, null, 4, null, 4, 0.0, null, 4)
    # nothing in this CPU-side module initialises the library; in a process that did, the null operands are what
    # is refused: either way nothing is launched
    assert rc != 0 and (b"thgpu_init" in L.lib.thgpu_last_error() or b"null operand" in L.lib.thgpu_last_error())


def test_flat_entry_points_refuse_null_operands_before_any_launch(pkg):
    """Every flat entry point that takes raw device pointers or tensor handles returns an error for a null one while
    its other arguments are valid: the refusal comes before the library is initialised or anything is enqueued (a null
    pointer that reached a kernel would fault on the GPU)."""
    L = pkg._lib
    lib = L.lib
    null = ctypes.POINTER(ctypes.c_float)()
    buf = (ctypes.c_float * 16)()          # a host buffer standing in for "some non-null pointer": never dereferenced
    ptr = ctypes.cast(buf, ctypes.POINTER(ctypes.c_float))
    geom = [1, 1, 4, 4, 3, 3, 1, 1, 1, 1]  # B, C, H, W, kH, kW, padH, padW, sH, sW
    for fn in (lib.thgpu_im2col, lib.thgpu_col2im):
        for a, b in ((null, ptr), (ptr, null), (null, null)):
            assert fn(a, *(geom + [b])) != 0 and b"null operand" in lib.thgpu_last_error()
    rc = lib.thgpu_gemm_strided_batched(b"n", b"n", 4, 4, 4, 1.0, null, 4, 16, ptr, 4, 0, 0.0, ptr, 4, 16, 2)
    assert rc != 0 and b"null operand" in lib.thgpu_last_error()
    rc = lib.thgpu_gemm_strided_batched(b"n", b"n", 4, 4, 4, 1.0, ptr, 4, 16, ptr, 4, 0, 0.0, null, 4, 16, 2)
    assert rc != 0 and b"null operand" in lib.thgpu_last_error()
    # an overflowing m * n is caught by the range check, not by the product
    rc = lib.thgpu_gemm_noalloc(b"n", b"n", 1 << 40, 1 << 40, 4, 1.0, ptr, 4, ptr, 4, 0.0, ptr, 4)
    assert rc != 0
    # operators on tensor handles: a null handle in any position
    nullt = L.TensorP()
    t = [pkg.GPUTensor() for _ in range(7)]
    P = [x._p for x in t]
    conv_geom = [3, 3, 1, 1, 0, 0]
    cases = [
        (lib.thgpu_SpatialConvolutionMM_updateOutput, 6, conv_geom),
        (lib.thgpu_SpatialConvolutionMM_updateOutputFused, 6, conv_geom + [0, 0.0, 0.0]),
        (lib.thgpu_SpatialConvolutionMM_updateGradInput, 6, conv_geom),
        (lib.thgpu_SpatialConvolutionMM_updateGradInputFused, 6, conv_geom + [0, 0.0]),
        (lib.thgpu_SpatialConvolutionMM_accGradParameters, 6, conv_geom + [1.0]),
        (lib.thgpu_SpatialConvolutionMM_accGradParametersFused, 6, conv_geom + [1.0, 0]),
        (lib.thgpu_SpatialMaxPooling_updateOutput, 3, [2, 2, 2, 2]),
        (lib.thgpu_SpatialMaxPooling_updateGradInput, 4, [2, 2, 2, 2]),
        (lib.thgpu_SpatialMaxPooling_updateGradInputMasked, 4, [2, 2, 2, 2, 0.0]),
        (lib.thgpu_Threshold_updateOutput, 2, [0.0, 0.0]),
        (lib.thgpu_Threshold_updateGradInput, 3, [0.0]),
    ]
    for fn, ntens, rest in cases:
        for hole in range(ntens):
            args = [nullt if i == hole else P[i] for i in range(ntens)]
            assert fn(*(args + rest)) != 0, (fn.__name__, hole)


def test_module_defaults_follow_the_lua_constructors(pkg):
    nn = pkg.nn
    c = nn.SpatialConvolutionMM(3, 8, 5, 7)
    assert (c.dW, c.dH, c.padding) == (1, 1, 0) and c.weight.shape == (8, 3 * 7 * 5)
    stdv = 1 / np.sqrt(5 * 7 * 3)
    assert np.abs(c.weight).max() <= stdv and np.abs(c.bias).max() <= stdv
    p = nn.SpatialMaxPooling(3, 2)
    assert (p.dW, p.dH) == (3, 2)
    t = nn.Threshold()
    assert t.threshold == 1e-6 and t.val == 0
    r = nn.ReLU()
    assert r.threshold == 0 and r.val == 0
    seq = nn.Sequential().add(c).add(r).add(p)
    assert seq.size() == 3 and seq.get(0) is c


def test_stack_bookkeeping_reproduces_the_benchmark_work(pkg):
    st = pkg.stacks
    assert abs(st.work("alexnet")["gemm_flops"] / 1e9 - 503.5) < 0.05
    assert abs(st.work("overfeat")["gemm_flops"] / 1e9 - 2051.7) < 0.05
    assert abs(st.work("vgg_a")["gemm_flops"] / 1e9 - 2874.4) < 0.05
    assert abs(st.work("conv1_b16")["gemm_flops"] / 1e9 - 6.75) < 0.01
    assert st.output_shape("alexnet") == (128, 256, 6, 6)
    assert st.output_shape("overfeat") == (128, 1024, 6, 6)
    assert st.output_shape("vgg_a") == (64, 512, 7, 7)


def test_more_module_defaults_follow_the_lua_constructors(pkg):
    nn = pkg.nn
    a = nn.SpatialAveragePooling(3, 2)
    assert (a.kW, a.kH, a.dW, a.dH) == (3, 2, 1, 1)                      # mcw_nn/SpatialAveragePooling.lua:8-9
    s = nn.SpatialSubSampling(6, 2, 3)
    assert (s.dW, s.dH) == (1, 1) and s.weight.shape == (6,) and s.gradBias.shape == (6,)
    bound = 1 / np.sqrt(2 * 3)                                           # mcw_nn/SpatialSubSampling.lua:28
    assert np.abs(s.weight).max() <= bound and np.abs(s.bias).max() <= bound
    c = nn.ClassNLLCriterion()
    assert c.sizeAverage is True and c.output == 0 and c.outputTensor.shape == (1,)
    v = nn.View(4, 5)
    assert v.size == (4, 5) and v.numElements == 20 and v.output is None and v.numInputDims is None
    r = nn.Reshape(2, 3, True)
    assert r.size == (2, 3) and r.nelement == 6 and r.batchMode is True
    seq = nn.Sequential().add(nn.Linear(3, 2)).add(nn.ReLU()).add(nn.Linear(2, 2))
    w, gw = seq.parameters()
    assert len(w) == 4 and len(gw) == 4                                  # weight, bias of both Linear modules
    seq.insert(nn.ReLU(), 0)
    assert seq.size() == 4 and isinstance(seq.get(0), nn.ReLU)
    with pytest.raises(pkg.THGPUError):
        seq.insert(nn.ReLU(), 9)


def test_product_never_imports_the_oracle_and_bench_refuses_more_than_one_gpu():
    import glob
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for path in glob.glob(os.path.join(root, "mcw_cppamp_torch_amd", "**", "*.py"), recursive=True):
        text = open(path).read()
        assert "import oracle" not in text and "from oracle" not in text, path
    for path in glob.glob(os.path.join(root, "mcw_cppamp_torch_amd", "csrc", "*")):
        assert "oracle" not in open(path, errors="ignore").read(), path
    proc = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, text=True, timeout=120)
    assert proc.returncode != 0 and "one GPU" in (proc.stdout + proc.stderr)

"""Builds libthgpu.so (the HIP library) in-tree with hipcc for gfx950.

    python mcw_cppamp_torch_amd/build.py

Each .hip source is compiled to an object file (in parallel) and linked into
mcw_cppamp_torch_amd/libthgpu.so.  hipcc cross-compiles without a GPU.
"""
import concurrent.futures
import glob
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(HERE, "libthgpu.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
    # Keep the compiler from forming packed-FP32 instructions.
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # a*b + c stays two roundings, as in the CPU modules the results are compared with bit for bit (hipcc's
    # default contracts them into fused multiply-adds, and its __fmul_rn / __fadd_rn are plain operators).
    "-ffp-contract=off",
]


def _compile(src):
    obj = os.path.join(OBJ_DIR, os.path.basename(src).replace(".hip", ".o"))
    cmd = [HIPCC] + FLAGS + ["-c", src, "-o", obj]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    # The host pass does not know the packed-fp32 feature and says so; drop that line.
    out = "\n".join(l for l in proc.stdout.splitlines() if "packed-fp32-ops" not in l)
    if proc.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    sources = sorted(glob.glob(os.path.join(CSRC, "*.hip")))
    if not sources:
        raise RuntimeError("no .hip sources under %s" % CSRC)
    jobs = jobs or min(len(sources), os.cpu_count() or 4, 8)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for obj, out in pool.map(_compile, sources):
            objs.append(obj)
            if verbose and out.strip():
                print(out)
    tmp = LIB_PATH + ".tmp"
    subprocess.check_call([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp] + objs)
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


def _first_dir_with(names, roots):
    """The first of `roots` that holds every file of `names`, or None."""
    for r in roots:
        if r and os.path.isdir(r) and all(os.path.exists(os.path.join(r, n)) for n in names):
            return r
    return None


def _lua_include_dirs():
    """Where the luaT glue finds its headers, or None when Lua or luaT is missing: LUA_INCDIR / TORCH_INSTALL first,
    then the usual prefixes.  Keys: lua (lua.h, lauxlib.h), luaT (luaT.h), and -- for the tensor half only -- TH (TH.h
    with its configured THGeneral.h) and templates (the directory that holds Torch's generic/Tensor.c and
    generic/Storage.c: gputorch/torch of a Torch7 source tree, TORCH7_SRC)."""
    install = os.environ.get("TORCH_INSTALL", "")
    src = os.environ.get("TORCH7_SRC", "")
    roots = [os.environ.get("LUA_INCDIR"), os.path.join(install, "include") if install else None,
             "/usr/include/luajit-2.1", "/usr/include/luajit-2.0", "/usr/include/lua5.1", "/usr/local/include",
             "/usr/include", os.path.expanduser("~/torch/install/include")]
    found = {"lua": _first_dir_with(["lua.h", "lauxlib.h"], roots), "luaT": _first_dir_with(["luaT.h"], roots)}
    if not found["lua"] or not found["luaT"]:
        return None
    found["TH"] = _first_dir_with(["TH.h", "THGeneral.h"], [os.path.join(r, "TH") for r in roots if r] + roots)
    found["templates"] = _first_dir_with([os.path.join("generic", "Tensor.c"), os.path.join("generic", "Storage.c")],
                                         [os.environ.get("GPUTORCH_TEMPLATES"),
                                          os.path.join(src, "gputorch", "torch") if src else None,
                                          os.path.join(src, "torch") if src else None])
    return found


def build_lua_glue(verbose=False):
    """Compiles the luaT glue where the Lua and luaT headers exist: lua/gpunn_glue.cpp into libgpunn.so
    (luaopen_libgpunn) and, where the TH headers and Torch's binding templates are found as well,
    lua/gputorch_glue.cpp into libgputorch.so (luaopen_libgputorch).  Returns the list of libraries built (empty
    without a Lua toolchain: the glue is then source only, syntax-checked by tests/test_lua_glue_syntax.py, and the
    Python mirror in nn.py / gputorch.py is the host side)."""
    inc = _lua_include_dirs()
    if inc is None:
        if verbose:
            print("lua.h / luaT.h not found: lua/gpunn_glue.cpp and lua/gputorch_glue.cpp not built")
        return []
    common = ["g++", "-O2", "-fPIC", "-shared", "-std=c++11"]
    link = ["-L" + HERE, "-lthgpu", "-lluaT", "-Wl,-rpath," + HERE]
    built = []
    out = os.path.join(HERE, "libgpunn.so")
    dirs = list(dict.fromkeys([inc["lua"], inc["luaT"]]))
    subprocess.check_call(common + [os.path.join(HERE, "lua", "gpunn_glue.cpp"), "-o", out] + link +
                          ["-I" + d for d in dirs])
    built.append(out)
    if inc["TH"] and inc["templates"]:
        out = os.path.join(HERE, "libgputorch.so")
        dirs = list(dict.fromkeys([inc["lua"], inc["luaT"], inc["TH"], inc["templates"]]))
        subprocess.check_call(common + [os.path.join(HERE, "lua", "gputorch_glue.cpp"), "-o", out] + link + ["-lTH"] +
                              ["-I" + d for d in dirs])
        built.append(out)
    elif verbose:
        print("TH.h or Torch's generic/Tensor.c not found (TORCH_INSTALL, TORCH7_SRC): lua/gputorch_glue.cpp not built")
    return built


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    build_lua_glue(verbose=True)

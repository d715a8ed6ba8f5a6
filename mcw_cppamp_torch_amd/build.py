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


def _lua_include_dirs():
    """Directories holding lua.h and luaT.h, or None: LUA_INCDIR / TORCH_INSTALL first, then the usual prefixes."""
    roots = [os.environ.get("LUA_INCDIR"), os.path.join(os.environ.get("TORCH_INSTALL", ""), "include"),
             "/usr/include/luajit-2.1", "/usr/include/luajit-2.0", "/usr/include/lua5.1", "/usr/local/include",
             "/usr/include", os.path.expanduser("~/torch/install/include")]
    roots = [r for r in roots if r and os.path.isdir(r)]
    lua = next((r for r in roots if os.path.exists(os.path.join(r, "lua.h"))), None)
    luat = next((r for r in roots if os.path.exists(os.path.join(r, "luaT.h"))), None)
    return [lua, luat] if lua and luat else None


def build_lua_glue(verbose=False):
    """Compiles lua/gpunn_glue.cpp into libgpunn.so where the Lua and luaT headers exist; returns its path or None
    (no Lua toolchain: the glue is source only, the Python mirror in nn.py / gputorch.py is the host side)."""
    inc = _lua_include_dirs()
    if inc is None:
        if verbose:
            print("lua.h / luaT.h not found: lua/gpunn_glue.cpp not built")
        return None
    out = os.path.join(HERE, "libgpunn.so")
    cmd = ["g++", "-O2", "-fPIC", "-shared", "-std=c++11", os.path.join(HERE, "lua", "gpunn_glue.cpp"), "-o", out,
           "-L" + HERE, "-lthgpu", "-lluaT", "-Wl,-rpath," + HERE] + ["-I" + d for d in dict.fromkeys(inc)]
    subprocess.check_call(cmd)
    return out


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))
    build_lua_glue(verbose=True)

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


if __name__ == "__main__":
    print(build(verbose="-v" in sys.argv))

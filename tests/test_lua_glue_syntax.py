"""CPU-only compile checks of the luaT glue (mcw_cppamp_torch_amd/lua/): both C++ files go through
`g++ -fsyntax-only` against real declarations -- luaT.h, the TH headers and Torch's binding templates
(torch/generic/{Storage,Tensor,TensorOperator}.c), all read in place from a Torch7 source tree -- and the Lua files
through a block-structure check.

Headers: a Lua installation's lua.h / lauxlib.h where one exists, else the declarations-only pair under
tests/lua_decl/ (written from the Lua 5.1 manual: enough to type-check every call, nothing to link or run).
TH's THGeneral.h is a configure-time product of THGeneral.h.in; the test performs that one substitution itself (what
cmake's configure_file does with the two @/#cmakedefine placeholders) into a temporary directory.  Skipped where no
Torch7 source tree is present (set TORCH7_SRC; the reference tree's layout is understood).

What the glue serves once built into a Torch7 install: gpunn/test/test.lua:718-920 (SpatialConvolutionMM forward /
backward, single and batch) and :1314-1528 (SpatialMaxPooling forward / backward) create torch.GPUTensor inputs with
:gpu(), call nn modules typed with :gpu() (Module:type -> tensor:type, lua/gputorch.lua), and compare with :float()
copies of the results: constructors and :copy dispatch from gputorch_glue.cpp, the operators from gpunn_glue.cpp.
"""
import os
import re
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LUA_DIR = os.path.join(ROOT, "mcw_cppamp_torch_amd", "lua")


def torch7_tree():
    for root in (os.environ.get("TORCH7_SRC"), "/root/reference"):
        if root and os.path.exists(os.path.join(root, "mcw_torch7_core", "lib", "luaT", "luaT.h")):
            return root
    return None


def lua_include_dir():
    for d in (os.environ.get("LUA_INCDIR"), "/usr/include/luajit-2.1", "/usr/include/luajit-2.0", "/usr/include/lua5.1",
              "/usr/local/include", "/usr/include"):
        if d and os.path.exists(os.path.join(d, "lua.h")) and os.path.exists(os.path.join(d, "lauxlib.h")):
            return d, True
    return os.path.join(ROOT, "tests", "lua_decl"), False


def configured_th_general(tree, out_dir):
    """THGeneral.h from THGeneral.h.in, as configure_file writes it for a build without BLAS / LAPACK."""
    text = open(os.path.join(tree, "mcw_torch7_core", "lib", "TH", "THGeneral.h.in")).read()
    text = re.sub(r"^#cmakedefine (\w+)$", r"/* #undef \1 */", text, flags=re.M)
    text = text.replace("@TH_INLINE@", "inline")
    assert "@" not in text and "cmakedefine" not in text
    with open(os.path.join(out_dir, "THGeneral.h"), "w") as f:
        f.write(text)


@pytest.fixture(scope="module")
def include_flags(tmp_path_factory):
    tree = torch7_tree()
    if tree is None or shutil.which("g++") is None:
        pytest.skip("no Torch7 source tree (TORCH7_SRC) or no g++")
    gen = tmp_path_factory.mktemp("th_generated")
    configured_th_general(tree, str(gen))
    lua_dir, real = lua_include_dir()
    dirs = [lua_dir, os.path.join(tree, "mcw_torch7_core", "lib", "luaT"), str(gen),
            os.path.join(tree, "mcw_torch7_core", "lib", "TH"), os.path.join(tree, "gputorch", "torch")]
    return ["-I" + d for d in dirs], real


@pytest.mark.parametrize("source", ["gpunn_glue.cpp", "gputorch_glue.cpp"])
def test_glue_compiles(include_flags, source):
    flags, real_lua = include_flags
    cmd = ["g++", "-std=c++11", "-fsyntax-only", "-Wall", "-Wextra", "-Wno-unused-parameter", "-Wno-unused-function",
           "-Wno-write-strings"] + flags + [os.path.join(LUA_DIR, source)]
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-4000:]
    # warnings from the glue itself count; the templates' own (2014 C compiled as C++) do not
    own = [l for l in proc.stdout.splitlines() if "warning:" in l and os.path.join("lua", source) in l.split("warning:")[0]]
    assert not own, "\n".join(own)


def test_glue_registers_both_entry_points_and_every_operator_name():
    nn_glue = open(os.path.join(LUA_DIR, "gpunn_glue.cpp")).read()
    th_glue = open(os.path.join(LUA_DIR, "gputorch_glue.cpp")).read()
    assert 'extern "C" int luaopen_libgpunn(lua_State *L)' in nn_glue
    assert 'extern "C" int luaopen_libgputorch(lua_State *L)' in th_glue
    # the names the reference registers under torch.GPUTensor's nn table (gpunn-impl/SpatialConvolutionMM.cpp:431-443,
    # SpatialMaxPooling.cpp:385-396, Threshold.cpp:83-94)
    for name in ("SpatialConvolutionMM_updateOutput", "SpatialConvolutionMM_updateGradInput",
                 "SpatialConvolutionMM_accGradParameters", "SpatialMaxPooling_updateOutput",
                 "SpatialMaxPooling_updateGradInput", "Threshold_updateOutput", "Threshold_updateGradInput"):
        assert '{"%s", ' % name in nn_glue, name
    # the module functions of gputorch/init.cpp:68-79
    for name in ("synchronize", "getDevice", "deviceReset", "getDeviceCount", "getDeviceProperties", "setDevice", "seed",
                 "initialSeed", "manualSeed"):
        assert '{"%s", ' % name in th_glue, name
    # operators return a named field pushed explicitly, never "whatever is on top of the stack"
    bodies = re.findall(r"\nint (\w+)\(lua_State \*L\) \{(.*?)\n\}", nn_glue, flags=re.S)
    ops = [(n, b) for n, b in bodies if re.match(r"(conv|pool|thr|avg|sub|lsm|nll)_", n)]
    assert len(ops) == 17
    for name, body in ops:
        last = body.strip().splitlines()[-1].strip()
        assert last == "return 0;" or last.startswith('return returning(L, "'), (name, last)
        # no module field is fetched inside another call's argument list
        for line in body.splitlines():
            if re.search(r"(?<![A-Za-z_])field\(L,", line):
                assert re.match(r'\s*THGPUTensor \*\w+ = field\(L, "\w+"\);$', line), (name, line)


# ---- Lua sources: strings and comments stripped, block openers against `end` / `until` ------------------------------
def lua_tokens(text):
    out, i, n = [], 0, len(text)
    while i < n:
        c = text[i]
        if text.startswith("--[[", i) or text.startswith("[[", i):
            j = text.index("]]", i) + 2
            i = j
        elif text.startswith("--", i):
            j = text.find("\n", i)
            i = n if j < 0 else j
        elif c in "\"'":
            j = i + 1
            while text[j] != c:
                j += 2 if text[j] == "\\" else 1
            i = j + 1
        elif c.isalpha() or c == "_":
            j = i
            while j < n and (text[j].isalnum() or text[j] == "_"):
                j += 1
            out.append(text[i:j])
            i = j
        else:
            if c in "(){}[]":
                out.append(c)
            i += 1
    return out


@pytest.mark.parametrize("source", ["fuse.lua", "gputorch.lua", "gpunn.lua"])
def test_lua_sources_are_well_formed(source):
    toks = lua_tokens(open(os.path.join(LUA_DIR, source)).read())
    stack = []
    pairs = {")": "(", "}": "{", "]": "["}
    for i, t in enumerate(toks):
        if t in ("function", "if", "do", "repeat") or t in "({[":
            # `while ... do` and `for ... do` open one block: their `do` is the opener
            stack.append(t)
        elif t == "end":
            assert stack and stack[-1] in ("function", "if", "do"), (source, i, stack[-3:])
            stack.pop()
        elif t == "until":
            assert stack and stack[-1] == "repeat", (source, i)
            stack.pop()
        elif t in pairs:
            assert stack and stack[-1] == pairs[t], (source, i, t, stack[-3:])
            stack.pop()
    assert not stack, (source, stack)

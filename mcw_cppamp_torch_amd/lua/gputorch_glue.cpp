// luaT glue, tensor half: luaopen_libgputorch.  A Torch7 install that builds this file instead of the reference's
// gputorch/{init,Storage,Tensor}.cpp gets torch.GPUStorage and torch.GPUTensor backed by libthgpu (hipMalloc memory,
// hipMemcpy copies, HIP kernels) with the Lua API unchanged.
//
// Like the reference (gputorch/Storage.cpp:7-35, gputorch/Tensor.cpp:22-36) the two classes are Torch's own binding
// templates, torch/generic/Storage.c and torch/generic/Tensor.c, instantiated with real = float,
// Real = GPU: every THGPUStorage_* / THGPUTensor_* call they make resolves to the C ABI of include/thgpu.h.  The
// templates are taken from the Torch7 sources at build time (-I <gputorch>/torch, see build.py:build_lua_glue); this
// file supplies what the reference supplied around them, re-done for device memory that the host cannot dereference:
//   * the raw file I/O of a storage's floats (GPUStorage:write / :read, gputorch/Storage.cpp:15-31): staged through a
//     host buffer with thgpu_memcpy_d2h / thgpu_memcpy_h2d;
//   * :copy between every pair of tensor / storage types (gputorch/Storage.cpp:43-146, gputorch/Tensor.cpp:38-231);
//   * GPUStorage:totable, which the template writes as a loop over storage->data[i]: here one copy to the host;
//   * the three masked operations the template references and the GPU tensor never had (gputorch/Tensor.cpp:7-20);
//   * the tensor math the hot path and nn.Linear use (fill, zero, add, mul, div, addmm, addmv, addr, dot) with
//     Torch's argument conventions, and the arithmetic operators + - * / of torch/generic/TensorOperator.c on them
//     -- the reference generates these and some two hundred more with cwrap (gputorch/TensorMath.cpp), which stays
//     out of scope;
//   * the module functions of gputorch/init.cpp:10-94, with a real synchronize and real device properties.
// apply / map / map2 of the template walk host pointers; lua/gputorch.lua replaces them with host-staged versions,
// as gputorch/Tensor.lua:1-5 does for apply.
#include <luaT.h>  // brings lua.h and lauxlib.h in, as C

#include <TH.h>  // Torch7's host tensor library: THLongStorage, THFile, the host tensor types

#include "../../include/thgpu.h"

#include <cstring>
#include <vector>

namespace {

void lua_error_handler(const char *msg, void *data) { luaL_error(static_cast<lua_State *>(data), "%s", msg); }

// A storage's floats between a Torch file and device memory.
void read_floats(THFile *file, float *device, long n) {
    if (n <= 0) return;
    std::vector<float> host(static_cast<size_t>(n));
    THFile_readFloatRaw(file, host.data(), n);
    if (thgpu_memcpy_h2d(device, host.data(), n)) THError("%s", thgpu_last_error());
}
void write_floats(THFile *file, const float *device, long n) {
    if (n <= 0) return;
    std::vector<float> host(static_cast<size_t>(n));
    if (thgpu_memcpy_d2h(host.data(), device, n)) THError("%s", thgpu_last_error());
    THFile_writeFloatRaw(file, host.data(), n);
}

}  // namespace

// ---- what torch/generic/Tensor.c expects beside the C ABI -------------------------------------------------------------
static void THGPUTensor_maskedFill(THGPUTensor *, THByteTensor *, float) { THError("not yet implemented for GPU"); }
static void THGPUTensor_maskedCopy(THGPUTensor *, THByteTensor *, THGPUTensor *) { THError("not yet implemented for GPU"); }
static void THGPUTensor_maskedSelect(THGPUTensor *, THGPUTensor *, THByteTensor *) { THError("not yet implemented for GPU"); }

#define THFile_readRealRaw(file, data, size) read_floats(file, data, size)
#define THFile_writeRealRaw(file, data, size) write_floats(file, data, size)

#define real float
#define Real GPU
#define torch_Storage_(NAME) TH_CONCAT_4(torch_, Real, Storage_, NAME)
#define torch_Storage TH_CONCAT_STRING_3(torch., Real, Storage)
#define torch_Tensor_(NAME) TH_CONCAT_4(torch_, Real, Tensor_, NAME)
#define torch_Tensor TH_CONCAT_STRING_3(torch., Real, Tensor)

#define TH_GENERIC_FILE "generic/Storage.c"
#include "generic/Storage.c"
#undef TH_GENERIC_FILE
#define TH_GENERIC_FILE "generic/Tensor.c"
#include "generic/Tensor.c"
#undef TH_GENERIC_FILE

#undef real
#undef Real

namespace {

const char *const kTensor = "torch.GPUTensor";
const char *const kStorage = "torch.GPUStorage";

// ---- :copy, by the type of the source ---------------------------------------------------------------------------------
// One Lua function serves every destination class: its upvalue names the class and lists, per source class, the C
// function that performs the copy.
struct CopyRule {
    const char *source;
    void (*run)(void *dst, void *src);
};
struct CopyClass {
    const char *destination;
    const char *family;  // for the error message: "torch.*Tensor" or "torch.*Storage"
    const CopyRule *rules;
};

int copy_method(lua_State *L) {
    const CopyClass *cls = static_cast<const CopyClass *>(lua_touserdata(L, lua_upvalueindex(1)));
    void *dst = luaT_checkudata(L, 1, cls->destination);
    for (const CopyRule *r = cls->rules; r->source; ++r) {
        if (void *src = luaT_toudata(L, 2, r->source)) {
            r->run(dst, src);
            lua_settop(L, 1);
            return 1;  // the destination, for chaining
        }
    }
    return luaL_typerror(L, 2, cls->family);
}

#define THGPU_RULE(DST, KIND, SRC, FN) \
    { "torch." #SRC #KIND, [](void *d, void *s) { FN(static_cast<TH##DST##KIND *>(d), static_cast<TH##SRC##KIND *>(s)); } }
// The rules of one destination class; SELF names the same-type copy.
#define THGPU_COPY_CLASS(DST, KIND, SELF)                                                              \
    const CopyRule k##DST##KIND##Rules[] = {THGPU_RULE(DST, KIND, DST, SELF),                          \
                                            THGPU_RULE(DST, KIND, Byte, TH##DST##KIND##_copyByte),     \
                                            THGPU_RULE(DST, KIND, Char, TH##DST##KIND##_copyChar),     \
                                            THGPU_RULE(DST, KIND, Short, TH##DST##KIND##_copyShort),   \
                                            THGPU_RULE(DST, KIND, Int, TH##DST##KIND##_copyInt),       \
                                            THGPU_RULE(DST, KIND, Long, TH##DST##KIND##_copyLong),     \
                                            THGPU_RULE(DST, KIND, Float, TH##DST##KIND##_copyFloat),   \
                                            THGPU_RULE(DST, KIND, Double, TH##DST##KIND##_copyDouble), \
                                            THGPU_RULE(DST, KIND, GPU, TH##DST##KIND##_copyGPU),       \
                                            {nullptr, nullptr}};                                       \
    const CopyClass k##DST##KIND##Copy = {"torch." #DST #KIND, "torch.*" #KIND, k##DST##KIND##Rules};

#define THGPU_COPY_CLASSES(KIND)                           \
    THGPU_COPY_CLASS(Byte, KIND, THByte##KIND##_copy)      \
    THGPU_COPY_CLASS(Char, KIND, THChar##KIND##_copy)      \
    THGPU_COPY_CLASS(Short, KIND, THShort##KIND##_copy)    \
    THGPU_COPY_CLASS(Int, KIND, THInt##KIND##_copy)        \
    THGPU_COPY_CLASS(Long, KIND, THLong##KIND##_copy)      \
    THGPU_COPY_CLASS(Float, KIND, THFloat##KIND##_copy)    \
    THGPU_COPY_CLASS(Double, KIND, THDouble##KIND##_copy)  \
    THGPU_COPY_CLASS(GPU, KIND, THGPU##KIND##_copy)        \
    const CopyClass *const k##KIND##CopyClasses[] = {&kByte##KIND##Copy,  &kChar##KIND##Copy,   &kShort##KIND##Copy, \
                                                     &kInt##KIND##Copy,   &kLong##KIND##Copy,   &kFloat##KIND##Copy, \
                                                     &kDouble##KIND##Copy, &kGPU##KIND##Copy};

THGPU_COPY_CLASSES(Tensor)
THGPU_COPY_CLASSES(Storage)

void install_copy(lua_State *L, const CopyClass *const *classes, int count) {
    for (int i = 0; i < count; ++i) {
        luaT_pushmetatable(L, classes[i]->destination);
        lua_pushlightuserdata(L, const_cast<CopyClass *>(classes[i]));
        lua_pushcclosure(L, copy_method, 1);
        lua_setfield(L, -2, "copy");
        lua_pop(L, 1);
    }
}

// ---- GPUStorage:totable without touching device memory from the host ----------------------------------------------
int storage_totable(lua_State *L) {
    THGPUStorage *storage = static_cast<THGPUStorage *>(luaT_checkudata(L, 1, kStorage));
    std::vector<float> host(static_cast<size_t>(storage->size > 0 ? storage->size : 0));
    if (storage->size > 0 && thgpu_memcpy_d2h(host.data(), storage->data, storage->size))
        return luaL_error(L, "%s", thgpu_last_error());
    lua_createtable(L, static_cast<int>(host.size()), 0);
    for (size_t i = 0; i < host.size(); ++i) {
        lua_pushnumber(L, static_cast<lua_Number>(host[i]));
        lua_rawseti(L, -2, static_cast<int>(i) + 1);
    }
    return 1;
}

// ---- the tensor math of the hot path, with Torch's argument conventions -------------------------------------------
THGPUTensor *self_arg(lua_State *L) { return static_cast<THGPUTensor *>(luaT_checkudata(L, 1, kTensor)); }
THGPUTensor *tensor_at(lua_State *L, int idx) { return static_cast<THGPUTensor *>(luaT_toudata(L, idx, kTensor)); }
int chain(lua_State *L) {
    lua_settop(L, 1);
    return 1;
}

int m_fill(lua_State *L) {
    THGPUTensor_fill(self_arg(L), static_cast<float>(luaL_checknumber(L, 2)));
    return chain(L);
}
int m_zero(lua_State *L) {
    THGPUTensor_zero(self_arg(L));
    return chain(L);
}
// x:add(v) | x:add(src, v) | x:add(v, src) [x += v*src] | x:add(src1, v, src2) | x:add(src) [v = 1]
int m_add(lua_State *L) {
    THGPUTensor *self = self_arg(L);
    const int n = lua_gettop(L);
    if (n == 2 && lua_isnumber(L, 2)) {
        THGPUTensor_add(self, self, static_cast<float>(lua_tonumber(L, 2)));
    } else if (n == 2 && tensor_at(L, 2)) {
        THGPUTensor_cadd(self, self, 1.0f, tensor_at(L, 2));
    } else if (n == 3 && tensor_at(L, 2) && lua_isnumber(L, 3)) {
        THGPUTensor_add(self, tensor_at(L, 2), static_cast<float>(lua_tonumber(L, 3)));
    } else if (n == 3 && lua_isnumber(L, 2) && tensor_at(L, 3)) {
        THGPUTensor_cadd(self, self, static_cast<float>(lua_tonumber(L, 2)), tensor_at(L, 3));
    } else if (n == 3 && tensor_at(L, 2) && tensor_at(L, 3)) {
        THGPUTensor_cadd(self, tensor_at(L, 2), 1.0f, tensor_at(L, 3));
    } else if (n == 4 && tensor_at(L, 2) && lua_isnumber(L, 3) && tensor_at(L, 4)) {
        THGPUTensor_cadd(self, tensor_at(L, 2), static_cast<float>(lua_tonumber(L, 3)), tensor_at(L, 4));
    } else {
        return luaL_error(L, "expected arguments: *GPUTensor* [GPUTensor] float | *GPUTensor* [GPUTensor] [float] GPUTensor");
    }
    return chain(L);
}
// x:mul(v) | x:mul(src, v); likewise div
template <void (*OP)(THGPUTensor *, THGPUTensor *, float)>
int m_scale(lua_State *L) {
    THGPUTensor *self = self_arg(L);
    if (lua_gettop(L) == 2 && lua_isnumber(L, 2)) OP(self, self, static_cast<float>(lua_tonumber(L, 2)));
    else if (lua_gettop(L) == 3 && tensor_at(L, 2) && lua_isnumber(L, 3))
        OP(self, tensor_at(L, 2), static_cast<float>(lua_tonumber(L, 3)));
    else return luaL_error(L, "expected arguments: *GPUTensor* [GPUTensor] float");
    return chain(L);
}
// x:addmm([beta,] [t,] [alpha,] a, b) and the same shape for addmv / addr: the trailing two tensors are the operands,
// a tensor before them is t (default: x itself), numbers are beta (before t) and alpha (after it); a single number
// is alpha.
template <void (*OP)(THGPUTensor *, float, THGPUTensor *, float, THGPUTensor *, THGPUTensor *)>
int m_blas3(lua_State *L) {
    THGPUTensor *self = self_arg(L);
    const int n = lua_gettop(L);
    if (n < 3 || !tensor_at(L, n - 1) || !tensor_at(L, n)) return luaL_error(L, "two GPUTensor operands expected");
    THGPUTensor *a = tensor_at(L, n - 1), *b = tensor_at(L, n), *t = self;
    float beta = 1.0f, alpha = 1.0f;
    bool seen_t = false;
    int numbers = 0;
    for (int i = 2; i <= n - 2; ++i) {
        if (tensor_at(L, i)) {
            if (seen_t) return luaL_error(L, "too many tensors");
            t = tensor_at(L, i);
            seen_t = true;
        } else if (lua_isnumber(L, i)) {
            const float v = static_cast<float>(lua_tonumber(L, i));
            if (++numbers > 2) return luaL_error(L, "too many numbers");
            // beta comes before t; without a t in the list the first of two numbers is beta, a single one is alpha
            if (!seen_t && (i + 1 <= n - 2)) beta = v;
            else alpha = v;
        } else {
            return luaL_typerror(L, i, "number or torch.GPUTensor");
        }
    }
    OP(self, beta, t, alpha, a, b);
    return chain(L);
}
int m_dot(lua_State *L) {
    THGPUTensor *other = static_cast<THGPUTensor *>(luaT_checkudata(L, 2, kTensor));
    lua_pushnumber(L, THGPUTensor_dot(self_arg(L), other));
    return 1;
}

// ---- a + b, a - b, -a, a * b, a / b (the semantics of torch/generic/TensorOperator.c:5-155) ------------------------
// The result is always a new tensor (or a number, for the product of two vectors).
THGPUTensor *push_result_like(lua_State *L, THGPUTensor *shape, bool copy) {
    THGPUTensor *r = THGPUTensor_new();
    luaT_pushudata(L, r, kTensor);  // owned by Lua from here on
    THGPUTensor_resizeAs(r, shape);
    if (copy) THGPUTensor_copy(r, shape);
    return r;
}
int op_add(lua_State *L) {
    THGPUTensor *a = tensor_at(L, 1), *b = tensor_at(L, 2);
    if (!a && !b) return luaL_error(L, "expecting two Tensors or one Tensor and one number");
    if (a && b) {
        THGPUTensor *r = push_result_like(L, a, true);
        THGPUTensor_cadd(r, r, 1.0f, b);
    } else {
        THGPUTensor *r = push_result_like(L, a ? a : b, true);
        THGPUTensor_add(r, r, static_cast<float>(luaL_checknumber(L, a ? 2 : 1)));
    }
    return 1;
}
int op_sub(lua_State *L) {
    THGPUTensor *a = tensor_at(L, 1), *b = tensor_at(L, 2);
    if (!a && !b) return luaL_error(L, "expecting two Tensors or one Tensor and one number");
    if (a && b) {
        THGPUTensor *r = push_result_like(L, a, true);
        THGPUTensor_cadd(r, r, -1.0f, b);
    } else if (a) {
        THGPUTensor *r = push_result_like(L, a, true);
        THGPUTensor_add(r, r, -static_cast<float>(luaL_checknumber(L, 2)));
    } else {  // number - tensor
        THGPUTensor *r = push_result_like(L, b, false);
        THGPUTensor_fill(r, static_cast<float>(luaL_checknumber(L, 1)));
        THGPUTensor_cadd(r, r, -1.0f, b);
    }
    return 1;
}
int op_unm(lua_State *L) {
    THGPUTensor *r = push_result_like(L, self_arg(L), true);
    THGPUTensor_mul(r, r, -1.0f);
    return 1;
}
int op_mul(lua_State *L) {
    THGPUTensor *a = tensor_at(L, 1), *b = tensor_at(L, 2);
    if (!a && !b) return luaL_error(L, "expecting two Tensors or one Tensor and one number");
    if (!a || !b) {
        THGPUTensor *r = push_result_like(L, a ? a : b, true);
        THGPUTensor_mul(r, r, static_cast<float>(luaL_checknumber(L, a ? 2 : 1)));
        return 1;
    }
    if (a->nDimension == 1 && b->nDimension == 1) {
        lua_pushnumber(L, THGPUTensor_dot(a, b));
    } else if (a->nDimension == 2 && b->nDimension == 1) {
        THGPUTensor *r = THGPUTensor_newWithSize1d(a->size[0]);
        luaT_pushudata(L, r, kTensor);
        THGPUTensor_zero(r);
        THGPUTensor_addmv(r, 1.0f, r, 1.0f, a, b);
    } else if (a->nDimension == 2 && b->nDimension == 2) {
        THGPUTensor *r = THGPUTensor_newWithSize2d(a->size[0], b->size[1]);
        luaT_pushudata(L, r, kTensor);
        THGPUTensor_zero(r);
        THGPUTensor_addmm(r, 1.0f, r, 1.0f, a, b);
    } else {
        return luaL_error(L, "multiplication between %dD and %dD tensors not yet supported", a->nDimension, b->nDimension);
    }
    return 1;
}
int op_div(lua_State *L) {
    THGPUTensor *a = self_arg(L);
    if (!lua_isnumber(L, 2)) return luaL_error(L, "Tensor division by a number expected");
    THGPUTensor *r = push_result_like(L, a, true);
    THGPUTensor_div(r, r, static_cast<float>(lua_tonumber(L, 2)));
    return 1;
}

const struct luaL_Reg kOperators[] = {{"__add__", op_add}, {"__sub__", op_sub}, {"__unm__", op_unm},
                                      {"__mul__", op_mul}, {"__div__", op_div}, {NULL, NULL}};

const struct luaL_Reg kMath[] = {{"fill", m_fill},
                                 {"zero", m_zero},
                                 {"add", m_add},
                                 {"mul", m_scale<THGPUTensor_mul>},
                                 {"div", m_scale<THGPUTensor_div>},
                                 {"addmm", m_blas3<THGPUTensor_addmm>},
                                 {"addmv", m_blas3<THGPUTensor_addmv>},
                                 {"addr", m_blas3<THGPUTensor_addr>},
                                 {"dot", m_dot},
                                 {NULL, NULL}};

// ---- module functions (gputorch/init.cpp:10-81) ---------------------------------------------------------------------
int l_synchronize(lua_State *L) {
    if (thgpu_synchronize()) return luaL_error(L, "%s", thgpu_last_error());
    return 0;
}
int l_get_device(lua_State *L) {  // one device, numbered from 1 as in Lua
    lua_pushnumber(L, 1);
    return 1;
}
int l_get_device_count(lua_State *L) {
    lua_pushnumber(L, 1);
    return 1;
}
int l_set_device(lua_State *L) {
    if (luaL_checkint(L, 1) != 1) return luaL_error(L, "this library drives one device (1)");
    return 0;
}
int l_device_reset(lua_State *L) {
    if (thgpu_synchronize() || thgpu_empty_cache()) return luaL_error(L, "%s", thgpu_last_error());
    return 0;
}
int l_device_properties(lua_State *L) {
    char name[256] = "";
    int cus = 0;
    long mem = 0;
    if (thgpu_device_info(name, sizeof(name), &cus, &mem)) return luaL_error(L, "%s", thgpu_last_error());
    lua_newtable(L);
    lua_pushstring(L, name);
    lua_setfield(L, -2, "name");
    lua_pushnumber(L, cus);
    lua_setfield(L, -2, "multiProcessorCount");
    lua_pushnumber(L, static_cast<lua_Number>(mem));
    lua_setfield(L, -2, "totalGlobalMem");
    return 1;
}
// The reference's seed functions are stubs (gputorch/init.cpp:54-68); nothing on this path draws random numbers on
// the device, so they stay inert: seed / initialSeed report 0, manualSeed accepts its argument.
int l_seed(lua_State *L) {
    lua_pushnumber(L, 0);
    return 1;
}
int l_manual_seed(lua_State *L) {
    (void)luaL_checknumber(L, 1);
    return 0;
}
int l_empty_cache(lua_State *L) {
    if (thgpu_empty_cache()) return luaL_error(L, "%s", thgpu_last_error());
    return 0;
}

const struct luaL_Reg kModule[] = {{"synchronize", l_synchronize},
                                   {"getDevice", l_get_device},
                                   {"deviceReset", l_device_reset},
                                   {"getDeviceCount", l_get_device_count},
                                   {"getDeviceProperties", l_device_properties},
                                   {"setDevice", l_set_device},
                                   {"seed", l_seed},
                                   {"initialSeed", l_seed},
                                   {"manualSeed", l_manual_seed},
                                   {"emptyCache", l_empty_cache},
                                   {NULL, NULL}};

}  // namespace

// gputorch/torch/utils.h:23-24: sizes given as numbers or as one torch.LongStorage.
extern "C" THLongStorage *gputorch_checklongargs(lua_State *L, int index) {
    const int narg = lua_gettop(L) - index + 1;
    if (narg == 1) {
        if (THLongStorage *given = static_cast<THLongStorage *>(luaT_toudata(L, index, "torch.LongStorage"))) {
            THLongStorage *copy = THLongStorage_newWithSize(given->size);
            THLongStorage_copy(copy, given);
            return copy;
        }
    }
    THLongStorage *sizes = THLongStorage_newWithSize(narg > 0 ? narg : 0);
    for (int i = 0; i < narg; ++i) {
        if (!lua_isnumber(L, index + i)) {
            THLongStorage_free(sizes);
            luaL_argerror(L, index + i, "number expected");
        }
        THLongStorage_set(sizes, i, static_cast<long>(lua_tonumber(L, index + i)));
    }
    return sizes;
}

extern "C" int gputorch_islongargs(lua_State *L, int index) {
    const int narg = lua_gettop(L) - index + 1;
    if (narg == 1 && luaT_toudata(L, index, "torch.LongStorage")) return 1;
    for (int i = 0; i < narg; ++i)
        if (!lua_isnumber(L, index + i)) return 0;
    return 1;
}

extern "C" int luaopen_libgputorch(lua_State *L) {
    // TH-named functions of the library report through this handler, as luaopen_libtorch arranges for TH itself
    // (mcw_torch7_core/init.c:38-55).
    THGPUSetErrorHandler(lua_error_handler, L);
    if (thgpu_init() != 0) return luaL_error(L, "%s", thgpu_last_error());

    lua_newtable(L);
    luaL_register(L, NULL, kModule);

    // the two classes from Torch's templates
    torch_GPUStorage_init(L);
    torch_GPUTensor_init(L);

    // what replaces or extends the templates' methods
    install_copy(L, kStorageCopyClasses, 8);
    install_copy(L, kTensorCopyClasses, 8);
    luaT_pushmetatable(L, kStorage);
    lua_pushcfunction(L, storage_totable);
    lua_setfield(L, -2, "totable");
    lua_pop(L, 1);
    luaT_pushmetatable(L, kTensor);
    luaL_register(L, NULL, kMath);
    luaL_register(L, NULL, kOperators);
    lua_pop(L, 1);
    return 1;
}

// luaT glue: registers libthgpu's operators under the names, and reading the module fields, that the reference's
// gpunn does, so that a Torch7 install can `require 'gpunn'` with this library behind it.
//
// Replaces gpunn/init.cpp:5-11 (luaopen_libgpunn -> open_libgpunn, gputorch/lib/THC/gpunn-impl/init.cpp:34-65) and the
// luaT halves of gpunn-impl/SpatialConvolutionMM.cpp:110-443, SpatialMaxPooling.cpp:205-396, Threshold.cpp:16-94,
// SpatialAveragePooling.cpp:67-248, SpatialSubSampling.cpp:246-452, LogSoftMax.cpp:115-194 and
// ClassNLLCriterion.cpp:96-198.  Every function is called from Lua as input.nn.<Name>(self, input[, gradOutput[,
// scale]]) (mcw_nn/SpatialConvolutionMM.lua:48-60): argument 1 is the module table, whose fields are read by the
// names the reference reads (SpatialConvolutionMM.cpp:116-128).
//
// Built by mcw_cppamp_torch_amd/build.py only where lua.h and luaT.h are found (LUA_INCDIR / TORCH_INSTALL, or the
// usual prefixes); link with -lthgpu -lluaT.  Optional module fields beyond the reference's:
//   padW, padH        separate paddings (default: the reference's single `padding`)
//   fusedThreshold, fusedValue   set by gpunn.fuse(net) on a convolution followed by nn.Threshold: the threshold is
//                     applied as the output is stored
//   inputThreshold    set by gpunn.fuse(net) on a convolution / max-pooling layer preceded by nn.Threshold: gradInput
//                     is zeroed where the input is not above it
//   inputInPaddedBuffer   set by gpunn.fuse(net) while the layer's input is a view into a zero-bordered buffer that
//                     the layer in front writes (lua/fuse.lua): the gathered convolution reads it there
//   twinTarget, gradOutputInTwin   set by the fused container's updateGradInput (lua/fuse.lua) for one call: a view to
//                     store a second copy of gradInput through, and the statement that gradOutput already lies in this
//                     layer's fgradInput; the call leaves wroteTwin (boolean) behind
//   gradOutputTwin    a torch.GPUTensor the module keeps for SpatialConvolutionMM_gradOutputTwin to turn into that view
extern "C" {
#include <lua.h>
#include <lauxlib.h>
#include <luaT.h>
}
#include "../../include/thgpu.h"

namespace {

const char *const kTensor = "torch.GPUTensor";

int fail(lua_State *L, int rc) { return rc ? luaL_error(L, "%s", thgpu_last_error()) : 0; }

THGPUTensor *field(lua_State *L, const char *name) {
    return static_cast<THGPUTensor *>(luaT_getfieldcheckudata(L, 1, name, kTensor));
}
// An optional tensor field: NULL when absent (or false).
THGPUTensor *opt_field(lua_State *L, const char *name) {
    lua_getfield(L, 1, name);
    THGPUTensor *t = lua_toboolean(L, -1) ? static_cast<THGPUTensor *>(luaT_toudata(L, -1, kTensor)) : NULL;
    lua_pop(L, 1);
    return t;
}
bool flag_field(lua_State *L, const char *name) {
    lua_getfield(L, 1, name);
    const bool on = lua_toboolean(L, -1) != 0;
    lua_pop(L, 1);
    return on;
}
void set_flag_field(lua_State *L, const char *name, bool value) {
    lua_pushboolean(L, value ? 1 : 0);
    lua_setfield(L, 1, name);
}
THGPUTensor *arg(lua_State *L, int idx) { return static_cast<THGPUTensor *>(luaT_checkudata(L, idx, kTensor)); }

bool has_field(lua_State *L, const char *name) {
    lua_getfield(L, 1, name);
    const bool present = !lua_isnil(L, -1);
    lua_pop(L, 1);
    return present;
}
double opt_number(lua_State *L, const char *name, double dflt) {
    lua_getfield(L, 1, name);
    const double v = lua_isnil(L, -1) ? dflt : lua_tonumber(L, -1);
    lua_pop(L, 1);
    return v;
}

struct ConvFields {
    int kW, kH, dW, dH, padW, padH;
};
ConvFields conv_fields(lua_State *L) {
    ConvFields f;
    f.kW = luaT_getfieldcheckint(L, 1, "kW");
    f.kH = luaT_getfieldcheckint(L, 1, "kH");
    f.dW = luaT_getfieldcheckint(L, 1, "dW");
    f.dH = luaT_getfieldcheckint(L, 1, "dH");
    const int pad = luaT_getfieldcheckint(L, 1, "padding");
    f.padW = static_cast<int>(opt_number(L, "padW", pad));
    f.padH = static_cast<int>(opt_number(L, "padH", pad));
    return f;
}
struct PoolFields {
    int kW, kH, dW, dH;
};
PoolFields pool_fields(lua_State *L) {
    return PoolFields{luaT_getfieldcheckint(L, 1, "kW"), luaT_getfieldcheckint(L, 1, "kH"),
                      luaT_getfieldcheckint(L, 1, "dW"), luaT_getfieldcheckint(L, 1, "dH")};
}

// Every operator fetches the module's tensors into named locals, one statement each (each fetch pushes the value on
// the Lua stack, and the order of evaluation of function arguments is unspecified in C++), and returns the field the
// reference's Lua wrappers return (mcw_nn/SpatialConvolutionMM.lua:48-55), pushed explicitly.
int returning(lua_State *L, const char *field_name) {
    lua_getfield(L, 1, field_name);
    return 1;
}

// ---- nn.SpatialConvolutionMM -------------------------------------------------------------------------------------
int conv_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    const ConvFields f = conv_fields(L);
    THGPUTensor *weight = field(L, "weight");
    THGPUTensor *bias = field(L, "bias");
    THGPUTensor *finput = field(L, "finput");
    THGPUTensor *fgradInput = field(L, "fgradInput");
    THGPUTensor *output = field(L, "output");
    const int flags = (has_field(L, "fusedThreshold") ? THGPU_FUSE_THRESHOLD : 0) |
                      (has_field(L, "inputInPaddedBuffer") ? THGPU_INPUT_IN_PADDED_BUFFER : 0);
    int rc;
    if (flags) {
        const float threshold = static_cast<float>(opt_number(L, "fusedThreshold", 0));
        const float value = static_cast<float>(opt_number(L, "fusedValue", 0));
        rc = thgpu_SpatialConvolutionMM_updateOutputFused(input, weight, bias, finput, fgradInput, output, f.kW, f.kH,
                                                          f.dW, f.dH, f.padW, f.padH, flags, threshold, value);
    } else {
        rc = thgpu_SpatialConvolutionMM_updateOutput(input, weight, bias, finput, fgradInput, output, f.kW, f.kH, f.dW,
                                                     f.dH, f.padW, f.padH);
    }
    fail(L, rc);
    return returning(L, "output");
}
int conv_updateGradInput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    const ConvFields f = conv_fields(L);
    THGPUTensor *weight = field(L, "weight");
    THGPUTensor *finput = field(L, "finput");
    THGPUTensor *fgradInput = field(L, "fgradInput");
    THGPUTensor *gradInput = field(L, "gradInput");
    THGPUTensor *twin = opt_field(L, "twinTarget");
    const bool delivered = flag_field(L, "gradOutputInTwin");
    int rc;
    if (twin || delivered) {
        const int flags = (has_field(L, "inputThreshold") ? THGPU_FUSE_INPUT_MASK : 0) |
                          (delivered ? THGPU_GRADOUTPUT_IN_TWIN : 0);
        const float threshold = static_cast<float>(opt_number(L, "inputThreshold", 0));
        int wrote = 0;
        rc = thgpu_SpatialConvolutionMM_updateGradInputTwin(input, gradOutput, weight, finput, fgradInput, gradInput,
                                                            f.kW, f.kH, f.dW, f.dH, f.padW, f.padH, flags, threshold,
                                                            twin, &wrote);
        set_flag_field(L, "wroteTwin", wrote != 0);
    } else if (has_field(L, "inputThreshold")) {
        const float threshold = static_cast<float>(opt_number(L, "inputThreshold", 0));
        rc = thgpu_SpatialConvolutionMM_updateGradInputFused(input, gradOutput, weight, finput, fgradInput, gradInput,
                                                             f.kW, f.kH, f.dW, f.dH, f.padW, f.padH,
                                                             THGPU_FUSE_INPUT_MASK, threshold);
    } else {
        rc = thgpu_SpatialConvolutionMM_updateGradInput(input, gradOutput, weight, finput, fgradInput, gradInput, f.kW,
                                                        f.kH, f.dW, f.dH, f.padW, f.padH);
    }
    fail(L, rc);
    return returning(L, "gradInput");
}
// input.nn.SpatialConvolutionMM_gradOutputTwin(self, input): the view through which the producer of this layer's
// gradOutput may store it in padded form (self.gradOutputTwin, returned), or nil when the layer's gradInput does not
// take the gathered route.
int conv_gradOutputTwin(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    const ConvFields f = conv_fields(L);
    THGPUTensor *weight = field(L, "weight");
    THGPUTensor *fgradInput = field(L, "fgradInput");
    THGPUTensor *twin = field(L, "gradOutputTwin");
    int available = 0;
    fail(L, thgpu_SpatialConvolutionMM_gradOutputTwin(input, weight, fgradInput, twin, f.kW, f.kH, f.dW, f.dH, f.padW,
                                                      f.padH, &available));
    if (!available) {
        lua_pushnil(L);
        return 1;
    }
    return returning(L, "gradOutputTwin");
}
int conv_accGradParameters(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    const float scale = static_cast<float>(luaL_optnumber(L, 4, 1));  // SpatialConvolutionMM.cpp:326
    const ConvFields f = conv_fields(L);
    THGPUTensor *gradWeight = field(L, "gradWeight");
    THGPUTensor *gradBias = field(L, "gradBias");
    THGPUTensor *finput = field(L, "finput");
    THGPUTensor *fgradInput = field(L, "fgradInput");
    const int flags = has_field(L, "inputInPaddedBuffer") ? THGPU_INPUT_IN_PADDED_BUFFER : 0;
    fail(L, thgpu_SpatialConvolutionMM_accGradParametersFused(input, gradOutput, gradWeight, gradBias, finput,
                                                              fgradInput, f.kW, f.kH, f.dW, f.dH, f.padW, f.padH, scale,
                                                              flags));
    return 0;
}

// ---- nn.SpatialMaxPooling ------------------------------------------------------------------------------------------
int pool_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    const PoolFields f = pool_fields(L);
    THGPUTensor *output = field(L, "output");
    THGPUTensor *indices = field(L, "indices");
    fail(L, thgpu_SpatialMaxPooling_updateOutput(input, output, indices, f.kW, f.kH, f.dW, f.dH));
    return returning(L, "output");
}
int pool_updateGradInput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    const PoolFields f = pool_fields(L);
    THGPUTensor *gradInput = field(L, "gradInput");
    THGPUTensor *indices = field(L, "indices");
    THGPUTensor *twin = opt_field(L, "twinTarget");
    int rc;
    if (twin) {
        const float threshold = static_cast<float>(opt_number(L, "inputThreshold", 0));
        int wrote = 0;
        rc = thgpu_SpatialMaxPooling_updateGradInputTwin(input, gradOutput, gradInput, indices, f.kW, f.kH, f.dW, f.dH,
                                                         has_field(L, "inputThreshold") ? THGPU_FUSE_INPUT_MASK : 0,
                                                         threshold, twin, &wrote);
        set_flag_field(L, "wroteTwin", wrote != 0);
    } else if (has_field(L, "inputThreshold")) {
        const float threshold = static_cast<float>(opt_number(L, "inputThreshold", 0));
        rc = thgpu_SpatialMaxPooling_updateGradInputMasked(input, gradOutput, gradInput, indices, f.kW, f.kH, f.dW, f.dH,
                                                           threshold);
    } else {
        rc = thgpu_SpatialMaxPooling_updateGradInput(input, gradOutput, gradInput, indices, f.kW, f.kH, f.dW, f.dH);
    }
    fail(L, rc);
    return returning(L, "gradInput");
}

// ---- nn.Threshold / nn.ReLU ------------------------------------------------------------------------------------------
int thr_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *output = field(L, "output");
    const float threshold = static_cast<float>(luaT_getfieldchecknumber(L, 1, "threshold"));
    const float value = static_cast<float>(luaT_getfieldchecknumber(L, 1, "val"));
    fail(L, thgpu_Threshold_updateOutput(input, output, threshold, value));
    return returning(L, "output");
}
int thr_updateGradInput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    THGPUTensor *gradInput = field(L, "gradInput");
    const float threshold = static_cast<float>(luaT_getfieldchecknumber(L, 1, "threshold"));
    fail(L, thgpu_Threshold_updateGradInput(input, gradOutput, gradInput, threshold));
    return returning(L, "gradInput");
}

// ---- nn.SpatialAveragePooling / nn.SpatialSubSampling ------------------------------------------------------------------
int avg_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    const PoolFields f = pool_fields(L);
    THGPUTensor *output = field(L, "output");
    fail(L, thgpu_SpatialAveragePooling_updateOutput(input, output, f.kW, f.kH, f.dW, f.dH));
    return returning(L, "output");
}
int avg_updateGradInput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    const PoolFields f = pool_fields(L);
    THGPUTensor *gradInput = field(L, "gradInput");
    fail(L, thgpu_SpatialAveragePooling_updateGradInput(input, gradOutput, gradInput, f.kW, f.kH, f.dW, f.dH));
    return returning(L, "gradInput");
}
int sub_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    const PoolFields f = pool_fields(L);
    THGPUTensor *weight = field(L, "weight");
    THGPUTensor *bias = field(L, "bias");
    THGPUTensor *output = field(L, "output");
    fail(L, thgpu_SpatialSubSampling_updateOutput(input, weight, bias, output, f.kW, f.kH, f.dW, f.dH));
    return returning(L, "output");
}
int sub_updateGradInput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    const PoolFields f = pool_fields(L);
    THGPUTensor *weight = field(L, "weight");
    THGPUTensor *gradInput = field(L, "gradInput");
    fail(L, thgpu_SpatialSubSampling_updateGradInput(input, gradOutput, weight, gradInput, f.kW, f.kH, f.dW, f.dH));
    return returning(L, "gradInput");
}
int sub_accGradParameters(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *gradOutput = arg(L, 3);
    const float scale = static_cast<float>(luaL_optnumber(L, 4, 1));
    const PoolFields f = pool_fields(L);
    THGPUTensor *gradWeight = field(L, "gradWeight");
    THGPUTensor *gradBias = field(L, "gradBias");
    fail(L, thgpu_SpatialSubSampling_accGradParameters(input, gradOutput, gradWeight, gradBias, f.kW, f.kH, f.dW, f.dH,
                                                       scale));
    return 0;
}

// ---- nn.LogSoftMax / nn.ClassNLLCriterion ----------------------------------------------------------------------------------
int lsm_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *output = field(L, "output");
    fail(L, thgpu_LogSoftMax_updateOutput(input, output));
    return returning(L, "output");
}
int lsm_updateGradInput(lua_State *L) {
    THGPUTensor *gradOutput = arg(L, 3);
    THGPUTensor *output = field(L, "output");
    THGPUTensor *gradInput = field(L, "gradInput");
    fail(L, thgpu_LogSoftMax_updateGradInput(gradOutput, output, gradInput));
    return returning(L, "gradInput");
}
int nll_updateOutput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *target = arg(L, 3);
    THGPUTensor *outputTensor = field(L, "outputTensor");
    const int size_average = luaT_getfieldcheckboolean(L, 1, "sizeAverage");
    fail(L, thgpu_ClassNLLCriterion_updateOutput(input, target, outputTensor, size_average));
    return returning(L, "outputTensor");
}
int nll_updateGradInput(lua_State *L) {
    THGPUTensor *input = arg(L, 2);
    THGPUTensor *target = arg(L, 3);
    THGPUTensor *gradInput = field(L, "gradInput");
    const int size_average = luaT_getfieldcheckboolean(L, 1, "sizeAverage");
    fail(L, thgpu_ClassNLLCriterion_updateGradInput(input, target, gradInput, size_average));
    return returning(L, "gradInput");
}

const struct luaL_Reg kOps[] = {
    {"SpatialConvolutionMM_updateOutput", conv_updateOutput},
    {"SpatialConvolutionMM_updateGradInput", conv_updateGradInput},
    {"SpatialConvolutionMM_accGradParameters", conv_accGradParameters},
    {"SpatialConvolutionMM_gradOutputTwin", conv_gradOutputTwin},
    {"SpatialMaxPooling_updateOutput", pool_updateOutput},
    {"SpatialMaxPooling_updateGradInput", pool_updateGradInput},
    {"Threshold_updateOutput", thr_updateOutput},
    {"Threshold_updateGradInput", thr_updateGradInput},
    {"SpatialAveragePooling_updateOutput", avg_updateOutput},
    {"SpatialAveragePooling_updateGradInput", avg_updateGradInput},
    {"SpatialSubSampling_updateOutput", sub_updateOutput},
    {"SpatialSubSampling_updateGradInput", sub_updateGradInput},
    {"SpatialSubSampling_accGradParameters", sub_accGradParameters},
    {"LogSoftMax_updateOutput", lsm_updateOutput},
    {"LogSoftMax_updateGradInput", lsm_updateGradInput},
    {"ClassNLLCriterion_updateOutput", nll_updateOutput},
    {"ClassNLLCriterion_updateGradInput", nll_updateGradInput},
    {NULL, NULL}};

// gputorch.synchronize() / the library's own switches, as a small table `gpunn.thgpu`.
int l_synchronize(lua_State *L) { return fail(L, thgpu_synchronize()); }
int l_conv_mode(lua_State *L) { return fail(L, thgpu_conv_set_mode(static_cast<int>(luaL_checkinteger(L, 1)))); }
int l_finput_reuse(lua_State *L) { return fail(L, thgpu_conv_set_finput_reuse(lua_toboolean(L, 1))); }
int l_conv_gathers(lua_State *L) {  // (B, C, H, W, M, kW, kH, dW, dH, padW, padH)
    int a[10];
    for (int i = 0; i < 10; ++i) a[i] = static_cast<int>(luaL_checkinteger(L, i + 2));
    lua_pushboolean(L, thgpu_conv_gathers(static_cast<long>(luaL_checkinteger(L, 1)), a[0], a[1], a[2], a[3], a[4], a[5],
                                          a[6], a[7], a[8], a[9]));
    return 1;
}
const struct luaL_Reg kLib[] = {{"synchronize", l_synchronize},    {"setConvMode", l_conv_mode},
                                {"setFinputReuse", l_finput_reuse}, {"convGathers", l_conv_gathers},
                                {NULL, NULL}};

void lua_error_handler(const char *msg, void *data) { luaL_error(static_cast<lua_State *>(data), "%s", msg); }

}  // namespace

extern "C" int luaopen_libgpunn(lua_State *L) {
    // TH-named functions report through this handler, as luaopen_libtorch arranges for TH
    // (mcw_torch7_core/init.c:38-55).
    THGPUSetErrorHandler(lua_error_handler, L);
    if (thgpu_init() != 0) return luaL_error(L, "%s", thgpu_last_error());
    luaT_pushmetatable(L, kTensor);
    luaT_registeratname(L, kOps, "nn");
    lua_pop(L, 1);
    lua_newtable(L);
    luaL_register(L, NULL, kLib);
    lua_setfield(L, LUA_GLOBALSINDEX, "thgpu");
    return 0;
}

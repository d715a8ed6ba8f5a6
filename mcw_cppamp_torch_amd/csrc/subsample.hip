// nn.SpatialAveragePooling and nn.SpatialSubSampling: kernels and operator entry points.
//
// Both walk kH x kW windows with strides dH x dW and no padding, Ho = (H - kH) / dH + 1.
//   SpatialAveragePooling  out = 0 + sum(window)            -- a window SUM: neither the CPU module
//                          (mcw_nn/generic/SpatialAveragePooling.c:56-90) nor the GPU one
//                          (gpunn-impl/SpatialAveragePooling.cpp:46-61) divides by the window size
//   SpatialSubSampling     out = bias[k] + weight[k] * sum(window), one weight and bias per plane
//                          (mcw_nn/generic/SpatialSubSampling.c:58-96)
// The window sum is taken ky ascending, kx ascending into a float that starts at zero, as the CPU
// loops do, and product and sum are rounded separately, so the forward results are bit-identical
// to the CPU modules'.  The backward pass is a gather: a thread owns one input pixel and adds the
// gradients of the windows that cover it in the order the CPU's scatter reaches that pixel (window
// row ascending, window column ascending, starting from the zero fill;
// SpatialAveragePooling.c:151-170, SpatialSubSampling.c:161-180) -- bit-identical again, with
// overlapping windows allowed (the reference GPU code insists on dW == kW, dH == kH:
// SpatialAveragePooling.cpp:194-195, SpatialSubSampling.cpp:329-330) and without atomics.
// accGradParameters (SpatialSubSampling.c:236-270) sums whole planes; the per-image sums are block
// reductions in a fixed order and the images are then added one after another as on the CPU, so the
// result is deterministic and agrees with the CPU to rounding.
#include "common.h"

using namespace thgpu;

namespace {

struct SubGeom {
    int H, W, kH, kW, dH, dW, Ho, Wo;
    FastDiv divWo, divHoWo, divW, divHW, divC, divDH, divDW;
};

inline float *dptr(const THGPUTensor *t) { return THGPUTensor_data(t); }

inline const char *sub_label(const char *family, const SubGeom &g, long planes) {
    if (!prof_enabled()) return family;
    return prof_label("%s planes=%ld %dx%d k=%dx%d s=%dx%d", family, planes, g.H, g.W, g.kH, g.kW, g.dH, g.dW);
}

// One thread per output element.
template <bool SUBSAMPLE>
__global__ __launch_bounds__(256) void subsample_fwd_kernel(const float *__restrict__ in, const float *__restrict__ weight,
                                                            const float *__restrict__ bias, float *__restrict__ out,
                                                            const SubGeom g, unsigned total) {
    const unsigned o = blockIdx.x * 256u + threadIdx.x;
    if (o >= total) return;
    unsigned plane, rem, i, j;
    g.divHoWo.divmod(o, plane, rem);
    g.divWo.divmod(rem, i, j);
    const float *p = in + ((long)plane * g.H + (long)i * g.dH) * g.W + (long)j * g.dW;
    float sum = 0.0f;
    for (int ky = 0; ky < g.kH; ++ky) {
        for (int kx = 0; kx < g.kW; ++kx) sum += p[kx];
        p += g.W;
    }
    if (SUBSAMPLE) {
        const unsigned k = plane - g.divC.div(plane) * g.divC.d;
        out[o] = __fadd_rn(bias[k], __fmul_rn(weight[k], sum));
    } else {
        out[o] = __fadd_rn(0.0f, sum);
    }
}

// One thread per input pixel: gradients of the covering windows, window row then window column ascending.
template <bool SUBSAMPLE>
__global__ __launch_bounds__(256) void subsample_bwd_kernel(const float *__restrict__ gout, const float *__restrict__ weight,
                                                            float *__restrict__ gin, const SubGeom g, unsigned total) {
    const unsigned idx = blockIdx.x * 256u + threadIdx.x;
    if (idx >= total) return;
    unsigned plane, rem, h, w;
    g.divHW.divmod(idx, plane, rem);
    g.divW.divmod(rem, h, w);
    // windows i with i*dH <= h <= i*dH + kH - 1
    const int i_lo = (int)h >= g.kH ? (int)g.divDH.div(h - g.kH) + 1 : 0;
    int i_hi = (int)g.divDH.div(h);
    if (i_hi > g.Ho - 1) i_hi = g.Ho - 1;
    const int j_lo = (int)w >= g.kW ? (int)g.divDW.div(w - g.kW) + 1 : 0;
    int j_hi = (int)g.divDW.div(w);
    if (j_hi > g.Wo - 1) j_hi = g.Wo - 1;
    float wk = 1.0f;
    if (SUBSAMPLE) wk = weight[plane - g.divC.div(plane) * g.divC.d];
    const float *go = gout + (long)plane * g.Ho * g.Wo;
    float acc = 0.0f;
    for (int i = i_lo; i <= i_hi; ++i)
        for (int j = j_lo; j <= j_hi; ++j) {
            const float z = SUBSAMPLE ? __fmul_rn(go[i * g.Wo + j], wk) : go[i * g.Wo + j];
            acc = __fadd_rn(acc, z);
        }
    gin[idx] = acc;
}

// One workgroup per (image, plane): sum of gradOutput, and sum over windows of gradOutput * input.
__global__ __launch_bounds__(256) void subsample_accgrad_partial_kernel(const float *__restrict__ in,
                                                                        const float *__restrict__ gout,
                                                                        float *__restrict__ partial, const SubGeom g) {
    __shared__ float sb[256], sw[256];
    const unsigned plane = blockIdx.x;
    const float *ip = in + (long)plane * g.H * g.W;
    const float *go = gout + (long)plane * g.Ho * g.Wo;
    const unsigned n = (unsigned)(g.Ho * g.Wo);
    float s1 = 0.0f, s2 = 0.0f;
    for (unsigned o = threadIdx.x; o < n; o += 256u) {
        unsigned i, j;
        g.divWo.divmod(o, i, j);
        const float z = go[o];
        const float *p = ip + (long)i * g.dH * g.W + (long)j * g.dW;
        float t = 0.0f;
        for (int ky = 0; ky < g.kH; ++ky) {
            for (int kx = 0; kx < g.kW; ++kx) t = __fadd_rn(t, __fmul_rn(z, p[kx]));
            p += g.W;
        }
        s1 += z;
        s2 += t;
    }
    sb[threadIdx.x] = s1;
    sw[threadIdx.x] = s2;
    __syncthreads();
    for (unsigned s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) {
            sb[threadIdx.x] += sb[threadIdx.x + s];
            sw[threadIdx.x] += sw[threadIdx.x + s];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) {
        partial[2 * plane] = sb[0];
        partial[2 * plane + 1] = sw[0];
    }
}

// One thread per plane: the images one after another, as the CPU loop does.
__global__ __launch_bounds__(256) void subsample_accgrad_final_kernel(const float *__restrict__ partial,
                                                                      float *__restrict__ gradWeight,
                                                                      float *__restrict__ gradBias, int B, int C,
                                                                      float scale) {
    const int k = blockIdx.x * 256 + threadIdx.x;
    if (k >= C) return;
    float gb = gradBias[k], gw = gradWeight[k];
    for (int b = 0; b < B; ++b) {
        gb = __fadd_rn(gb, __fmul_rn(scale, partial[2 * ((long)b * C + k)]));
        gw = __fadd_rn(gw, __fmul_rn(scale, partial[2 * ((long)b * C + k) + 1]));
    }
    gradBias[k] = gb;
    gradWeight[k] = gw;
}

struct SubShape {
    long B, C;
    int H, W, Ho, Wo;
    bool batched;
};

// Argument checks with the reference's messages (SpatialSubSampling.c:34-48, SpatialAveragePooling.c:31-46).
int sub_shape(const char *name, SubShape &s, SubGeom &g, const THGPUTensor *input, int kW, int kH, int dW, int dH) {
    if (!input) return fail("%s: null tensor", name);
    if (!(input->nDimension == 3 || input->nDimension == 4)) return fail("3D or 4D(batch mode) tensor expected");
    if (kW <= 0 || kH <= 0 || dW <= 0 || dH <= 0) return fail("%s: invalid kernel/stride", name);
    s.batched = input->nDimension == 4;
    const int o = s.batched ? 1 : 0;
    s.B = s.batched ? input->size[0] : 1;
    s.C = input->size[o];
    s.H = (int)input->size[o + 1];
    s.W = (int)input->size[o + 2];
    if (!(s.W >= kW && s.H >= kH)) return fail("input image smaller than kernel size");
    s.Ho = (s.H - kH) / dH + 1;
    s.Wo = (s.W - kW) / dW + 1;
    if (s.B * s.C * (long)s.H * s.W >= (1L << 31)) return fail("%s: tensor too large for 32-bit indexing", name);
    g.H = s.H; g.W = s.W; g.kH = kH; g.kW = kW; g.dH = dH; g.dW = dW; g.Ho = s.Ho; g.Wo = s.Wo;
    g.divWo = FastDiv((uint32_t)s.Wo);
    g.divHoWo = FastDiv((uint32_t)(s.Ho * s.Wo));
    g.divW = FastDiv((uint32_t)s.W);
    g.divHW = FastDiv((uint32_t)(s.H * s.W));
    g.divC = FastDiv((uint32_t)(s.C > 0 ? s.C : 1));
    g.divDH = FastDiv((uint32_t)dH);
    g.divDW = FastDiv((uint32_t)dW);
    return 0;
}

int plane_vector(const char *name, const THGPUTensor *t, long C, const char *what) {
    if (!t) return fail("%s: null %s", name, what);
    if (THGPUTensor_nElement(t) != C || !THGPUTensor_isContiguous(t))
        return fail("%s: %s must be a contiguous vector of nInputPlane elements", name, what);
    return 0;
}

int forward(const char *name, bool subsample, THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
            THGPUTensor *output, int kW, int kH, int dW, int dH) {
    SubShape s;
    SubGeom g;
    if (!output) return fail("%s: null tensor", name);
    if (sub_shape(name, s, g, input, kW, kH, dW, dH)) return 1;
    if (subsample) {
        if (weight && THGPUTensor_nElement(weight) != s.C) return fail("invalid number of input planes");
        if (plane_vector(name, weight, s.C, "weight") || plane_vector(name, bias, s.C, "bias")) return 1;
    }
    hipStream_t st = stream();
    if (!st) return 1;
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    if (!in) return 1;
    if (s.batched) THGPUTensor_resize4d(output, s.B, s.C, s.Ho, s.Wo);
    else THGPUTensor_resize3d(output, s.C, s.Ho, s.Wo);
    const long total = s.B * s.C * s.Ho * s.Wo;
    int rc = 0;
    if (!tensor_ready(output, total))
        rc = fail("%s: could not size output", name);
    if (!rc && total > 0) {
        const char *family = subsample ? "subsample_fwd" : "avgpool_fwd";
        {
            LaunchScope scope(sub_label(family, g, s.B * s.C), 0.0, 4.0 * (s.B * s.C * (double)s.H * s.W + total));
            const dim3 grid((unsigned)((total + 255) / 256)), block(256);
            if (subsample)
                hipLaunchKernelGGL(subsample_fwd_kernel<true>, grid, block, 0, st, dptr(in), dptr(weight), dptr(bias),
                                   dptr(output), g, (unsigned)total);
            else
                hipLaunchKernelGGL(subsample_fwd_kernel<false>, grid, block, 0, st, dptr(in), nullptr, nullptr,
                                   dptr(output), g, (unsigned)total);
        }
        rc = check_launch(family);
    }
    THGPUTensor_free(in);
    return rc;
}

int check_grad_output(const char *name, const SubShape &s, const THGPUTensor *input, const THGPUTensor *gradOutput) {
    if (!gradOutput) return fail("%s: null tensor", name);
    const int o = s.batched ? 1 : 0;
    if (gradOutput->nDimension != input->nDimension || gradOutput->size[o] != s.C || gradOutput->size[o + 1] != s.Ho ||
        gradOutput->size[o + 2] != s.Wo || (s.batched && gradOutput->size[0] != s.B))
        return fail("%s: gradOutput size does not match the output size", name);
    return 0;
}

int backward(const char *name, bool subsample, THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
             THGPUTensor *gradInput, int kW, int kH, int dW, int dH) {
    SubShape s;
    SubGeom g;
    if (!gradInput) return fail("%s: null tensor", name);
    if (sub_shape(name, s, g, input, kW, kH, dW, dH)) return 1;
    if (check_grad_output(name, s, input, gradOutput)) return 1;
    if (subsample && plane_vector(name, weight, s.C, "weight")) return 1;
    hipStream_t st = stream();
    if (!st) return 1;
    THGPUTensor *go = THGPUTensor_newContiguous(gradOutput);
    if (!go) return 1;
    THGPUTensor_resizeAs(gradInput, input);
    const long total = s.B * s.C * (long)s.H * s.W;
    int rc = 0;
    if (!tensor_ready(gradInput, total))
        rc = fail("%s: could not size gradInput", name);
    if (!rc && total > 0) {
        const char *family = subsample ? "subsample_bwd" : "avgpool_bwd";
        {
            LaunchScope scope(sub_label(family, g, s.B * s.C), 0.0,
                              4.0 * ((double)total + s.B * s.C * (double)s.Ho * s.Wo));
            const dim3 grid((unsigned)((total + 255) / 256)), block(256);
            if (subsample)
                hipLaunchKernelGGL(subsample_bwd_kernel<true>, grid, block, 0, st, dptr(go), dptr(weight),
                                   dptr(gradInput), g, (unsigned)total);
            else
                hipLaunchKernelGGL(subsample_bwd_kernel<false>, grid, block, 0, st, dptr(go), nullptr, dptr(gradInput),
                                   g, (unsigned)total);
        }
        rc = check_launch(family);
    }
    THGPUTensor_free(go);
    return rc;
}

}  // namespace

extern "C" {

int thgpu_SpatialAveragePooling_updateOutput(THGPUTensor *input, THGPUTensor *output, int kW, int kH, int dW, int dH) {
    return forward("SpatialAveragePooling", false, input, nullptr, nullptr, output, kW, kH, dW, dH);
}

int thgpu_SpatialAveragePooling_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradInput,
                                                int kW, int kH, int dW, int dH) {
    return backward("SpatialAveragePooling", false, input, gradOutput, nullptr, gradInput, kW, kH, dW, dH);
}

int thgpu_SpatialSubSampling_updateOutput(THGPUTensor *input, THGPUTensor *weight, THGPUTensor *bias,
                                          THGPUTensor *output, int kW, int kH, int dW, int dH) {
    return forward("SpatialSubSampling", true, input, weight, bias, output, kW, kH, dW, dH);
}

int thgpu_SpatialSubSampling_updateGradInput(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *weight,
                                             THGPUTensor *gradInput, int kW, int kH, int dW, int dH) {
    return backward("SpatialSubSampling", true, input, gradOutput, weight, gradInput, kW, kH, dW, dH);
}

int thgpu_SpatialSubSampling_accGradParameters(THGPUTensor *input, THGPUTensor *gradOutput, THGPUTensor *gradWeight,
                                               THGPUTensor *gradBias, int kW, int kH, int dW, int dH, float scale) {
    const char *name = "SpatialSubSampling";
    SubShape s;
    SubGeom g;
    if (sub_shape(name, s, g, input, kW, kH, dW, dH)) return 1;
    if (check_grad_output(name, s, input, gradOutput)) return 1;
    if (plane_vector(name, gradWeight, s.C, "gradWeight") || plane_vector(name, gradBias, s.C, "gradBias")) return 1;
    if (s.C >= (1L << 31) || s.B >= (1L << 31)) return fail("%s: too many planes", name);
    hipStream_t st = stream();
    if (!st) return 1;
    const long planes = s.B * s.C;
    if (planes == 0) return 0;
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    if (!in) return 1;
    THGPUTensor *go = THGPUTensor_newContiguous(gradOutput);
    if (!go) {
        THGPUTensor_free(in);
        return 1;
    }
    int rc = 0;
    float *partial = workspace(sizeof(float) * 2 * (size_t)planes);
    if (!partial) rc = 1;
    if (!rc) {
        {
            LaunchScope scope(sub_label("subsample_accgrad", g, planes), 0.0,
                              4.0 * planes * ((double)s.H * s.W + (double)s.Ho * s.Wo));
            hipLaunchKernelGGL(subsample_accgrad_partial_kernel, dim3((unsigned)planes), dim3(256), 0, st, dptr(in),
                               dptr(go), partial, g);
        }
        rc = check_launch("subsample_accgrad");
    }
    if (!rc) {
        {
            LaunchScope scope("subsample_accgrad_final", 0.0, 4.0 * (2.0 * planes + 4.0 * s.C));
            hipLaunchKernelGGL(subsample_accgrad_final_kernel, dim3((unsigned)((s.C + 255) / 256)), dim3(256), 0, st,
                               partial, dptr(gradWeight), dptr(gradBias), (int)s.B, (int)s.C, scale);
        }
        rc = check_launch("subsample_accgrad_final");
    }
    THGPUTensor_free(in);
    THGPUTensor_free(go);
    return rc;
}

}  // extern "C"

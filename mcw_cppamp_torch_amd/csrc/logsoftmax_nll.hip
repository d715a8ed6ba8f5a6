// nn.LogSoftMax and nn.ClassNLLCriterion: the two modules that close a classifier stack.
//
// LogSoftMax follows the CPU module (mcw_nn/generic/LogSoftMax.c:37-53, 85-97), which is what the
// results are compared with: per frame, the maximum; logsum = max + log(sum of
// THExpMinusApprox(max - x)) accumulated in double, where THExpMinusApprox is the
// (1 + x/8 + x^2/128 + ...)^8 polynomial of mcw_torch7_core/lib/TH/THLogAdd.c:56-86 (exactly zero
// from x = 13 on), not exp; output = x - logsum.  Backward: gradInput = gradOutput -
// exp(output) * sum(gradOutput), sum and product in double.  (The reference GPU kernels,
// gpunn-impl/LogSoftMax.cpp:5-112, use float and the exact exponential; the reference's own test
// allows 1e-2 between the two, gpunn/test/test.lua:2149.)  A workgroup owns one frame; the double
// sums are tree reductions, so a result can differ from the CPU's sequential sum in the last bit of
// the double, which almost never reaches the float output.
//
// ClassNLLCriterion follows gpunn-impl/ClassNLLCriterion.cpp:9-92 (the only implementation for GPU
// tensors; mcw_nn/ClassNLLCriterion.lua:13-19,47-52 routes there when no class weights are given):
// output = -(sum over frames of input[i][target[i]-1]) [/ nframe], targets are 1-based class numbers
// stored as floats, a target below 1 is skipped; updateGradInput writes -1 [/ nframe] at the target
// positions of a gradInput the Lua module has already zeroed.
#include "common.h"

using namespace thgpu;

namespace {

inline float *dptr(const THGPUTensor *t) { return THGPUTensor_data(t); }

// exp(-x) for x >= 0 as mcw_torch7_core/lib/TH/THLogAdd.c:56-86 approximates it.
__device__ inline double exp_minus_approx(double x) {
    if (x < 13.0) {
        double y = 1.0 + x * (0.125 + x * (0.0078125 + x * (0.00032552083 + x * 1.0172526e-5)));
        y *= y;
        y *= y;
        y *= y;
        return 1.0 / y;
    }
    return 0.0;
}

template <typename T, typename Op>
__device__ inline T block_reduce(T v, T *scratch, Op op) {
    scratch[threadIdx.x] = v;
    __syncthreads();
    for (unsigned s = 128; s > 0; s >>= 1) {
        if (threadIdx.x < s) scratch[threadIdx.x] = op(scratch[threadIdx.x], scratch[threadIdx.x + s]);
        __syncthreads();
    }
    const T r = scratch[0];
    __syncthreads();
    return r;
}

__global__ __launch_bounds__(256) void logsoftmax_fwd_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                             long dim) {
    __shared__ double sd[256];
    __shared__ float sf[256];
    const float *x = in + (long)blockIdx.x * dim;
    float *y = out + (long)blockIdx.x * dim;
    float m = -INFINITY;
    for (long d = threadIdx.x; d < dim; d += 256) m = fmaxf(m, x[d]);
    m = block_reduce(m, sf, [](float a, float b) { return fmaxf(a, b); });
    double s = 0.0;
    for (long d = threadIdx.x; d < dim; d += 256) s += exp_minus_approx((double)(m - x[d]));
    s = block_reduce(s, sd, [](double a, double b) { return a + b; });
    const double logsum = (double)m + log(s);
    for (long d = threadIdx.x; d < dim; d += 256) y[d] = (float)((double)x[d] - logsum);
}

__global__ __launch_bounds__(256) void logsoftmax_bwd_kernel(const float *__restrict__ gout, const float *__restrict__ out,
                                                             float *__restrict__ gin, long dim) {
    __shared__ double sd[256];
    const float *go = gout + (long)blockIdx.x * dim;
    const float *y = out + (long)blockIdx.x * dim;
    float *gi = gin + (long)blockIdx.x * dim;
    double s = 0.0;
    for (long d = threadIdx.x; d < dim; d += 256) s += (double)go[d];
    s = block_reduce(s, sd, [](double a, double b) { return a + b; });
    for (long d = threadIdx.x; d < dim; d += 256) gi[d] = (float)((double)go[d] - exp((double)y[d]) * s);
}

// One workgroup: the sum over frames (and targets per frame) of input[i][target - 1].
__global__ __launch_bounds__(256) void nll_fwd_kernel(const float *__restrict__ in, const float *__restrict__ target,
                                                      float *__restrict__ out, long nframe, long ndim, long ntarget,
                                                      int size_average) {
    __shared__ double sd[256];
    double s = 0.0;
    for (long i = threadIdx.x; i < nframe; i += 256)
        for (long j = 0; j < ntarget; ++j) {
            const long t = (long)target[i * ntarget + j] - 1;
            if (t >= 0 && t < ndim) s += (double)in[i * ndim + t];
        }
    s = block_reduce(s, sd, [](double a, double b) { return a + b; });
    if (threadIdx.x == 0) {
        if (size_average) s /= (double)nframe;
        out[0] = (float)(-s);
    }
}

__global__ __launch_bounds__(256) void nll_bwd_kernel(const float *__restrict__ target, float *__restrict__ gin,
                                                      long nframe, long ndim, long ntarget, float grad) {
    const long i = (long)blockIdx.x * 256 + threadIdx.x;
    if (i >= nframe) return;
    for (long j = 0; j < ntarget; ++j) {
        const long t = (long)target[i * ntarget + j] - 1;
        if (t >= 0 && t < ndim) gin[i * ndim + t] = grad;
    }
}

// nframe x dim of a vector or matrix; 0 on success.
int frames(const THGPUTensor *t, long &nframe, long &dim) {
    if (t->nDimension == 1) {
        nframe = 1;
        dim = t->size[0];
    } else if (t->nDimension == 2) {
        nframe = t->size[0];
        dim = t->size[1];
    } else {
        return fail("vector or matrix expected");
    }
    return 0;
}

}  // namespace

extern "C" {

int thgpu_LogSoftMax_updateOutput(THGPUTensor *input, THGPUTensor *output) {
    if (!input || !output) return fail("LogSoftMax: null tensor");
    long nframe, dim;
    if (frames(input, nframe, dim)) return 1;
    if (nframe >= (1L << 31)) return fail("LogSoftMax: too many frames");
    hipStream_t st = stream();
    if (!st) return 1;
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    if (!in) return 1;
    THGPUTensor_resizeAs(output, in);
    int rc = 0;
    if (!tensor_ready(output, nframe * dim))
        rc = fail("LogSoftMax: could not size output");
    if (!rc && nframe * dim > 0) {
        {
            LaunchScope scope("logsoftmax_fwd", 0.0, 16.0 * nframe * dim);
            hipLaunchKernelGGL(logsoftmax_fwd_kernel, dim3((unsigned)nframe), dim3(256), 0, st, dptr(in), dptr(output),
                               dim);
        }
        rc = check_launch("logsoftmax_fwd");
    }
    THGPUTensor_free(in);
    return rc;
}

int thgpu_LogSoftMax_updateGradInput(THGPUTensor *gradOutput, THGPUTensor *output, THGPUTensor *gradInput) {
    if (!gradOutput || !output || !gradInput) return fail("LogSoftMax: null tensor");
    long nframe, dim;
    if (frames(output, nframe, dim)) return 1;
    if (nframe >= (1L << 31)) return fail("LogSoftMax: too many frames");
    if (THGPUTensor_nElement(gradOutput) != nframe * dim) return fail("LogSoftMax: gradOutput size does not match the output");
    hipStream_t st = stream();
    if (!st) return 1;
    THGPUTensor *out = THGPUTensor_newContiguous(output);
    if (!out) return 1;
    THGPUTensor *go = THGPUTensor_newContiguous(gradOutput);
    if (!go) {
        THGPUTensor_free(out);
        return 1;
    }
    THGPUTensor_resizeAs(gradInput, out);
    int rc = 0;
    if (!tensor_ready(gradInput, nframe * dim))
        rc = fail("LogSoftMax: could not size gradInput");
    if (!rc && nframe * dim > 0) {
        {
            LaunchScope scope("logsoftmax_bwd", 0.0, 16.0 * nframe * dim);
            hipLaunchKernelGGL(logsoftmax_bwd_kernel, dim3((unsigned)nframe), dim3(256), 0, st, dptr(go), dptr(out),
                               dptr(gradInput), dim);
        }
        rc = check_launch("logsoftmax_bwd");
    }
    THGPUTensor_free(out);
    THGPUTensor_free(go);
    return rc;
}

int thgpu_ClassNLLCriterion_updateOutput(THGPUTensor *input, THGPUTensor *target, THGPUTensor *outputTensor,
                                         int sizeAverage) {
    if (!input || !target || !outputTensor) return fail("ClassNLLCriterion: null tensor");
    long nframe, ndim;
    if (frames(input, nframe, ndim)) return 1;
    const long ntarget = target->nDimension > 1 ? target->size[1] : 1;
    if (THGPUTensor_nElement(target) != nframe * ntarget) return fail("ClassNLLCriterion: one target per frame expected");
    if (THGPUTensor_nElement(outputTensor) < 1 || !THGPUTensor_isContiguous(outputTensor))
        return fail("ClassNLLCriterion: outputTensor must hold one element");
    hipStream_t st = stream();
    if (!st) return 1;
    THGPUTensor *in = THGPUTensor_newContiguous(input);
    if (!in) return 1;
    THGPUTensor *tg = THGPUTensor_newContiguous(target);
    if (!tg) {
        THGPUTensor_free(in);
        return 1;
    }
    {
        LaunchScope scope("nll_fwd", 0.0, 8.0 * nframe * ntarget);
        // a vector input is one frame and is never averaged (ClassNLLCriterion.cpp:113-118)
        hipLaunchKernelGGL(nll_fwd_kernel, dim3(1), dim3(256), 0, st, dptr(in), dptr(tg), dptr(outputTensor), nframe,
                           ndim, ntarget, input->nDimension == 2 && sizeAverage ? 1 : 0);
    }
    const int rc = check_launch("nll_fwd");
    THGPUTensor_free(in);
    THGPUTensor_free(tg);
    return rc;
}

int thgpu_ClassNLLCriterion_updateGradInput(THGPUTensor *input, THGPUTensor *target, THGPUTensor *gradInput,
                                            int sizeAverage) {
    if (!input || !target || !gradInput) return fail("ClassNLLCriterion: null tensor");
    long nframe, ndim;
    if (frames(input, nframe, ndim)) return 1;
    const long ntarget = target->nDimension > 1 ? target->size[1] : 1;
    if (input->nDimension == 1 && ntarget > 1) return fail("multi-target not implemented");
    if (THGPUTensor_nElement(target) != nframe * ntarget) return fail("ClassNLLCriterion: one target per frame expected");
    if (!tensor_ready(gradInput, nframe * ndim))
        return fail("ClassNLLCriterion: gradInput must be contiguous and sized like the input");
    hipStream_t st = stream();
    if (!st) return 1;
    if (nframe == 0) return 0;
    THGPUTensor *tg = THGPUTensor_newContiguous(target);
    if (!tg) return 1;
    float grad = -1.0f;
    if (input->nDimension == 2 && sizeAverage) grad /= (float)nframe;
    {
        LaunchScope scope("nll_bwd", 0.0, 8.0 * nframe * ntarget);
        hipLaunchKernelGGL(nll_bwd_kernel, dim3((unsigned)((nframe + 255) / 256)), dim3(256), 0, st, dptr(tg),
                           dptr(gradInput), nframe, ndim, ntarget, grad);
    }
    const int rc = check_launch("nll_bwd");
    THGPUTensor_free(tg);
    return rc;
}

}  // extern "C"

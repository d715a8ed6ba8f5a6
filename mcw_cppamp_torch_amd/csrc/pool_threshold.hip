// nn.SpatialMaxPooling and nn.Threshold kernels.
//
// Max-pool forward: one lane per output element, lanes along the output row;
// the window is scanned ky ascending, kx ascending with a strict '>' from -inf,
// so the first maximum wins ties exactly as the CPU module's scan does
// (mcw_nn/generic/SpatialMaxPooling.c:30-45).  The two index planes hold
// ky+1 and kx+1 as floats (:51-52).
//
// Max-pool backward is index driven and atomics-free: one lane per input
// pixel visits the windows that cover it in (i ascending, j ascending) order
// and adds gradOutput where the saved argmax points back at the pixel.  This
// is the float addition order of the CPU module's scatter (:165-174), so
// overlapping windows give bit-identical sums, and no zero-fill pass is
// needed.  It replaces gpunn-impl/SpatialMaxPooling.cpp:87-203, which only
// handled non-overlapping windows.
#include "common.h"

#include <cmath>

namespace thgpu {

namespace {

struct PoolGeom {
    int H, W, Ho, Wo, kH, kW, dH, dW;
    FastDiv divWo, divHoWo, divW, divHW;
};

__global__ __launch_bounds__(256) void maxpool_fwd_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                          float *__restrict__ indy, float *__restrict__ indx,
                                                          const PoolGeom g, unsigned total) {
    unsigned o = blockIdx.x * blockDim.x + threadIdx.x;
    if (o >= total) return;
    unsigned plane, rem, i, j;
    g.divHoWo.divmod(o, plane, rem);
    g.divWo.divmod(rem, i, j);
    const float *win = in + ((long)plane * g.H + (long)i * g.dH) * g.W + (long)j * g.dW;
    float best = -INFINITY;
    int by = -1, bx = 0;
    for (int y = 0; y < g.kH; ++y) {
        for (int x = 0; x < g.kW; ++x) {
            float v = win[y * g.W + x];
            if (v > best) {
                best = v;
                by = y;
                bx = x;
            }
        }
    }
    out[o] = best;
    // A window of NaNs never updates the maximum; the CPU code then stores
    // (int)(-1 / kW) + 1 and (-1 % kW) + 1, i.e. (1, 0).
    indy[o] = by < 0 ? 1.0f : (float)(by + 1);
    indx[o] = by < 0 ? 0.0f : (float)(bx + 1);
}

__global__ __launch_bounds__(256) void maxpool_bwd_kernel(const float *__restrict__ gout,
                                                          const float *__restrict__ indy,
                                                          const float *__restrict__ indx, float *__restrict__ gin,
                                                          const PoolGeom g, unsigned total) {
    unsigned p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= total) return;
    unsigned plane, rem, h, w;
    g.divHW.divmod(p, plane, rem);
    g.divW.divmod(rem, h, w);
    // Windows (i, j) covering the pixel: i*dH <= h <= i*dH + kH - 1.
    int i_lo = (int)h - g.kH + 1;
    i_lo = i_lo <= 0 ? 0 : (i_lo + g.dH - 1) / g.dH;
    int i_hi = (int)h / g.dH;
    if (i_hi > g.Ho - 1) i_hi = g.Ho - 1;
    int j_lo = (int)w - g.kW + 1;
    j_lo = j_lo <= 0 ? 0 : (j_lo + g.dW - 1) / g.dW;
    int j_hi = (int)w / g.dW;
    if (j_hi > g.Wo - 1) j_hi = g.Wo - 1;
    const long obase = (long)plane * g.Ho * g.Wo;
    float acc = 0.0f;
    for (int i = i_lo; i <= i_hi; ++i) {
        const float wy = (float)((int)h - i * g.dH + 1);  // 1-based ky that would hit this row
        for (int j = j_lo; j <= j_hi; ++j) {
            long o = obase + (long)i * g.Wo + j;
            const float wx = (float)((int)w - j * g.dW + 1);
            if (indy[o] == wy && indx[o] == wx) acc += gout[o];
        }
    }
    gin[p] = acc;
}

__global__ __launch_bounds__(256) void threshold_fwd_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                            long n, float th, float val) {
    long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 3 < n) {
        float4 v = *reinterpret_cast<const float4 *>(in + i);
        v.x = v.x > th ? v.x : val;
        v.y = v.y > th ? v.y : val;
        v.z = v.z > th ? v.z : val;
        v.w = v.w > th ? v.w : val;
        *reinterpret_cast<float4 *>(out + i) = v;
    } else {
        for (; i < n; ++i) out[i] = in[i] > th ? in[i] : val;
    }
}

__global__ __launch_bounds__(256) void threshold_bwd_kernel(const float *__restrict__ in,
                                                            const float *__restrict__ gout, float *__restrict__ gin,
                                                            long n, float th) {
    long i = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 4;
    if (i + 3 < n) {
        float4 v = *reinterpret_cast<const float4 *>(in + i);
        float4 g = *reinterpret_cast<const float4 *>(gout + i);
        g.x = v.x > th ? g.x : 0.0f;
        g.y = v.y > th ? g.y : 0.0f;
        g.z = v.z > th ? g.z : 0.0f;
        g.w = v.w > th ? g.w : 0.0f;
        *reinterpret_cast<float4 *>(gin + i) = g;
    } else {
        for (; i < n; ++i) gin[i] = in[i] > th ? gout[i] : 0.0f;
    }
}

__global__ __launch_bounds__(256) void threshold_fwd_scalar(const float *__restrict__ in, float *__restrict__ out,
                                                            long n, float th, float val) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) out[i] = in[i] > th ? in[i] : val;
}

__global__ __launch_bounds__(256) void threshold_bwd_scalar(const float *__restrict__ in,
                                                            const float *__restrict__ gout, float *__restrict__ gin,
                                                            long n, float th) {
    long i = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) gin[i] = in[i] > th ? gout[i] : 0.0f;
}

// gradBias[m] += scale * sum over images and positions of gradOutput[b][m][n].
// One workgroup per output plane; fixed-shape tree, so reruns are identical.
__global__ __launch_bounds__(256) void gradbias_kernel(const float *__restrict__ gout, float *__restrict__ gbias,
                                                       int B, int M, int N, float scale) {
    const int m = blockIdx.x;
    float sum = 0.0f;
    for (int b = 0; b < B; ++b) {
        const float *row = gout + ((long)b * M + m) * N;
        for (int n = threadIdx.x; n < N; n += 256) sum += row[n];
    }
    __shared__ float red[256];
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) gbias[m] += scale * red[0];
}

}  // namespace

int maxpool_fwd_launch(const float *in, long planes, int H, int W, int kH, int kW, int dH, int dW, float *out,
                       float *indices) {
    hipStream_t s = stream();
    if (!s) return 1;
    PoolGeom g;
    g.H = H; g.W = W; g.kH = kH; g.kW = kW; g.dH = dH; g.dW = dW;
    g.Ho = (H - kH) / dH + 1;
    g.Wo = (W - kW) / dW + 1;
    long total = planes * g.Ho * g.Wo;
    if (total == 0) return 0;
    if (total >= (1L << 31) || planes * (long)H * W >= (1L << 31))
        return fail("SpatialMaxPooling: tensor too large for 32-bit indexing");
    g.divWo = FastDiv((uint32_t)g.Wo);
    g.divHoWo = FastDiv((uint32_t)(g.Ho * g.Wo));
    g.divW = FastDiv((uint32_t)W);
    g.divHW = FastDiv((uint32_t)(H * W));
    {
        LaunchScope scope("maxpool_fwd", 0.0, 4.0 * (planes * (double)H * W + 3.0 * total));
        hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, in, out,
                           indices, indices + total, g, (unsigned)total);
    }
    return check_launch("maxpool_fwd");
}

int maxpool_bwd_launch(const float *gout, const float *indices, long planes, int H, int W, int Ho, int Wo, int kH,
                       int kW, int dH, int dW, float *gin) {
    hipStream_t s = stream();
    if (!s) return 1;
    PoolGeom g;
    g.H = H; g.W = W; g.kH = kH; g.kW = kW; g.dH = dH; g.dW = dW; g.Ho = Ho; g.Wo = Wo;
    long total = planes * (long)H * W, ototal = planes * (long)Ho * Wo;
    if (total == 0) return 0;
    if (total >= (1L << 31)) return fail("SpatialMaxPooling: tensor too large for 32-bit indexing");
    g.divWo = FastDiv((uint32_t)(Wo > 0 ? Wo : 1));
    g.divHoWo = FastDiv((uint32_t)(Ho * Wo > 0 ? Ho * Wo : 1));
    g.divW = FastDiv((uint32_t)W);
    g.divHW = FastDiv((uint32_t)(H * W));
    {
        LaunchScope scope("maxpool_bwd", 0.0, 4.0 * ((double)total + 3.0 * ototal));
        hipLaunchKernelGGL(maxpool_bwd_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gout, indices,
                           indices + ototal, gin, g, (unsigned)total);
    }
    return check_launch("maxpool_bwd");
}

int threshold_fwd_launch(const float *in, float *out, long n, float th, float val) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (n == 0) return 0;
    const bool vec = (((uintptr_t)in | (uintptr_t)out) & 15) == 0;
    long threads = vec ? (n + 3) / 4 : n;
    long blocks = (threads + 255) / 256;
    if (blocks >= (1L << 31)) return fail("Threshold: tensor too large for one launch");
    {
        LaunchScope scope("threshold_fwd", 0.0, 8.0 * n);
        if (vec)
            hipLaunchKernelGGL(threshold_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, s, in, out, n, th, val);
        else
            hipLaunchKernelGGL(threshold_fwd_scalar, dim3((unsigned)blocks), dim3(256), 0, s, in, out, n, th, val);
    }
    return check_launch("threshold_fwd");
}

int threshold_bwd_launch(const float *in, const float *gout, float *gin, long n, float th) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (n == 0) return 0;
    const bool vec = (((uintptr_t)in | (uintptr_t)gout | (uintptr_t)gin) & 15) == 0;
    long threads = vec ? (n + 3) / 4 : n;
    long blocks = (threads + 255) / 256;
    if (blocks >= (1L << 31)) return fail("Threshold: tensor too large for one launch");
    {
        LaunchScope scope("threshold_bwd", 0.0, 12.0 * n);
        if (vec)
            hipLaunchKernelGGL(threshold_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, s, in, gout, gin, n, th);
        else
            hipLaunchKernelGGL(threshold_bwd_scalar, dim3((unsigned)blocks), dim3(256), 0, s, in, gout, gin, n, th);
    }
    return check_launch("threshold_bwd");
}

int gradbias_launch(const float *gout, float *gbias, long B, int M, long N, float scale) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (M == 0) return 0;
    if (B >= (1L << 31) || N >= (1L << 31)) return fail("gradBias: tensor too large");
    {
        LaunchScope scope("gradbias", 0.0, 4.0 * B * M * N);
        hipLaunchKernelGGL(gradbias_kernel, dim3((unsigned)M), dim3(256), 0, s, gout, gbias, (int)B, M, (int)N,
                           scale);
    }
    return check_launch("gradbias");
}

}  // namespace thgpu

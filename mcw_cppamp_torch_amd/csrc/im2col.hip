// Batched im2col and col2im for nn.SpatialConvolutionMM.
//
// Column buffer layout (the CPU module's finput, mcw_nn/generic/
// SpatialConvolutionMM.c:179): col[b][k][n], k = (c*kH + kh)*kW + kw,
// n = ho*Wo + wo; flat, the buffer is [B*C planes][kH*kW taps][Ho][Wo].
//
// im2col is store-bound (K*N floats out for C*H*W in), so the kernel is
// organised around the stores: the whole batch is one flat array and every
// lane owns four consecutive floats of it, written with one 16-byte store; a
// wavefront therefore covers 1 KiB of consecutive columns, i.e. a strip of
// output rows of one tap.  The input taps are gathered from L1/L2 (the image
// is re-read kH*kW/(sH*sW) times but stays cache resident).
//
// col2im is a gather with no atomics: one lane per image pixel adds the
// column entries that cover it, kh ascending then kw ascending from +0.0f --
// the float addition order of nn_(unfolded_acc) (mcw_nn/generic/
// SpatialConvolutionMM.c:6-50), which makes the result bit-identical to the
// CPU module's.  Lanes run along w, so for a fixed tap the reads are
// consecutive in wo.
#include "common.h"

namespace thgpu {

namespace {

struct ConvGeom {
    int C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo;
    FastDiv divN, divTaps, divKW, divWo;  // im2col decomposition
    FastDiv divW, divH;                   // col2im decomposition
};

__device__ inline float im2col_tap(const float *__restrict__ im, const ConvGeom &g, unsigned plane, unsigned tap,
                                   unsigned ho, unsigned wo) {
    unsigned kh, kw;
    g.divKW.divmod(tap, kh, kw);
    int iy = (int)ho * g.sH - g.pH + (int)kh;
    int ix = (int)wo * g.sW - g.pW + (int)kw;
    if (iy < 0 || iy >= g.H || ix < 0 || ix >= g.W) return 0.0f;
    return im[((long)plane * g.H + iy) * g.W + ix];
}

// total = number of floats in col; each thread writes elements [4t, 4t+4).
template <bool VEC>
__global__ __launch_bounds__(256) void im2col_kernel(const float *__restrict__ im, float *__restrict__ col,
                                                     const ConvGeom g, long total, long chunk_base) {
    long f = chunk_base + ((long)blockIdx.x * blockDim.x + threadIdx.x) * (VEC ? 4 : 1);
    if (f >= total) return;
    // f = row*N + n with row = plane*taps + tap; 32-bit magic division when the
    // whole buffer is below 2^31 floats (uniform branch), 64-bit otherwise.
    unsigned row, n;
    if (total < (1L << 31)) {
        g.divN.divmod((unsigned)f, row, n);
    } else {
        const long N = (long)g.Ho * g.Wo;
        long r64 = f / N;
        row = (unsigned)r64;
        n = (unsigned)(f - r64 * N);
    }
    unsigned plane, tap, ho, wo;
    g.divTaps.divmod(row, plane, tap);
    g.divWo.divmod(n, ho, wo);
    if (VEC) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            v[e] = (f + e < total) ? im2col_tap(im, g, plane, tap, ho, wo) : 0.0f;
            if (++wo == (unsigned)g.Wo) {
                wo = 0;
                if (++ho == (unsigned)g.Ho) {
                    ho = 0;
                    if (++tap == g.divTaps.d) {
                        tap = 0;
                        ++plane;
                    }
                }
            }
        }
        if (f + 3 < total) {
            *reinterpret_cast<float4 *>(col + f) = make_float4(v[0], v[1], v[2], v[3]);
        } else {
            for (int e = 0; e < 4 && f + e < total; ++e) col[f + e] = v[e];
        }
    } else {
        col[f] = im2col_tap(im, g, plane, tap, ho, wo);
    }
}

__global__ __launch_bounds__(256) void col2im_kernel(const float *__restrict__ col, float *__restrict__ im,
                                                     const ConvGeom g, long total) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    const long HW = (long)g.H * g.W;
    long plane = idx / HW;  // b*C + c
    unsigned pix = (unsigned)(idx - plane * HW), h, w;
    g.divW.divmod(pix, h, w);
    const long N = (long)g.Ho * g.Wo;
    const float *src = col + plane * (long)(g.kH * g.kW) * N;
    float acc = 0.0f;
    // Taps that can reach this pixel: kh == (h+pH) mod sH, stepping by sH.
    const int hp = (int)h + g.pH, wp = (int)w + g.pW;
    for (int kh = hp % g.sH; kh < g.kH; kh += g.sH) {
        int ho = (hp - kh) / g.sH;
        if (ho < 0) break;  // larger kh only lowers ho further
        if (ho >= g.Ho) continue;
        for (int kw = wp % g.sW; kw < g.kW; kw += g.sW) {
            int wo = (wp - kw) / g.sW;
            if (wo < 0) break;
            if (wo >= g.Wo) continue;
            acc += src[(long)(kh * g.kW + kw) * N + (long)ho * g.Wo + wo];
        }
    }
    im[idx] = acc;
}

int make_geom(ConvGeom &g, long B, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW) {
    if (B < 0 || C <= 0 || H <= 0 || W <= 0 || kH <= 0 || kW <= 0 || sH <= 0 || sW <= 0 || pH < 0 || pW < 0)
        return fail("im2col/col2im: invalid geometry");
    if (H + 2 * pH < kH || W + 2 * pW < kW) return fail("im2col/col2im: kernel larger than padded input");
    g.C = C; g.H = H; g.W = W; g.kH = kH; g.kW = kW; g.pH = pH; g.pW = pW; g.sH = sH; g.sW = sW;
    g.Ho = (H + 2 * pH - kH) / sH + 1;
    g.Wo = (W + 2 * pW - kW) / sW + 1;
    g.divN = FastDiv((uint32_t)(g.Ho * g.Wo));
    g.divTaps = FastDiv((uint32_t)(kH * kW));
    g.divKW = FastDiv((uint32_t)kW);
    g.divWo = FastDiv((uint32_t)g.Wo);
    g.divW = FastDiv((uint32_t)W);
    g.divH = FastDiv((uint32_t)H);
    if ((long)g.Ho * g.Wo >= (1L << 31) || (long)H * W >= (1L << 31) || B * C * (long)kH * kW >= (1L << 31))
        return fail("im2col/col2im: plane or row count exceeds 32-bit indexing");
    return 0;
}

}  // namespace

int im2col_launch(const float *im, long B, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW,
                  float *col) {
    ConvGeom g;
    if (make_geom(g, B, C, H, W, kH, kW, pH, pW, sH, sW)) return 1;
    hipStream_t s = stream();
    if (!s) return 1;
    const long N = (long)g.Ho * g.Wo;
    const long total = B * (long)C * kH * kW * N;
    if (total == 0) return 0;
    const bool vec = ((uintptr_t)col & 15) == 0;
    const long per_thread = vec ? 4 : 1;
    const long threads = (total + per_thread - 1) / per_thread;
    // At most 2^30 threads per launch keeps blockIdx.x*blockDim.x in range.
    const long max_threads = 1L << 30;
    for (long t0 = 0; t0 < threads; t0 += max_threads) {
        long nthr = threads - t0 < max_threads ? threads - t0 : max_threads;
        unsigned blocks = (unsigned)((nthr + 255) / 256);
        double bytes = 4.0 * ((double)B * C * H * W + (double)total) * ((double)nthr / threads);
        {
            LaunchScope scope("im2col", 0.0, bytes);
            if (vec)
                hipLaunchKernelGGL(im2col_kernel<true>, dim3(blocks), dim3(256), 0, s, im, col, g, total, t0 * 4);
            else
                hipLaunchKernelGGL(im2col_kernel<false>, dim3(blocks), dim3(256), 0, s, im, col, g, total, t0);
        }
        if (check_launch("im2col")) return 1;
    }
    return 0;
}

int col2im_launch(const float *col, long B, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW,
                  float *im) {
    ConvGeom g;
    if (make_geom(g, B, C, H, W, kH, kW, pH, pW, sH, sW)) return 1;
    hipStream_t s = stream();
    if (!s) return 1;
    const long total = B * (long)C * H * W;
    if (total == 0) return 0;
    const long blocks = (total + 255) / 256;
    if (blocks >= (1L << 31)) return fail("col2im: image batch too large for one launch");
    const double bytes = 4.0 * ((double)total + (double)B * C * kH * kW * g.Ho * g.Wo);
    {
        LaunchScope scope("col2im", 0.0, bytes);
        hipLaunchKernelGGL(col2im_kernel, dim3((unsigned)blocks), dim3(256), 0, s, col, im, g, total);
    }
    return check_launch("col2im");
}

}  // namespace thgpu

using namespace thgpu;

extern "C" {

int thgpu_im2col(const float *im, long B, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                 float *col) {
    return im2col_launch(im, B, C, H, W, kH, kW, padH, padW, sH, sW, col);
}

int thgpu_col2im(const float *col, long B, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                 float *im) {
    return col2im_launch(col, B, C, H, W, kH, kW, padH, padW, sH, sW, im);
}

}  // extern "C"

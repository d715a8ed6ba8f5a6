// Batched im2col and col2im for nn.SpatialConvolutionMM.
//
// Column buffer layout (the CPU module's finput, mcw_nn/generic/
// SpatialConvolutionMM.c:179): col[b][k][n], k = (c*kH + kh)*kW + kw,
// n = ho*Wo + wo; flat, the buffer is [B*C planes][kH*kW taps][Ho][Wo].
//
// im2col is store-bound (K*N floats out for C*H*W in), so both kernels are
// organised around the stores:
//   * unit horizontal stride: the batch of columns is one flat array, a lane
//     owns four consecutive floats of it and writes them with one aligned
//     128-bit store (a wavefront covers 1 KiB: a strip of output rows of one
//     tap); consecutive lanes read consecutive input pixels;
//   * strided: a wavefront takes a strip of output positions n of one
//     (plane, kh) pair, a lane owns one n and reads four consecutive taps at
//     once (one 128-bit load: consecutive lanes are sW floats apart, so the
//     wavefront reads a contiguous span) and writes one float to each of four
//     column rows.
// The input stays cache resident; HBM sees the image once and the columns once.
//
// col2im is a gather with no atomics: one lane per image pixel adds the
// column entries that cover it, kh ascending then kw ascending from +0.0f --
// the float addition order of nn_(unfolded_acc) (mcw_nn/generic/
// SpatialConvolutionMM.c:6-50), which makes the result bit-identical to the
// CPU module's.  Lanes run along w, so for a fixed tap the reads are
// consecutive in wo.  Candidate taps are visited in groups of four with
// clamped addresses and the invalid ones contribute +0.0f (which leaves a
// float sum unchanged), so the loads of a group are in flight together.
#include "common.h"

namespace thgpu {

namespace {

struct ConvGeom {
    int C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo, N;
    FastDiv divN, divKH, divWo, divTaps, divKW;  // im2col decomposition
    FastDiv divW, divHW, divSH, divSW;  // col2im decomposition
};

// Four floats at a 4-byte aligned address (the hardware handles the
// misalignment; the type only tells the compiler not to assume 16 bytes).
struct __attribute__((packed, aligned(4))) float4u {
    float x, y, z, w;
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

// Unit horizontal stride: the whole column buffer is one flat array and every
// lane owns four consecutive floats of it (one aligned 128-bit store; a
// wavefront writes 1 KiB of consecutive columns).  total = floats in col.
template <bool VEC>
__global__ __launch_bounds__(256) void im2col_flat_kernel(const float *__restrict__ im, float *__restrict__ col,
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

// Any stride.  Thread t: prow = t / N (= plane*kH + kh), n = t % N; four taps per step.
__global__ __launch_bounds__(256) void im2col_tapvec_kernel(const float *__restrict__ im, float *__restrict__ col,
                                                            const ConvGeom g, unsigned threads) {
    const unsigned t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= threads) return;
    unsigned prow, n, plane, kh, ho, wo;
    g.divN.divmod(t, prow, n);
    g.divKH.divmod(prow, plane, kh);
    g.divWo.divmod(n, ho, wo);
    const int iy = (int)ho * g.sH - g.pH + (int)kh;
    const bool row_ok = iy >= 0 && iy < g.H;
    const float *row = im + ((long)plane * g.H + (row_ok ? iy : 0)) * g.W;
    float *out = col + (long)prow * g.kW * g.N + n;
    int ix = (int)wo * g.sW - g.pW;
    for (int kw = 0; kw < g.kW; kw += 4, ix += 4, out += 4L * g.N) {
        float4u v;
        if (row_ok && ix >= 0 && ix + 3 < g.W) {
            v = *reinterpret_cast<const float4u *>(row + ix);
        } else {
            v.x = (row_ok && ix >= 0 && ix < g.W) ? row[ix] : 0.0f;
            v.y = (row_ok && ix + 1 >= 0 && ix + 1 < g.W) ? row[ix + 1] : 0.0f;
            v.z = (row_ok && ix + 2 >= 0 && ix + 2 < g.W) ? row[ix + 2] : 0.0f;
            v.w = (row_ok && ix + 3 >= 0 && ix + 3 < g.W) ? row[ix + 3] : 0.0f;
        }
        out[0] = v.x;
        if (kw + 1 < g.kW) out[g.N] = v.y;
        if (kw + 2 < g.kW) out[2L * g.N] = v.z;
        if (kw + 3 < g.kW) out[3L * g.N] = v.w;
    }
}

// One lane per image pixel; see the file comment for the order of additions.
__global__ __launch_bounds__(256) void col2im_kernel(const float *__restrict__ col, float *__restrict__ im,
                                                     const ConvGeom g, long total, int TH, int TW) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= total) return;
    unsigned plane, pix, h, w;
    if (total < (1L << 31)) {
        g.divHW.divmod((unsigned)idx, plane, pix);
    } else {
        const long HW = (long)g.H * g.W;
        long p64 = idx / HW;
        plane = (unsigned)p64;
        pix = (unsigned)(idx - p64 * HW);
    }
    g.divW.divmod(pix, h, w);
    const float *src = col + (long)plane * (g.kH * g.kW) * g.N;
    // Taps that can reach the pixel: kh = rh + th*sH with (h+pH) = qh*sH + rh
    // pairs with ho = qh - th; likewise kw = rw + tw*sW with wo = qw - tw.
    unsigned qh, rh, qw, rw;
    g.divSH.divmod(h + (unsigned)g.pH, qh, rh);
    g.divSW.divmod(w + (unsigned)g.pW, qw, rw);
    float acc = 0.0f;
    for (int th = 0; th < TH; ++th) {
        const int kh = (int)rh + th * g.sH, ho = (int)qh - th;
        const bool h_ok = kh < g.kH && ho >= 0 && ho < g.Ho;
        const int row_off = (kh * g.kW) * g.N + ho * g.Wo;
        for (int tw0 = 0; tw0 < TW; tw0 += 4) {
            float v[4];
            bool ok[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int tw = tw0 + u;
                const int kw = (int)rw + tw * g.sW, wo = (int)qw - tw;
                ok[u] = h_ok && tw < TW && kw < g.kW && wo >= 0 && wo < g.Wo;
                v[u] = src[ok[u] ? row_off + kw * g.N + wo : 0];
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) acc += ok[u] ? v[u] : 0.0f;
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
    if ((long)g.Ho * g.Wo >= (1L << 31)) return fail("im2col/col2im: output plane exceeds 32-bit indexing");
    g.N = g.Ho * g.Wo;
    g.divTaps = FastDiv((uint32_t)(kH * kW));
    g.divKW = FastDiv((uint32_t)kW);
    g.divN = FastDiv((uint32_t)g.N);
    g.divKH = FastDiv((uint32_t)kH);
    g.divWo = FastDiv((uint32_t)g.Wo);
    g.divW = FastDiv((uint32_t)W);
    g.divHW = FastDiv((uint32_t)(H * W));
    g.divSH = FastDiv((uint32_t)sH);
    g.divSW = FastDiv((uint32_t)sW);
    if ((long)g.Ho * g.Wo >= (1L << 31) || (long)H * W >= (1L << 31) || B * C * (long)kH * kW >= (1L << 31) ||
        (long)kH * kW * g.Ho * g.Wo >= (1L << 31))
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
    const long total = B * (long)C * kH * kW * g.N;
    if (total == 0) return 0;
    const double bytes = 4.0 * ((double)B * C * H * W + (double)total);
    if (sW == 1) {
        const bool vec = ((uintptr_t)col & 15) == 0;
        const long per_thread = vec ? 4 : 1;
        const long threads = (total + per_thread - 1) / per_thread;
        // At most 2^30 threads per launch keeps blockIdx.x*blockDim.x in range.
        const long max_threads = 1L << 30;
        for (long t0 = 0; t0 < threads; t0 += max_threads) {
            const long nthr = threads - t0 < max_threads ? threads - t0 : max_threads;
            const unsigned blocks = (unsigned)((nthr + 255) / 256);
            {
                LaunchScope scope("im2col", 0.0, bytes * ((double)nthr / threads));
                if (vec)
                    hipLaunchKernelGGL(im2col_flat_kernel<true>, dim3(blocks), dim3(256), 0, s, im, col, g, total,
                                       t0 * 4);
                else
                    hipLaunchKernelGGL(im2col_flat_kernel<false>, dim3(blocks), dim3(256), 0, s, im, col, g, total,
                                       t0);
            }
            if (check_launch("im2col")) return 1;
        }
        return 0;
    }
    const long prows = B * (long)C * kH;  // (plane, kh) pairs
    const long max_prows = ((1L << 31) - 256) / g.N / kH * kH;  // whole planes per launch
    if (max_prows < kH) return fail("im2col: column rows too long for one launch");
    for (long p0 = 0; p0 < prows; p0 += max_prows) {
        const long np = prows - p0 < max_prows ? prows - p0 : max_prows;
        const unsigned threads = (unsigned)(np * g.N);
        const unsigned blocks = (threads + 255) / 256;
        const float *im0 = im + (p0 / kH) * (long)H * W;
        float *col0 = col + p0 * (long)kW * g.N;
        {
            LaunchScope scope("im2col", 0.0, bytes * ((double)np / prows));
            hipLaunchKernelGGL(im2col_tapvec_kernel, dim3(blocks), dim3(256), 0, s, im0, col0, g, threads);
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
        hipLaunchKernelGGL(col2im_kernel, dim3((unsigned)blocks), dim3(256), 0, s, col, im, g, total,
                           (kH + sH - 1) / sH, (kW + sW - 1) / sW);
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

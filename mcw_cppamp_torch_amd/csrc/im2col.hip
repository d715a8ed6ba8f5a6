// Batched im2col and col2im for nn.SpatialConvolutionMM.
//
// Column buffer layout (the CPU module's finput, mcw_nn/generic/
// SpatialConvolutionMM.c:179): col[b][k][n], k = (c*kH + kh)*kW + kw,
// n = ho*Wo + wo; flat, the buffer is [B*C planes][kH*kW taps][Ho][Wo].
//
// im2col is store-bound (K*N floats out for C*H*W in).  Both kernels give a
// wavefront a strip of consecutive output positions n of one (plane, kh) pair
// and let it walk the kW taps, so the index arithmetic is paid once per strip
// and every store instruction writes consecutive floats of one column row:
//   * unit horizontal stride: a lane owns four consecutive n; per tap it reads
//     four consecutive input pixels (one 128-bit load when they share an output
//     row) and writes them with one 128-bit store;
//   * strided: a lane owns one n and reads four consecutive taps at once (one
//     128-bit load: consecutive lanes are sW floats apart, so the wavefront
//     reads a contiguous span), writing one float to each of four column rows.
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
    int G;                              // groups of four output positions per column row
    FastDiv divG, divN, divKH, divWo;   // im2col decomposition
    FastDiv divW, divHW, divSH, divSW;  // col2im decomposition
};

// Four floats at a 4-byte aligned address (the hardware handles the
// misalignment; the type only tells the compiler not to assume 16 bytes).
struct __attribute__((packed, aligned(4))) float4u {
    float x, y, z, w;
};

// Unit horizontal stride.  Thread t: prow = t / G (= plane*kH + kh), group = t % G.
__global__ __launch_bounds__(256) void im2col_nvec_kernel(const float *__restrict__ im, float *__restrict__ col,
                                                          const ConvGeom g, unsigned threads) {
    const unsigned t = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= threads) return;
    unsigned prow, gi, plane, kh, ho, wo;
    g.divG.divmod(t, prow, gi);
    g.divKH.divmod(prow, plane, kh);
    const int n0 = (int)gi * 4;
    g.divWo.divmod((unsigned)n0, ho, wo);
    const float *src = im + (long)plane * g.H * g.W;
    float *out = col + (long)prow * g.kW * g.N + n0;
    const bool full = n0 + 3 < g.N;
    if ((int)wo + 3 < g.Wo) {
        // The four outputs share an output row (and all exist).
        const int iy = (int)ho * g.sH - g.pH + (int)kh;
        const bool row_ok = iy >= 0 && iy < g.H;
        const float *row = src + (long)(row_ok ? iy : 0) * g.W;
        int ix = (int)wo - g.pW;
        for (int kw = 0; kw < g.kW; ++kw, ++ix, out += g.N) {
            float4u v;
            if (row_ok && ix >= 0 && ix + 3 < g.W) {
                v = *reinterpret_cast<const float4u *>(row + ix);
            } else {
                v.x = (row_ok && ix >= 0 && ix < g.W) ? row[ix] : 0.0f;
                v.y = (row_ok && ix + 1 >= 0 && ix + 1 < g.W) ? row[ix + 1] : 0.0f;
                v.z = (row_ok && ix + 2 >= 0 && ix + 2 < g.W) ? row[ix + 2] : 0.0f;
                v.w = (row_ok && ix + 3 >= 0 && ix + 3 < g.W) ? row[ix + 3] : 0.0f;
            }
            *reinterpret_cast<float4u *>(out) = v;
        }
        return;
    }
    // The group wraps to the next output row or runs past the end of the column row.
    int yy[4], xx[4];
    bool ok[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        ok[e] = n0 + e < g.N;
        yy[e] = (int)ho * g.sH - g.pH + (int)kh;
        xx[e] = (int)wo - g.pW;
        if (++wo == (unsigned)g.Wo) {
            wo = 0;
            ++ho;
        }
    }
    for (int kw = 0; kw < g.kW; ++kw, out += g.N) {
        float v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int x = xx[e] + kw;
            const bool in = ok[e] && yy[e] >= 0 && yy[e] < g.H && x >= 0 && x < g.W;
            v[e] = in ? src[(long)yy[e] * g.W + x] : 0.0f;
        }
        if (full) {
            float4u q;
            q.x = v[0]; q.y = v[1]; q.z = v[2]; q.w = v[3];
            *reinterpret_cast<float4u *>(out) = q;
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (ok[e]) out[e] = v[e];
        }
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
    g.G = (g.N + 3) / 4;
    g.divG = FastDiv((uint32_t)g.G);
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
    const long prows = B * (long)C * kH;  // (plane, kh) pairs
    if (prows == 0) return 0;
    const bool nvec = sW == 1;
    const long per_prow = nvec ? g.G : g.N;
    // The batch is cut into launches of at most 2^31 - 1 threads (whole prows each).
    const long max_prows = ((1L << 31) - 256) / per_prow / kH * kH;  // whole planes per launch
    if (max_prows < kH) return fail("im2col: column rows too long for one launch");
    const double bytes_per_prow = 4.0 * ((double)kW * g.N + (double)H * W / kH);
    for (long p0 = 0; p0 < prows; p0 += max_prows) {
        const long np = prows - p0 < max_prows ? prows - p0 : max_prows;
        const unsigned threads = (unsigned)(np * per_prow);
        const unsigned blocks = (threads + 255) / 256;
        const float *im0 = im + (p0 / kH) * (long)H * W;
        float *col0 = col + p0 * (long)kW * g.N;
        {
            LaunchScope scope("im2col", 0.0, bytes_per_prow * np);
            if (nvec)
                hipLaunchKernelGGL(im2col_nvec_kernel, dim3(blocks), dim3(256), 0, s, im0, col0, g, threads);
            else
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

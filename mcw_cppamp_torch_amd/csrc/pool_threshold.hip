// nn.SpatialMaxPooling and nn.Threshold kernels.
//
// Max-pool forward: one lane per output element, lanes along the output row;
// the window is scanned ky ascending, kx ascending with a strict '>' from -inf,
// so the first maximum wins ties exactly as the CPU module's scan does
// (mcw_nn/generic/SpatialMaxPooling.c:30-45).  The two index planes hold
// ky+1 and kx+1 as floats (:51-52).
//
// Max-pool backward is index driven and atomics-free: every input pixel visits
// the windows that cover it in (i ascending, j ascending) order and adds
// gradOutput where the saved argmax points back at the pixel.  This is the
// float addition order of the CPU module's scatter (:165-174), so overlapping
// windows give bit-identical sums, and no zero-fill pass is needed.  It
// replaces gpunn-impl/SpatialMaxPooling.cpp:87-203, which only handled
// non-overlapping windows.  A workgroup takes a strip of pixel rows of one
// plane (or several small planes), turns the windows that can reach it into
// (target pixel, gradient) pairs in LDS -- padded with pairs that target no
// pixel, so the pixel loop has no bounds to check -- and then each pixel
// compares at most ceil(kH/dH)*ceil(kW/dW) pairs against its own index.
#include "common.h"

#include <cmath>
#include <cstdlib>

namespace thgpu {

namespace {

struct PoolGeom {
    int H, W, Ho, Wo, kH, kW, dH, dW;
    FastDiv divWo, divHoWo, divW, divHW, divDH, divDW;
};

// Timing label: the kernel family alone, or with the geometry while per-kernel timing is on.
inline const char *pool_label(const char *family, const PoolGeom &g, long planes) {
    if (!prof_enabled()) return family;
    return prof_label("%s planes=%ld %dx%d k=%dx%d s=%dx%d", family, planes, g.H, g.W, g.kH, g.kW, g.dH, g.dW);
}

// KH, KW > 0 fix the window at compile time (fully unrolled: all loads of a
// window are in flight before the compare chain); 0 takes the run-time sizes.
template <int KH, int KW>
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
    if (KH > 0) {
        float v[KH > 0 ? KH : 1][KW > 0 ? KW : 1];
#pragma unroll
        for (int y = 0; y < KH; ++y)
#pragma unroll
            for (int x = 0; x < KW; ++x) v[y][x] = win[y * g.W + x];
#pragma unroll
        for (int y = 0; y < KH; ++y)
#pragma unroll
            for (int x = 0; x < KW; ++x)
                if (v[y][x] > best) {
                    best = v[y][x];
                    by = y;
                    bx = x;
                }
    } else {
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
    }
    out[o] = best;
    // A window of NaNs never updates the maximum; the CPU code then stores
    // (int)(-1 / kW) + 1 and (-1 % kW) + 1, i.e. (1, 0).
    indy[o] = by < 0 ? 1.0f : (float)(by + 1);
    indx[o] = by < 0 ? 0.0f : (float)(bx + 1);
}

// Launch shape of the LDS-tile backward kernel.
struct PoolBwdPlan {
    int G;      // planes per workgroup (more than one only when a strip is the whole plane)
    int PR;     // pixel rows per strip
    int tiles;  // strips per plane
    int RW;     // window rows kept per strip (with TH-1 rows of history)
    int CW;     // window columns kept per row (with TW-1 columns of history and the uncovered right edge)
    FastDiv divTiles, divEnt, divCW, divPix;
    FastDiv divW2, divPix2;  // pixel pairs (dW == 2): pairs per row, pairs per plane
};

// TH x TW = the most windows that can cover one pixel.  Pixel (h, w) can only
// be the argmax of windows (i_hi - a, j_hi - b), i_hi = h / dH, j_hi = w / dW,
// a < TH, b < TW; visiting a and b downwards is (i ascending, j ascending).
// PAIRS (horizontal stride 2): a lane takes the two pixels (h, 2k) and (h, 2k+1), which share j_hi = k and
// with it all their candidate windows, so each staged pair is read once for both.
template <int TH, int TW, bool PAIRS>
__global__ __launch_bounds__(256) void maxpool_bwd_tile_kernel(const float *__restrict__ gout,
                                                               const float *__restrict__ indy,
                                                               const float *__restrict__ indx,
                                                               float *__restrict__ gin, const PoolGeom g,
                                                               const PoolBwdPlan p, unsigned planes) {
    extern __shared__ int2 ent[];  // [G][RW][CW]: (target pixel inside the plane or -1, gradient bits)
    const int tid = threadIdx.x, nthr = blockDim.x;
    unsigned grp, strip;
    p.divTiles.divmod(blockIdx.x, grp, strip);
    const unsigned plane0 = grp * (unsigned)p.G;
    const int np = (int)(planes - plane0 < (unsigned)p.G ? planes - plane0 : (unsigned)p.G);
    const int h0 = (int)strip * p.PR;
    const int nh = g.H - h0 < p.PR ? g.H - h0 : p.PR;
    const int i_first = (int)g.divDH.div((unsigned)h0) - (TH - 1);
    const int per_plane = p.RW * p.CW;
    const int HoWo = g.Ho * g.Wo;

    // ---- windows -> (target, gradient) pairs ------------------------------------------------
    const int E = np * per_plane;
    for (int e0 = tid; e0 < E; e0 += 4 * nthr) {
        float vy[4], vx[4], vg[4];
        int wi[4], wj[4];
        bool ok[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int idx = e0 + u * nthr;
            unsigned pl, rem, rr, cc;
            p.divEnt.divmod((unsigned)(idx < E ? idx : 0), pl, rem);
            p.divCW.divmod(rem, rr, cc);
            wi[u] = i_first + (int)rr;
            wj[u] = (int)cc - (TW - 1);
            ok[u] = idx < E && wi[u] >= 0 && wi[u] < g.Ho && wj[u] >= 0 && wj[u] < g.Wo;
            const long o = (long)(plane0 + pl) * HoWo + (ok[u] ? wi[u] * g.Wo + wj[u] : 0);
            vy[u] = indy[o];
            vx[u] = indx[o];
            vg[u] = gout[o];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int idx = e0 + u * nthr;
            if (idx < E) {
                const int t = (wi[u] * g.dH + (int)vy[u] - 1) * g.W + wj[u] * g.dW + (int)vx[u] - 1;
                ent[idx] = make_int2(ok[u] ? t : -1, __float_as_int(vg[u]));
            }
        }
    }
    __syncthreads();

    // ---- pixels ----------------------------------------------------------------------------------
    if (PAIRS) {
        const int W2 = (g.W + 1) / 2;
        const int P2 = nh * W2;
        const int total2 = np * P2;
        for (int q = tid; q < total2; q += nthr) {
            unsigned pl = 0, r = (unsigned)q, hh, w2;
            if (p.G > 1) p.divPix2.divmod(r, pl, r);  // grouped planes are whole: P2 == H*W2
            p.divW2.divmod(r, hh, w2);
            const int h = h0 + (int)hh, w = 2 * (int)w2;
            const int i_hi = (int)g.divDH.div((unsigned)h), j_hi = (int)w2;
            const int2 *e = ent + (int)pl * per_plane + (i_hi - i_first) * p.CW + j_hi + (TW - 1);
            const int pix = h * g.W + w;
            float acc0 = 0.0f, acc1 = 0.0f;
#pragma unroll
            for (int a = TH - 1; a >= 0; --a)
#pragma unroll
                for (int b = TW - 1; b >= 0; --b) {
                    const int2 c = e[-a * p.CW - b];
                    acc0 += c.x == pix ? __int_as_float(c.y) : 0.0f;
                    acc1 += c.x == pix + 1 ? __int_as_float(c.y) : 0.0f;
                }
            float *out = gin + (long)(plane0 + pl) * g.H * g.W + pix;
            out[0] = acc0;
            if (w + 1 < g.W) out[1] = acc1;
        }
        return;
    }
    const int P = nh * g.W;
    const int total = np * P;
    for (int q = tid; q < total; q += nthr) {
        unsigned pl = 0, r = (unsigned)q, hh, w;
        if (p.G > 1) p.divPix.divmod(r, pl, r);  // grouped planes are whole: P == H*W
        g.divW.divmod(r, hh, w);
        const int h = h0 + (int)hh;
        const int i_hi = (int)g.divDH.div((unsigned)h), j_hi = (int)g.divDW.div(w);
        const int2 *e = ent + (int)pl * per_plane + (i_hi - i_first) * p.CW + j_hi + (TW - 1);
        const int pix = h * g.W + (int)w;
        float acc = 0.0f;
#pragma unroll
        for (int a = TH - 1; a >= 0; --a)
#pragma unroll
            for (int b = TW - 1; b >= 0; --b) {
                const int2 c = e[-a * p.CW - b];
                acc += c.x == pix ? __int_as_float(c.y) : 0.0f;
            }
        gin[(long)(plane0 + pl) * g.H * g.W + pix] = acc;
    }
}

// The most LDS the tile kernel may ask for.
constexpr long kPoolBwdLdsBytes = 32 * 1024;

// Strip shape of the tile kernel; false when one pixel row's windows do not fit in LDS.
bool plan_pool_bwd(const PoolGeom &g, long planes, int TH, int TW, PoolBwdPlan &p) {
    const int right = (g.W - 1) / g.dW - (g.Wo - 1);
    p.CW = g.Wo + (TW - 1) + (right > 0 ? right : 0);
    auto rows = [&](long PR) { return (PR + g.dH - 1) / g.dH + TH; };
    auto bytes = [&](long G, long PR) { return G * rows(PR) * (long)p.CW * 8; };
    if (bytes(1, 1) > kPoolBwdLdsBytes) return false;
    const long want = 2048;  // pixels per workgroup
    p.G = 1;
    if ((long)g.H * g.W <= want / 2 && bytes(1, g.H) <= kPoolBwdLdsBytes) {
        p.PR = g.H;
        long G = want / ((long)g.H * g.W);
        if (G > planes) G = planes;
        while (G > 1 && bytes(G, p.PR) > kPoolBwdLdsBytes) --G;
        p.G = (int)(G < 1 ? 1 : G);
    } else {
        long PR = want / g.W;
        if (PR < 1) PR = 1;
        if (PR > g.H) PR = g.H;
        while (PR > 1 && bytes(1, PR) > kPoolBwdLdsBytes) --PR;
        const long tiles = (g.H + PR - 1) / PR;
        p.PR = (int)((g.H + tiles - 1) / tiles);
    }
    p.tiles = (g.H + p.PR - 1) / p.PR;
    p.RW = (int)rows(p.PR);
    p.divTiles = FastDiv((uint32_t)p.tiles);
    p.divEnt = FastDiv((uint32_t)(p.RW * p.CW));
    p.divCW = FastDiv((uint32_t)p.CW);
    p.divPix = FastDiv((uint32_t)(g.H * g.W));
    p.divW2 = FastDiv((uint32_t)((g.W + 1) / 2));
    p.divPix2 = FastDiv((uint32_t)(g.H * ((g.W + 1) / 2)));
    return true;
}

// The direct kernel, for windows the tile kernel is not built for.
// TH x TW = the most windows that can cover one pixel (ceil(kH/dH) x ceil(kW/dW));
// candidates outside [lo, hi] are read at a clamped address and contribute +0.0f,
// so the loads of all candidates are in flight together.
template <int TH, int TW>
__global__ __launch_bounds__(256) void maxpool_bwd_kernel(const float *__restrict__ gout,
                                                          const float *__restrict__ indy,
                                                          const float *__restrict__ indx, float *__restrict__ gin,
                                                          const PoolGeom g, unsigned total, int th_rt, int tw_rt) {
    unsigned p = blockIdx.x * blockDim.x + threadIdx.x;
    if (p >= total) return;
    unsigned plane, rem, h, w;
    g.divHW.divmod(p, plane, rem);
    g.divW.divmod(rem, h, w);
    // Windows (i, j) covering the pixel: i*dH <= h <= i*dH + kH - 1, i.e.
    // i from ceil((h - kH + 1) / dH) (at least 0) to floor(h / dH) (at most Ho-1).
    const int ht = (int)h - g.kH + g.dH, wt = (int)w - g.kW + g.dW;  // numerators of the ceilings
    const int i_lo = ht <= 0 ? 0 : (int)g.divDH.div((unsigned)ht);
    const int j_lo = wt <= 0 ? 0 : (int)g.divDW.div((unsigned)wt);
    int i_hi = (int)g.divDH.div(h);
    if (i_hi > g.Ho - 1) i_hi = g.Ho - 1;
    int j_hi = (int)g.divDW.div(w);
    if (j_hi > g.Wo - 1) j_hi = g.Wo - 1;
    const float *go = gout + (long)plane * g.Ho * g.Wo;
    const float *iy = indy + (long)plane * g.Ho * g.Wo;
    const float *ix = indx + (long)plane * g.Ho * g.Wo;
    float acc = 0.0f;
    if (TH > 0) {
        float vy[TH > 0 ? TH : 1][TW > 0 ? TW : 1], vx[TH > 0 ? TH : 1][TW > 0 ? TW : 1],
            vg[TH > 0 ? TH : 1][TW > 0 ? TW : 1];
#pragma unroll
        for (int a = 0; a < TH; ++a)
#pragma unroll
            for (int b = 0; b < TW; ++b) {
                const int i = i_lo + a, j = j_lo + b;
                const int o = (i <= i_hi && j <= j_hi) ? i * g.Wo + j : 0;
                vy[a][b] = iy[o];
                vx[a][b] = ix[o];
                vg[a][b] = go[o];
            }
#pragma unroll
        for (int a = 0; a < TH; ++a)
#pragma unroll
            for (int b = 0; b < TW; ++b) {
                const int i = i_lo + a, j = j_lo + b;
                const float wy = (float)((int)h - i * g.dH + 1), wx = (float)((int)w - j * g.dW + 1);
                const bool hit = i <= i_hi && j <= j_hi && vy[a][b] == wy && vx[a][b] == wx;
                acc += hit ? vg[a][b] : 0.0f;
            }
    } else {
        (void)th_rt;
        (void)tw_rt;
        for (int i = i_lo; i <= i_hi; ++i) {
            const float wy = (float)((int)h - i * g.dH + 1);  // 1-based ky that would hit this row
            for (int j = j_lo; j <= j_hi; ++j) {
                const int o = i * g.Wo + j;
                const float wx = (float)((int)w - j * g.dW + 1);
                if (iy[o] == wy && ix[o] == wx) acc += go[o];
            }
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

// gradBias[m] += scale * sum over images and positions of gradOutput[b][m][n],
// in two fixed-shape stages so that reruns are bit-identical: stage 1 sums a
// slice of the batch per workgroup into part[m][slice], stage 2 adds the slices
// in order.
__global__ __launch_bounds__(256) void gradbias_partial_kernel(const float *__restrict__ gout,
                                                               float *__restrict__ part, int B, int M, int N,
                                                               int imgs_per_slice, int nslices, const FastDiv divN) {
    const int m = blockIdx.x, slice = blockIdx.y;
    const int b0 = slice * imgs_per_slice;
    const int b1 = b0 + imgs_per_slice < B ? b0 + imgs_per_slice : B;
    // The slice is (b1-b0) rows of N floats, M*N apart; lanes walk it as one
    // flat array, eight loads in flight each, whatever N is.
    const unsigned total = (unsigned)(b1 - b0) * (unsigned)N;
    const float *base = gout + ((long)b0 * M + m) * N;
    const long row_gap = (long)(M - 1) * N;  // from the end of one row to the start of the next
    float sum = 0.0f;
    for (unsigned f0 = threadIdx.x; f0 < total; f0 += 256 * 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const unsigned f = f0 + 256u * u;
            const unsigned row = divN.div(f < total ? f : 0);
            v[u] = f < total ? base[f + row * row_gap] : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += v[u];
    }
    __shared__ float red[256];
    red[threadIdx.x] = sum;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) red[threadIdx.x] += red[threadIdx.x + s];
        __syncthreads();
    }
    if (threadIdx.x == 0) part[(long)m * nslices + slice] = red[0];
}

__global__ __launch_bounds__(256) void gradbias_final_kernel(const float *__restrict__ part,
                                                             float *__restrict__ gbias, int M, int nslices,
                                                             float scale) {
    const int m = blockIdx.x * blockDim.x + threadIdx.x;
    if (m >= M) return;
    float sum = 0.0f;
    for (int s = 0; s < nslices; ++s) sum += part[(long)m * nslices + s];
    gbias[m] += scale * sum;
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
        LaunchScope scope(pool_label("maxpool_fwd", g, planes), 0.0, 4.0 * (planes * (double)H * W + 3.0 * total));
        const dim3 grid((unsigned)((total + 255) / 256)), block(256);
        if (kH == 3 && kW == 3)
            hipLaunchKernelGGL((maxpool_fwd_kernel<3, 3>), grid, block, 0, s, in, out, indices, indices + total, g,
                               (unsigned)total);
        else if (kH == 2 && kW == 2)
            hipLaunchKernelGGL((maxpool_fwd_kernel<2, 2>), grid, block, 0, s, in, out, indices, indices + total, g,
                               (unsigned)total);
        else
            hipLaunchKernelGGL((maxpool_fwd_kernel<0, 0>), grid, block, 0, s, in, out, indices, indices + total, g,
                               (unsigned)total);
    }
    return check_launch("maxpool_fwd");
}

// Host check of the backward tile planner: the window rows and columns a strip's pixels look up must
// lie inside the staged tile, which must fit its LDS budget.
long pool_plan_selftest() {
    long bad = 0;
    const int sizes[] = {2, 3, 6, 7, 12, 13, 14, 24, 27, 28, 55, 56, 112, 224, 231, 1000, 5000};
    for (int H : sizes)
        for (int W : sizes)
            for (int k = 1; k <= 4; ++k)
                for (int kw : {k, 2})  // square windows, and every height against a width of 2
                    for (int d = 1; d <= 4; ++d)
                        for (int dw : {d, 2}) {
                    // the tile kernel takes th == tw in {1, 2}, as the launcher requires
                    const int th = (k + d - 1) / d, tw = (kw + dw - 1) / dw;
                    if (H < k || W < kw || th != tw || !(th == 1 || th == 2)) continue;
                    PoolGeom g;
                    g.H = H; g.W = W; g.kH = k; g.kW = kw; g.dH = d; g.dW = dw;
                    g.Ho = (H - k) / d + 1;
                    g.Wo = (W - kw) / dw + 1;
                    for (long planes : {1L, 5L, 4096L}) {
                        PoolBwdPlan p;
                        if (!plan_pool_bwd(g, planes, th, tw, p)) continue;
                        bool ok = p.G >= 1 && p.G <= planes && p.PR >= 1 && p.PR <= H && (p.G == 1 || p.PR == H) &&
                                  (long)p.G * p.RW * p.CW * 8 <= kPoolBwdLdsBytes && (long)p.tiles * p.PR >= H &&
                                  (long)(p.tiles - 1) * p.PR < H && p.CW >= (W - 1) / dw + tw;
                        for (int t = 0; t < p.tiles && ok; ++t) {
                            const int h0 = t * p.PR, h1 = (h0 + p.PR < H ? h0 + p.PR : H) - 1;
                            const int i_first = h0 / d - (th - 1);
                            ok = h1 / d - i_first < p.RW;  // the last pixel row's newest window row
                        }
                        if (!ok) ++bad;
                    }
                }
    return bad;
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
    g.divDH = FastDiv((uint32_t)dH);
    g.divDW = FastDiv((uint32_t)dW);
    const int th = (kH + dH - 1) / dH, tw = (kW + dW - 1) / dW;
    const double bytes = 4.0 * ((double)total + 3.0 * ototal);
    PoolBwdPlan plan;
    // The pool_bwd_direct switch forces the direct kernel (a testing and tuning aid).
    if (!tuning().pool_bwd_direct && ((th == 2 && tw == 2) || (th == 1 && tw == 1)) &&
        plan_pool_bwd(g, planes, th, tw, plan)) {
        const long blocks = ((planes + plan.G - 1) / plan.G) * plan.tiles;
        if (blocks < (1L << 31)) {
            const size_t lds = sizeof(int2) * (size_t)plan.G * plan.RW * plan.CW;
            {
                LaunchScope scope(pool_label("maxpool_bwd", g, planes), 0.0, bytes);
                const dim3 grid((unsigned)blocks), block(256);
                float *ix = const_cast<float *>(indices) + ototal;
#define THGPU_POOL_BWD(TH_, TW_, PAIRS_)                                                                          \
    hipLaunchKernelGGL((maxpool_bwd_tile_kernel<TH_, TW_, PAIRS_>), grid, block, lds, s, gout, indices, ix, gin, g, \
                       plan, (unsigned)planes)
                if (th == 2 && dW == 2) THGPU_POOL_BWD(2, 2, true);
                else if (th == 2) THGPU_POOL_BWD(2, 2, false);
                else if (dW == 2) THGPU_POOL_BWD(1, 1, true);
                else THGPU_POOL_BWD(1, 1, false);
#undef THGPU_POOL_BWD
            }
            return check_launch("maxpool_bwd");
        }
    }
    {
        LaunchScope scope(pool_label("maxpool_bwd", g, planes), 0.0, bytes);
        const dim3 grid((unsigned)((total + 255) / 256)), block(256);
        if (th == 2 && tw == 2)
            hipLaunchKernelGGL((maxpool_bwd_kernel<2, 2>), grid, block, 0, s, gout, indices, indices + ototal, gin, g,
                               (unsigned)total, th, tw);
        else if (th == 1 && tw == 1)
            hipLaunchKernelGGL((maxpool_bwd_kernel<1, 1>), grid, block, 0, s, gout, indices, indices + ototal, gin, g,
                               (unsigned)total, th, tw);
        else
            hipLaunchKernelGGL((maxpool_bwd_kernel<0, 0>), grid, block, 0, s, gout, indices, indices + ototal, gin, g,
                               (unsigned)total, th, tw);
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
    if (M == 0 || N == 0 || B == 0) return 0;  // an empty sum leaves gradBias as it is
    if (B >= (1L << 31) || N >= (1L << 31) || B * N >= (1L << 32)) return fail("gradBias: tensor too large");
    // About four workgroups per CU in stage 1.
    long nslices = (4L * num_cus() + M - 1) / M;
    if (nslices > B) nslices = B;
    if (nslices > 65535) nslices = 65535;
    if (nslices < 1) nslices = 1;
    const int ips = (int)((B + nslices - 1) / nslices);
    nslices = (B + ips - 1) / ips;
    if (nslices < 1) nslices = 1;
    // The partial sums live behind the GEMM's split workspace, which the
    // gradWeight GEMM enqueued before has finished with (same stream).
    float *part = workspace(sizeof(float) * (size_t)M * nslices);
    if (!part) return 1;
    {
        LaunchScope scope("gradbias", 0.0, 4.0 * B * M * N);
        hipLaunchKernelGGL(gradbias_partial_kernel, dim3((unsigned)M, (unsigned)nslices), dim3(256), 0, s, gout,
                           part, (int)B, M, (int)N, ips, (int)nslices, FastDiv((uint32_t)N));
    }
    if (check_launch("gradbias")) return 1;
    {
        LaunchScope scope("gradbias_final", 0.0, 4.0 * M * (nslices + 2));
        hipLaunchKernelGGL(gradbias_final_kernel, dim3((unsigned)((M + 255) / 256)), dim3(256), 0, s, part, gbias,
                           M, (int)nslices, scale);
    }
    return check_launch("gradbias_final");
}

}  // namespace thgpu

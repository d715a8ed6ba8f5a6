// Batched im2col and col2im for nn.SpatialConvolutionMM.
//
// Column buffer layout (the CPU module's finput, mcw_nn/generic/
// SpatialConvolutionMM.c:179): col[b][k][n], k = (c*kH + kh)*kW + kw,
// n = ho*Wo + wo; flat, the buffer is [B*C planes][kH*kW taps][Ho][Wo].
//
// im2col is store-bound (K*N floats out for C*H*W in) and, at four cycles per
// wavefront instruction, easily instruction-bound as well, so every kernel
// spends only a few instructions per 64 floats written and builds addresses
// as a scalar (per tap) part plus a per-lane constant:
//   * unit strides, 3x3 (or 5x5) window known at compile time: a lane owns one
//     output position, requests its KH*KW input pixels at once and writes one
//     float into each column row (the wavefront: 256 consecutive bytes a row);
//   * other unit-stride layers: a workgroup copies the input rows of a strip
//     of output rows (or of several small planes) into LDS once, zero padding
//     included, and its lanes walk the taps with one LDS read and one store
//     per position and tap;
//   * strided layers, and rows too long for LDS: two direct kernels, a flat one
//     for unit horizontal stride (a lane owns four consecutive floats of the
//     column buffer) and one that reads four taps at a time.
// HBM sees the image once (plus halo rows between strips; neighbouring lanes
// share input through the caches) and the columns once.
//
// col2im is a gather with no atomics: one lane per image pixel adds the
// column entries that cover it, kh ascending then kw ascending from +0.0f --
// the float addition order of nn_(unfolded_acc) (mcw_nn/generic/
// SpatialConvolutionMM.c:6-50), which makes the result bit-identical to the
// CPU module's.  Lanes run along w, so for a fixed tap the reads are
// consecutive in wo.  Taps that do not reach a pixel contribute +0.0f (which
// leaves a float sum unchanged), so no add depends on a branch.  Unit-stride
// 3x3 and 5x5 layers have all their taps in flight per pixel; strided layers
// with wide rows walk the pixels by residue class of (h+pH, w+pW) modulo the
// strides, which makes every read a long contiguous run; the general kernel
// visits candidate taps in groups of four with clamped addresses.
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "common.h"
#include "kernels.h"

namespace thgpu {

namespace {

struct ConvGeom {
    int C, H, W, kH, kW, pH, pW, sH, sW, Ho, Wo, N;
    FastDiv divN, divKH, divWo, divTaps, divKW;  // im2col decomposition
    FastDiv divW, divHW, divSH, divSW, divH;  // col2im decomposition
};

// Timing label: the kernel family alone, or with the layer geometry while per-kernel timing is on.
inline const char *geom_label(const char *family, const ConvGeom &g, long B) {
    if (!prof_enabled()) return family;
    return prof_label("%s B=%ld C=%d %dx%d k=%dx%d s=%dx%d p=%dx%d", family, B, g.C, g.H, g.W, g.kH, g.kW, g.sH, g.sW, g.pH,
                      g.pW);
}

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

// Launch shape of the LDS-staged im2col.
struct StripPlan {
    int G;        // planes per workgroup (more than one only when a strip is the whole plane)
    int TR;       // output rows per strip
    int tiles;    // strips per plane
    int PL;       // lanes along the positions (multiple of 64)
    int TG;       // lane groups along the taps
    int LW;       // input columns kept per row: (Wo-1)*sW + kW
    int LH;       // input rows kept per strip: (TR-1)*sH + kH
    FastDiv divTiles, divLP, divLW;
};

// The LDS-staged kernel described at the top of the file.  NS = position slots per lane and pass.
template <int NS>
__global__ __launch_bounds__(256) void im2col_strip_kernel(const float *__restrict__ im, float *__restrict__ col,
                                                           const ConvGeom g, const StripPlan p, unsigned planes) {
    extern __shared__ float tile[];
    const int tid = threadIdx.x, nthr = blockDim.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6), nwaves = nthr >> 6;
    unsigned grp, strip;
    p.divTiles.divmod(blockIdx.x, grp, strip);
    const unsigned plane0 = grp * (unsigned)p.G;
    const int np = (int)(planes - plane0 < (unsigned)p.G ? planes - plane0 : (unsigned)p.G);
    const int r0 = (int)strip * p.TR;
    const int nr = g.Ho - r0 < p.TR ? g.Ho - r0 : p.TR;
    const int LP = p.LH * p.LW;

    // ---- stage the input rows -----------------------------------------------------------
    // tile[pl][r][c] is input pixel (r0*sH - pH + r, c - pW) of plane plane0+pl,
    // or zero outside the image.  Eight loads are in flight per lane before
    // the first is written to LDS.
    const int iy0 = r0 * g.sH - g.pH;
    if (p.LW >= 48 && p.LW <= 128) {
        // a wavefront takes whole rows: row number and source pointer are scalar, lanes run along the row
        const int rows = np * p.LH;
        for (int rb = wave; rb < rows; rb += 4 * nwaves) {
            float v[4][2];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int row = rb + u * nwaves;
                const int pl = row / p.LH, r = row - pl * p.LH;
                const int iy = iy0 + r;
                const bool row_ok = row < rows && iy >= 0 && iy < g.H;
                const float *src = im + ((long)(plane0 + pl) * g.H + (row_ok ? iy : 0)) * g.W - g.pW;
#pragma unroll
                for (int h = 0; h < 2; ++h) {
                    const int c = lane + 64 * h, ix = c - g.pW;
                    v[u][h] = (row_ok && c < p.LW && ix >= 0 && ix < g.W) ? src[c] : 0.0f;
                }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int row = rb + u * nwaves;
                if (row < rows) {
#pragma unroll
                    for (int h = 0; h < 2; ++h) {
                        const int c = lane + 64 * h;
                        if (c < p.LW) tile[row * p.LW + c] = v[u][h];
                    }
                }
            }
        }
    } else {
        // narrow or very wide rows: the tile as one flat array
        const int E = np * LP;
        for (int e0 = tid; e0 < E; e0 += nthr * 8) {
            float v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = e0 + u * nthr;
                unsigned pl, rem, r, c;
                p.divLP.divmod((unsigned)(idx < E ? idx : 0), pl, rem);
                p.divLW.divmod(rem, r, c);
                const int iy = iy0 + (int)r, ix = (int)c - g.pW;
                const bool ok = idx < E && iy >= 0 && iy < g.H && ix >= 0 && ix < g.W;
                v[u] = ok ? im[((long)(plane0 + pl) * g.H + iy) * g.W + ix] : 0.0f;
            }
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int idx = e0 + u * nthr;
                if (idx < E) tile[idx] = v[u];
            }
        }
    }
    __syncthreads();

    // ---- write the columns --------------------------------------------------------------
    // Positions of the workgroup: i = pl*Pn + n' over its planes and the strip's
    // Pn output positions.  A lane takes positions i = pi, pi + PL, ... (at
    // most four per pass) and keeps, for each, the LDS address of its tap
    // (0,0) and its byte offset from the column row of plane0 and tap 0.
    const int Pn = nr * g.Wo;
    const int total = np * Pn;
    const int pi = tid % p.PL;
    const int tg = __builtin_amdgcn_readfirstlane(tid / p.PL);  // PL is a multiple of 64: uniform
    const int taps = g.kH * g.kW;
    const long plane_floats = (long)taps * g.N;
    // scalar: start of (plane0, tap 0, first position of the strip)
    char *const row0 = reinterpret_cast<char *>(col + (long)plane0 * plane_floats + (long)r0 * g.Wo);
    for (int base = 0; base < total; base += NS * p.PL) {
        int lb[NS];
        unsigned voff[NS];
#pragma unroll
        for (int e = 0; e < NS; ++e) {
            // A lane past the end repeats the last position: the same value to the same address.
            int i = base + e * p.PL + pi;
            i = i < total ? i : total - 1;
            unsigned pl = 0, n = (unsigned)i, hr, wo;
            if (p.G > 1) g.divN.divmod(n, pl, n);  // grouped planes are whole: Pn == N
            g.divWo.divmod(n, hr, wo);
            lb[e] = ((int)pl * LP + (int)hr * g.sH * p.LW + (int)wo * g.sW) * 4;
            voff[e] = (unsigned)(((long)pl * plane_floats + n) * 4);
            asm volatile("" : "+v"(lb[e]), "+v"(voff[e]));  // keep both as single registers
        }
        int kh = tg / g.kW, kw = tg - kh * g.kW;
        for (int tap = tg; tap < taps; tap += p.TG) {
            const int loff = (kh * p.LW + kw) * 4;
            char *const row = row0 + (long)tap * g.N * 4;  // scalar
            float v[NS];
#pragma unroll
            for (int e = 0; e < NS; ++e)
                v[e] = *reinterpret_cast<const float *>(reinterpret_cast<const char *>(tile) + (lb[e] + loff));
#pragma unroll
            for (int e = 0; e < NS; ++e) *reinterpret_cast<float *>(row + voff[e]) = v[e];
            kw += p.TG;
            while (kw >= g.kW) {
                kw -= g.kW;
                ++kh;
            }
        }
    }
}

// Chooses the strip shape; false when even one output row's input rows exceed the LDS budget.
// A workgroup of PL*TG lanes runs ceil(positions/PL) slots (at most four, one
// pass) over ceil(taps/TG) taps; lanes past the strip's end repeat stores.
// Measured on gfx950 (strip-shape sweeps over the AlexNet/OverFeat/VGG layer
// geometries): three slots of a wide PL run best, planes of up to 1024
// positions are best taken whole, small planes are best grouped by few.
bool plan_strips(const ConvGeom &g, long planes, StripPlan &p) {
    constexpr long kLdsBytes = 32 * 1024;
    p.LW = (g.Wo - 1) * g.sW + g.kW;
    auto bytes = [&](long G, long TR) { return G * ((TR - 1) * g.sH + g.kH) * (long)p.LW * 4; };
    if (bytes(1, 1) > kLdsBytes) return false;
    const int taps = g.kH * g.kW;
    const bool grouped = g.N <= 256;                 // several whole planes per workgroup
    const bool whole = !grouped && g.N <= 1024 && bytes(1, g.Ho) <= kLdsBytes;  // one whole plane
    if (grouped && bytes(1, g.Ho) > kLdsBytes) return false;
    // The im2col_plan switch "v,PL,TG" pins the shape (a tuning aid): v = planes per group or rows per strip.
    const int fv = tuning().im2col_plan[0], fPL = tuning().im2col_plan[1], fTG = tuning().im2col_plan[2];
    long vmax = grouped ? 1024 / g.N : whole ? g.Ho : 1024 / g.Wo;
    if (grouped && vmax > planes) vmax = planes;
    if (!grouped && vmax > g.Ho) vmax = g.Ho;
    if (vmax < 1) vmax = 1;
    double best = -1;
    for (long v = whole ? g.Ho : 1; v <= vmax; ++v) {
        if (fv > 0 && v != (fv < vmax ? fv : vmax)) continue;
        const long G = grouped ? v : 1, TR = grouped ? g.Ho : v;
        if (bytes(G, TR) > kLdsBytes) break;
        if ((long)G * taps * g.N * 4 >= (1L << 32)) break;  // lane offsets are 32-bit
        if (!grouped && !whole && fv == 0) {
            const long tiles = (g.Ho + TR - 1) / TR;
            if (TR != (g.Ho + tiles - 1) / tiles) continue;  // only even strips
        }
        const long positions = grouped ? G * (long)g.N : TR * (long)g.Wo;
        for (int PL = 64; PL <= 256; PL += 64) {
            if (fPL > 0 && PL != fPL) continue;
            const long slots = (positions + PL - 1) / PL;
            if (slots > 4 && !(v == 1 && PL == 256)) continue;  // more than one pass only when unavoidable
            static const double kSlotWeight[5] = {0, 0.8, 0.9, 1.0, 0.95};
            double score = (double)positions / (double)(slots * PL) * (slots <= 4 ? kSlotWeight[slots] : 0.5);
            if (!grouped && PL < 256) score *= 0.9;          // strips: wide workgroups measured faster
            score += grouped ? -1e-4 * v : 0.0;              // ties: few planes per group
            if (score > best) {
                best = score;
                p.G = (int)G;
                p.TR = (int)TR;
                p.PL = PL;
            }
        }
    }
    if (best < 0) return false;
    p.TG = 1;
    double eff_best = 0;
    for (int tg = 1; tg <= 256 / p.PL; ++tg) {
        if (fTG > 0 && tg != (fTG < 256 / p.PL ? fTG : 256 / p.PL)) continue;
        const double eff = (double)taps / (tg * ((taps + tg - 1) / tg));
        if (eff >= eff_best) {
            eff_best = eff;
            p.TG = tg;
        }
    }
    p.tiles = (g.Ho + p.TR - 1) / p.TR;
    p.LH = (p.TR - 1) * g.sH + g.kH;
    p.divTiles = FastDiv((uint32_t)p.tiles);
    p.divLP = FastDiv((uint32_t)(p.LH * p.LW));
    p.divLW = FastDiv((uint32_t)p.LW);
    return true;
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
                                                     const ConvGeom g, long total, int TH, int TW,
                                                     const InputMask mask) {
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
    if (mask.in) acc = mask.in[idx] > mask.threshold ? acc : 0.0f;
    im[idx] = acc;
}

// im2col for unit strides and a window known at compile time: the mirror of
// col2im_unit_kernel below.  A lane owns one output position (plane, ho, wo),
// requests its KH*KW input pixels (neighbouring lanes share them through the
// vector cache), then writes one float to each of the KH*KW column rows at a
// per-tap scalar offset from a per-lane constant.
template <int KH, int KW>
__global__ __launch_bounds__(256) void im2col_unit_kernel(const float *__restrict__ im, float *__restrict__ col,
                                                          const ConvGeom g, unsigned total) {
    const unsigned q0 = blockIdx.x * 256u;  // scalar
    const unsigned q = q0 + threadIdx.x;
    const unsigned plane_first = g.divN.div(q0);
    unsigned plane, n, ho, wo;
    g.divN.divmod(q < total ? q : total - 1, plane, n);
    g.divWo.divmod(n, ho, wo);
    const int hi = (int)ho - g.pH, wi = (int)wo - g.pW;  // input pixel of tap (0, 0)
    const long in_plane = (long)g.H * g.W, out_plane = (long)(KH * KW) * g.N;
    const char *src = reinterpret_cast<const char *>(im + (long)plane_first * in_plane);
    char *dst = reinterpret_cast<char *>(col + (long)plane_first * out_plane);
    // 32-bit lane offsets; the input one may start before the plane (padding) but is only used where valid
    const long in_lane = (long)(plane - plane_first) * in_plane + (long)hi * g.W + wi;
    const unsigned out_off = (unsigned)(((long)(plane - plane_first) * out_plane + n) * 4);
    float v[KH][KW];
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) {
        const bool okh = (unsigned)(hi + kh) < (unsigned)g.H;
#pragma unroll
        for (int kw = 0; kw < KW; ++kw) {
            const bool ok = okh && (unsigned)(wi + kw) < (unsigned)g.W;
            v[kh][kw] = ok ? *reinterpret_cast<const float *>(src + (in_lane + (long)kh * g.W + kw) * 4) : 0.0f;
        }
    }
    if (q < total) {
#pragma unroll
        for (int kh = 0; kh < KH; ++kh)
#pragma unroll
            for (int kw = 0; kw < KW; ++kw)
                *reinterpret_cast<float *>(dst + (long)(kh * KW + kw) * g.N * 4 + out_off) = v[kh][kw];
    }
}

// col2im for unit strides and a window known at compile time.  With unit
// strides every tap can reach a pixel, and the column entry of tap (kh, kw) for
// pixel (h, w) sits at a per-tap scalar offset from a per-lane constant:
//   col[plane][kh*KW + kw][(h+pH-kh)*Wo + (w+pW-kw)]
//     = plane block + (tap*N - kh*Wo - kw)  +  ((h+pH)*Wo + (w+pW)).
// All KH*KW loads of a pixel are requested before the first add; the adds run
// kh ascending, kw ascending, out-of-range taps contributing +0.0f.
template <int KH, int KW>
__global__ __launch_bounds__(256) void col2im_unit_kernel(const float *__restrict__ col, float *__restrict__ im,
                                                          const ConvGeom g, unsigned total, const InputMask mask) {
    const unsigned q0 = blockIdx.x * 256u;  // scalar
    const unsigned q = q0 + threadIdx.x;
    const unsigned plane_first = g.divHW.div(q0);
    unsigned plane, pix, h, w;
    g.divHW.divmod(q < total ? q : total - 1, plane, pix);
    g.divW.divmod(pix, h, w);
    const int hp = (int)h + g.pH, wp = (int)w + g.pW;
    const long plane_floats = (long)(KH * KW) * g.N;
    const unsigned voff = (unsigned)(((long)(plane - plane_first) * plane_floats + (long)hp * g.Wo + wp) * 4);
    const char *base = reinterpret_cast<const char *>(col + (long)plane_first * plane_floats);
    float mv = 0.0f;
    if (mask.in) mv = mask.in[q < total ? q : total - 1];  // requested together with the taps
    float v[KH][KW];
#pragma unroll
    for (int kh = 0; kh < KH; ++kh) {
        const bool okh = (unsigned)(hp - kh) < (unsigned)g.Ho;
#pragma unroll
        for (int kw = 0; kw < KW; ++kw) {
            const bool ok = okh && (unsigned)(wp - kw) < (unsigned)g.Wo;
            const long tap_off = ((long)(kh * KW + kw) * g.N - (long)kh * g.Wo - kw) * 4;  // scalar, never negative
            v[kh][kw] = ok ? *reinterpret_cast<const float *>(base + tap_off + voff) : 0.0f;
        }
    }
    float acc = 0.0f;
#pragma unroll
    for (int kh = 0; kh < KH; ++kh)
#pragma unroll
        for (int kw = 0; kw < KW; ++kw) acc += v[kh][kw];
    if (mask.in) acc = mv > mask.threshold ? acc : 0.0f;
    if (q < total) im[q] = acc;
}

// col2im for strided convolutions with wide rows.  Write (h+pH, w+pW) =
// (qh*sH + rh, qw*sW + rw).  For one residue pair (rh, rw) the taps that reach
// a pixel are kh = rh + th*sH, kw = rw + tw*sW -- scalars -- and the column
// entry of tap (th, tw) for quotient pair (qh, qw) is
//   col[plane][kh*kW + kw][(qh-th)*Wo + (qw-tw)]
//     = scalar(plane, kh, kw, th, tw) + (qh*Wo + qw),
// a per-lane constant again, and lanes with consecutive (qh, qw) read
// consecutive column entries: the reads, nearly all of this kernel's traffic,
// are long contiguous runs.  A workgroup owns R quotient rows of one plane
// (R*sH image rows), one lane per (qh, qw) pair, walks the sH*sW residue pairs
// with all TH*TW taps of a pixel in flight (kh ascending, kw ascending, an
// unreachable tap contributing +0.0f), and collects the sums in an LDS copy of
// its image rows so that the image is written contiguously as well.
template <int TH, int TW>
__global__ __launch_bounds__(256) void col2im_strided_kernel(const float *__restrict__ col, float *__restrict__ im,
                                                             const ConvGeom g, int R, int Qw, int qtiles,
                                                             const FastDiv divQw, const FastDiv divTiles,
                                                             const InputMask mask) {
    extern __shared__ float rows[];  // [R*sH][W]
    unsigned plane, qt;
    divTiles.divmod(blockIdx.x, plane, qt);
    const int qh0 = (int)qt * R;
    const int h_base = qh0 * g.sH - g.pH;  // image row of the tile's first LDS row (may be negative)
    const float *src = col + (long)plane * (g.kH * g.kW) * g.N;
    for (int e = threadIdx.x; e < R * Qw; e += blockDim.x) {
        unsigned ql, qw;
        divQw.divmod((unsigned)e, ql, qw);
        const int qh = qh0 + (int)ql;
        const int lane_off = qh * g.Wo + (int)qw;
        for (int rh = 0; rh < g.sH; ++rh) {
            const int h = qh * g.sH + rh - g.pH;
            for (int rw = 0; rw < g.sW; ++rw) {
                const int w = (int)qw * g.sW + rw - g.pW;
                float v[TH][TW];
#pragma unroll
                for (int th = 0; th < TH; ++th) {
                    const int kh = rh + th * g.sH;
                    const bool okh = kh < g.kH && qh - th >= 0 && qh - th < g.Ho;
#pragma unroll
                    for (int tw = 0; tw < TW; ++tw) {
                        const int kw = rw + tw * g.sW;
                        const bool tap = kh < g.kH && kw < g.kW;  // scalar
                        const long tap_off = tap ? (long)(kh * g.kW + kw) * g.N - (long)th * g.Wo - tw : 0L;  // scalar
                        const bool ok = tap && okh && (int)qw - tw >= 0 && (int)qw - tw < g.Wo;
                        v[th][tw] = ok ? src[tap_off + lane_off] : 0.0f;
                    }
                }
                float acc = 0.0f;
#pragma unroll
                for (int th = 0; th < TH; ++th)
#pragma unroll
                    for (int tw = 0; tw < TW; ++tw) acc += v[th][tw];
                if (h >= 0 && h < g.H && w >= 0 && w < g.W) rows[(h - h_base) * g.W + w] = acc;
            }
        }
    }
    __syncthreads();
    // The tile's image rows [max(h_base, 0), min(h_base + R*sH, H)) are contiguous in the image.
    const int h_lo = h_base < 0 ? 0 : h_base;
    const int h_hi = h_base + R * g.sH < g.H ? h_base + R * g.sH : g.H;
    float *dst = im + ((long)plane * g.H + h_lo) * g.W;
    const float *from = rows + (h_lo - h_base) * g.W;
    if (mask.in) {
        const float *m = mask.in + (dst - im);
        for (int i = threadIdx.x; i < (h_hi - h_lo) * g.W; i += blockDim.x)
            dst[i] = m[i] > mask.threshold ? from[i] : 0.0f;
    } else {
        for (int i = threadIdx.x; i < (h_hi - h_lo) * g.W; i += blockDim.x) dst[i] = from[i];
    }
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
    g.divH = FastDiv((uint32_t)H);
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
    StripPlan plan;
    const long planes = B * (long)C;
    // Kernel choice.  Measured on gfx950: 3x3 unit-stride layers run fastest on the
    // per-position kernel, other unit-stride layers on the LDS-staged strips
    // (many column rows per workgroup favour its few, long stores), strided
    // first layers on the direct kernel.  The im2col_kernel switch (unit | strip | direct)
    // forces one where it applies (a testing and tuning aid).
    const char *force = tuning().im2col_kernel;
    const bool f_unit = !std::strcmp(force, "unit"), f_strip = !std::strcmp(force, "strip"),
               f_direct = !std::strcmp(force, "direct");
    const long span_out = 256 / (long)g.N + 2;  // planes one workgroup of the per-position kernel can touch
    const bool unit_ok = sH == 1 && sW == 1 && kH == kW && (kH == 3 || kH == 5) && planes * g.N < (1L << 32) &&
                         span_out * kH * kW * g.N * 4 < (1L << 32) && span_out * H * W * 4 < (1L << 31);
    if (unit_ok && !f_strip && !f_direct && (kH == 3 || f_unit)) {
        const long positions = planes * g.N;
        const unsigned blocks = (unsigned)((positions + 255) / 256);
        {
            LaunchScope scope(geom_label("im2col", g, B), 0.0, bytes);
            if (kH == 3)
                hipLaunchKernelGGL((im2col_unit_kernel<3, 3>), dim3(blocks), dim3(256), 0, s, im, col, g,
                                   (unsigned)positions);
            else
                hipLaunchKernelGGL((im2col_unit_kernel<5, 5>), dim3(blocks), dim3(256), 0, s, im, col, g,
                                   (unsigned)positions);
        }
        return check_launch("im2col");
    }
    if (!f_direct && (sW == 1 || f_strip) && plan_strips(g, planes, plan)) {
        const long groups = (planes + plan.G - 1) / plan.G;
        const long blocks = groups * plan.tiles;
        if (blocks < (1L << 31) && planes < (1L << 31)) {
            const size_t lds = sizeof(float) * (size_t)plan.G * plan.LH * plan.LW;
            {
                LaunchScope scope(geom_label("im2col", g, B), 0.0, bytes);
                const long positions = (long)plan.G * plan.TR * g.Wo;
                const long slots = (positions + plan.PL - 1) / plan.PL;
                const dim3 grid((unsigned)blocks), block(plan.PL * plan.TG);
                if (slots <= 1)
                    hipLaunchKernelGGL(im2col_strip_kernel<1>, grid, block, lds, s, im, col, g, plan, (unsigned)planes);
                else if (slots == 2)
                    hipLaunchKernelGGL(im2col_strip_kernel<2>, grid, block, lds, s, im, col, g, plan, (unsigned)planes);
                else if (slots == 3)
                    hipLaunchKernelGGL(im2col_strip_kernel<3>, grid, block, lds, s, im, col, g, plan, (unsigned)planes);
                else
                    hipLaunchKernelGGL(im2col_strip_kernel<4>, grid, block, lds, s, im, col, g, plan, (unsigned)planes);
            }
            return check_launch("im2col");
        }
    }
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
                LaunchScope scope(geom_label("im2col", g, B), 0.0, bytes * ((double)nthr / threads));
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
            LaunchScope scope(geom_label("im2col", g, B), 0.0, bytes * ((double)np / prows));
            hipLaunchKernelGGL(im2col_tapvec_kernel, dim3(blocks), dim3(256), 0, s, im0, col0, g, threads);
        }
        if (check_launch("im2col")) return 1;
    }
    return 0;
}

// Host check of the strip planner over a grid of geometries: every plan must keep the LDS tile within
// its budget, cover the plane exactly, and keep every LDS index of the kernel inside the tile.
long im2col_plan_selftest() {
    long bad = 0;
    const int sizes[] = {1, 2, 5, 6, 7, 12, 13, 14, 24, 27, 28, 55, 56, 57, 112, 224, 231, 300, 1000, 5000};
    const int kernels[] = {1, 2, 3, 5, 7, 11};
    const int strides[] = {1, 2, 4};
    for (int H : sizes)
        for (int W : sizes)
            for (int k : kernels)
                for (int kw : {k, 3})  // square kernels, and every height against a width of 3
                    for (int sH : strides)
                        for (int sW : strides)
                            for (int pad = 0; pad <= k / 2; pad += (k / 2 > 0 ? k / 2 : 1)) {
                        ConvGeom g;
                        const int padw = pad < kw ? pad : kw - 1;
                        if (H + 2 * pad < k || W + 2 * padw < kw) continue;
                        if (make_geom(g, 4, 3, H, W, k, kw, pad, padw, sH, sW)) continue;
                        for (long planes : {1L, 7L, 4096L}) {
                            StripPlan p;
                            if (!plan_strips(g, planes, p)) continue;
                            const long LP = (long)p.LH * p.LW;
                            const long positions = (long)p.G * p.TR * g.Wo;
                            const long slots = (positions + p.PL - 1) / p.PL;
                            bool ok = p.G >= 1 && p.TR >= 1 && p.TR <= g.Ho && (p.G == 1 || p.TR == g.Ho) &&
                                      p.G <= planes && p.G * LP * 4 <= 32 * 1024 &&
                                      p.LW == (g.Wo - 1) * g.sW + g.kW && p.LH == (p.TR - 1) * g.sH + g.kH &&
                                      p.PL % 64 == 0 && p.PL >= 64 && p.TG >= 1 && p.PL * p.TG <= 256 &&
                                      (slots <= 4 || p.PL == 256) && (long)p.tiles * p.TR >= g.Ho &&
                                      (long)(p.tiles - 1) * p.TR < g.Ho &&
                                      (long)p.G * g.kH * g.kW * g.N * 4 < (1L << 32);
                            // largest LDS index the column loop forms: last plane, last row and column, last tap
                            const long last = (p.G - 1) * LP + (long)(p.TR - 1) * g.sH * p.LW + (long)(g.Wo - 1) * g.sW +
                                              (long)(g.kH - 1) * p.LW + (g.kW - 1);
                            ok = ok && last < p.G * LP;
                            if (!ok) ++bad;
                        }
                    }
    return bad;
}

int col2im_launch(const float *col, long B, int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW,
                  float *im, InputMask mask) {
    ConvGeom g;
    if (make_geom(g, B, C, H, W, kH, kW, pH, pW, sH, sW)) return 1;
    hipStream_t s = stream();
    if (!s) return 1;
    const long total = B * (long)C * H * W;
    if (total == 0) return 0;
    const long blocks = (total + 255) / 256;
    if (blocks >= (1L << 31)) return fail("col2im: image batch too large for one launch");
    const double bytes = 4.0 * ((mask.in ? 2.0 : 1.0) * (double)total + (double)B * C * kH * kW * g.Ho * g.Wo);
    // Lane offsets of the unit-stride kernel are 32-bit: the planes one workgroup can touch must span < 4 GiB.
    const long span_planes = 256 / ((long)H * W) + 2;
    // The col2im_generic switch forces the general kernel (a testing and tuning aid).
    if (!tuning().col2im_generic && sH == 1 && sW == 1 && kH == kW && (kH == 3 || kH == 5) &&
        span_planes * kH * kW * g.N * 4 < (1L << 32) && total < (1L << 32)) {
        {
            LaunchScope scope(geom_label("col2im", g, B), 0.0, bytes);
            if (kH == 3)
                hipLaunchKernelGGL((col2im_unit_kernel<3, 3>), dim3((unsigned)blocks), dim3(256), 0, s, col, im, g,
                                   (unsigned)total, mask);
            else
                hipLaunchKernelGGL((col2im_unit_kernel<5, 5>), dim3((unsigned)blocks), dim3(256), 0, s, col, im, g,
                                   (unsigned)total, mask);
        }
        return check_launch("col2im");
    }
    const int th = (kH + sH - 1) / sH, tw = (kW + sW - 1) / sW;
    const int Qh = (H - 1 + pH) / sH + 1, Qw = (W - 1 + pW) / sW + 1;  // quotient ranges of (h+pH)/sH, (w+pW)/sW
    if (!tuning().col2im_generic && (sW > 1 || sH > 1) && W >= 64 && th <= 3 && tw <= 3) {
        // R quotient rows per workgroup: about 256 (qh, qw) pairs, image rows within the LDS budget
        int R = 256 / Qw;
        if (R < 1) R = 1;
        if (R > Qh) R = Qh;
        while (R > 1 && (long)R * sH * W * 4 > 48 * 1024) --R;
        const int qtiles = (Qh + R - 1) / R;
        const long wgs = B * (long)C * qtiles;
        if ((long)R * sH * W * 4 <= 48 * 1024 && wgs < (1L << 31)) {
            const size_t lds = sizeof(float) * (size_t)R * sH * W;
            const int lanes = (R * Qw + 63) / 64 * 64;
            const dim3 grid((unsigned)wgs), block(lanes < 256 ? lanes : 256);
            {
                LaunchScope scope(geom_label("col2im", g, B), 0.0, bytes);
                if (th == 3 || tw == 3)
                    hipLaunchKernelGGL((col2im_strided_kernel<3, 3>), grid, block, lds, s, col, im, g, R, Qw, qtiles,
                                       FastDiv((uint32_t)Qw), FastDiv((uint32_t)qtiles), mask);
                else
                    hipLaunchKernelGGL((col2im_strided_kernel<2, 2>), grid, block, lds, s, col, im, g, R, Qw, qtiles,
                                       FastDiv((uint32_t)Qw), FastDiv((uint32_t)qtiles), mask);
            }
            return check_launch("col2im");
        }
    }
    {
        LaunchScope scope(geom_label("col2im", g, B), 0.0, bytes);
        hipLaunchKernelGGL(col2im_kernel, dim3((unsigned)blocks), dim3(256), 0, s, col, im, g, total,
                           (kH + sH - 1) / sH, (kW + sW - 1) / sW, mask);
    }
    return check_launch("col2im");
}

}  // namespace thgpu

using namespace thgpu;

extern "C" {

int thgpu_im2col(const float *im, long B, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                 float *col) {
    // a null operand with a valid geometry would reach a launch and fault there
    if (!im || !col) return fail("thgpu_im2col: null operand");
    return im2col_launch(im, B, C, H, W, kH, kW, padH, padW, sH, sW, col);
}

int thgpu_col2im(const float *col, long B, int C, int H, int W, int kH, int kW, int padH, int padW, int sH, int sW,
                 float *im) {
    if (!im || !col) return fail("thgpu_col2im: null operand");
    return col2im_launch(col, B, C, H, W, kH, kW, padH, padW, sH, sW, im, InputMask());
}

}  // extern "C"

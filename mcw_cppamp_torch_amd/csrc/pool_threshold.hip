// nn.SpatialMaxPooling and nn.Threshold kernels.
//
// Max-pool forward, wavefront-level formulation (maxpool_fwd_tile_kernel; the default is the direct kernel, see
// there): a workgroup stages a group of small planes (or a strip of rows of a large one) in
// LDS with one contiguous, coalesced read -- every input row leaves memory once -- and its wavefronts
// then take output rows one at a time with their lanes along the INPUT columns: a lane reduces its
// column over the window rows (ky ascending, strict '>' from -inf, so the smallest ky wins a tie), and
// output lane j combines the kW columns j*dW + kx through cross-lane reads, keeping the larger value
// and, between equal values, the smaller (ky, kx) pair.  That is the first maximum of the CPU module's
// row-major strict-'>' scan (mcw_nn/generic/SpatialMaxPooling.c:30-45).  Planes narrower than half a
// wavefront are packed side by side.  The two index planes hold ky+1 and kx+1 as floats (:51-52).
//
// Max-pool backward is an index-driven scatter without atomics and without a zero-fill pass over
// memory: a workgroup owns the pixels of a group of planes (or a strip of rows) as a zeroed LDS tile,
// reads the windows that can reach them once (contiguous reads of the three window arrays), and adds
// each gradient at the pixel its saved argmax names.  The adds happen in ceil(kH/dH)*ceil(kW/dW)
// phases: a window whose argmax is pixel (h, w) belongs to phase (h/dH - i, w/dW - j), phases run with
// both differences descending, and inside one phase no two windows name the same pixel -- so every
// pixel receives its gradients in (i ascending, j ascending) order, the float addition order of the
// CPU module's scatter (:165-174), and overlapping windows give bit-identical sums.  It replaces
// gpunn-impl/SpatialMaxPooling.cpp:87-203, which only handled non-overlapping windows.  The tile is
// written out as one contiguous stream; the backward of a Threshold in front of the pooling layer can
// be applied on the way (InputMask).
#include "common.h"
#include "kernels.h"
#include "side_jobs.h"

#include <cmath>

namespace thgpu {

namespace {

struct PoolGeom {
    int H, W, Ho, Wo, kH, kW, dH, dW;
    long oplane;  // floats between the forward output's planes and rows (Ho*Wo and Wo when densely packed)
    int opitch;
    FastDiv divWo, divHoWo, divW, divHW, divDH, divDW;
};

// Timing label: the kernel family alone, or with the geometry while per-kernel timing is on.
inline const char *pool_label(const char *family, const PoolGeom &g, long planes) {
    if (!prof_enabled()) return family;
    return prof_label("%s planes=%ld %dx%d k=%dx%d s=%dx%d", family, planes, g.H, g.W, g.kH, g.kW, g.dH, g.dW);
}

// ---- forward ---------------------------------------------------------------------------------------

// The direct kernel: one lane per output element, lanes along the output row, scanning its own window in
// global memory (neighbouring lanes share the rows through the vector cache).  KH, KW > 0 fix the window at
// compile time (fully unrolled: all loads of a window are in flight before the compare chain); 0 takes the
// run-time sizes.  Measured on gfx950 this is the fastest forward kernel on every geometry of the benchmark
// stacks (at 13x13 .. 55x55 planes a launch lasts 10-35 us and is bound by its ramp-up, not by traffic), so it
// is the default; the tile kernel below is the wavefront-level formulation, kept behind the pool_fwd_wave switch.
template <int KH, int KW>
__global__ __launch_bounds__(256) void maxpool_fwd_direct_kernel(const float *__restrict__ in, float *__restrict__ out,
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
    out[(long)plane * g.oplane + (long)i * g.opitch + j] = best;
    // A window of NaNs never updates the maximum; the CPU code then stores
    // (int)(-1 / kW) + 1 and (-1 % kW) + 1, i.e. (1, 0).
    indy[o] = by < 0 ? 1.0f : (float)(by + 1);
    indx[o] = by < 0 ? 0.0f : (float)(bx + 1);
}

// Launch shape of the forward tile kernel.
struct PoolFwdPlan {
    int G;       // planes per workgroup (more than one only when a strip is the whole plane)
    int SR;      // output rows per strip
    int strips;  // strips per plane
    int P;       // planes (or row items) a wavefront takes side by side: 64 / W when the row fits twice
    int CO;      // outputs per column chunk: a wavefront covers (CO-1)*dW + kW input columns
    int chunks;  // column chunks per output row
    FastDiv divStrips, divItemRows, divChunks, divLaneW;
};

// The wavefront-level argmax described at the top of the file.  KH, KW, DH, DW > 0 fix the window at compile time;
// 0 takes the run-time values.
template <int KH, int KW, int DH, int DW>
__global__ __launch_bounds__(256) void maxpool_fwd_tile_kernel(const float *__restrict__ in, float *__restrict__ out,
                                                               float *__restrict__ indy, float *__restrict__ indx,
                                                               const PoolGeom g, const PoolFwdPlan p, unsigned planes) {
    extern __shared__ float tile[];  // [np][nh][W]: the staged input rows, then [3][np][ni][Wo]: the results
    const int kH = KH > 0 ? KH : g.kH, kW = KW > 0 ? KW : g.kW, dH = DH > 0 ? DH : g.dH, dW = DW > 0 ? DW : g.dW;
    const int tid = threadIdx.x;
    unsigned grp, strip;
    p.divStrips.divmod(blockIdx.x, grp, strip);
    const unsigned plane0 = grp * (unsigned)p.G;
    const int np = (int)(planes - plane0 < (unsigned)p.G ? planes - plane0 : (unsigned)p.G);
    const int i0 = (int)strip * p.SR;
    const int ni = g.Ho - i0 < p.SR ? g.Ho - i0 : p.SR;  // output rows of this strip
    const int h0 = i0 * dH;
    const int nh = p.G > 1 ? g.H : (ni - 1) * dH + kH;   // grouped planes are staged whole
    const int rows_w = nh * g.W;
    // results of the strip: values, ky+1, kx+1, each [np][ni][Wo], behind the staged rows
    const int nout = np * ni * g.Wo;
    float *res = tile + ((p.G * (p.G > 1 ? g.H : (p.SR - 1) * dH + kH) * g.W + 3) & ~3);

    // ---- stage: one contiguous range (grouped planes lie back to back; a strip is a run of whole rows) ----
    {
        const float *src = in + (long)plane0 * g.H * g.W + (p.G > 1 ? 0 : (long)h0 * g.W);
        const int n = np * rows_w;
        // 128-bit reads from the first 16-byte boundary on; single floats before it and at the end
        const int head = (int)(((16u - (unsigned)(reinterpret_cast<uintptr_t>(src) & 15u)) & 15u) >> 2);
        const int lead = head < n ? head : n;
        if (tid < lead) tile[tid] = src[tid];
        const int nv = (n - lead) >> 2;
        const float4 *src4 = reinterpret_cast<const float4 *>(src + lead);
        for (int q0 = tid; q0 < nv; q0 += 4 * 256) {
            float4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (q0 + u * 256 < nv) v[u] = src4[q0 + u * 256];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (q0 + u * 256 < nv) {
                    const int e = lead + 4 * (q0 + u * 256);
                    tile[e] = v[u].x;
                    tile[e + 1] = v[u].y;
                    tile[e + 2] = v[u].z;
                    tile[e + 3] = v[u].w;
                }
        }
        const int done = lead + 4 * nv;
        if (tid < n - done) tile[done + tid] = src[done + tid];
    }
    __syncthreads();

    // ---- wavefronts take (plane, output row, column chunk) items, P of them side by side ----------------------
    const int lane = tid & 63, wave = tid >> 6;
    unsigned sub, c;
    p.divLaneW.divmod((unsigned)lane, sub, c);  // lane -> (which of the P items, input column inside the chunk)
    const int span = (p.CO - 1) * dW + kW;      // input columns a chunk covers
    const int items = np * ni * p.chunks;
    for (int it0 = wave * p.P; it0 < items; it0 += 4 * p.P) {
        const int it = it0 + (int)sub;
        const bool live = (int)sub < p.P && it < items;
        unsigned rowitem, chunk = 0, pl, il;
        if (p.chunks > 1)
            p.divChunks.divmod((unsigned)(live ? it : 0), rowitem, chunk);
        else
            rowitem = (unsigned)(live ? it : 0);
        p.divItemRows.divmod(rowitem, pl, il);  // il: output row inside the strip
        const int j0 = (int)chunk * p.CO;
        const int col = j0 * dW + (int)c;       // the lane's input column
        // column reduce over the window rows: smallest ky wins ties
        float cv = -INFINITY;
        int cky = -1;
        if (live && (int)c < span && col < g.W) {
            const float *colp = tile + (int)pl * rows_w + ((int)il * dH) * g.W + col;  // the tile starts at row i0*dH
#pragma unroll
            for (int ky = 0; ky < (KH > 0 ? KH : 8); ++ky) {
                if (KH == 0 && ky >= kH) break;
                const float v = colp[ky * g.W];
                if (v > cv) {
                    cv = v;
                    cky = ky;
                }
            }
            if (KH == 0)
                for (int ky = 8; ky < kH; ++ky) {
                    const float v = colp[ky * g.W];
                    if (v > cv) {
                        cv = v;
                        cky = ky;
                    }
                }
        }
        // combine the kW columns of each output across lanes: larger value, then the smaller (ky, kx)
        float best = -INFINITY;
        int bky = -1, bkx = 0;
        const int lane_base = lane - (int)c;  // first lane of this lane's item
#pragma unroll
        for (int kx = 0; kx < (KW > 0 ? KW : 8); ++kx) {
            if (KW == 0 && kx >= kW) break;
            int srcl = lane_base + (int)c * dW + kx;
            srcl = srcl < 64 ? srcl : 63;       // lanes that are no output lanes read anything: discarded below
            const float v = __shfl(cv, srcl, 64);
            const int vy = __shfl(cky, srcl, 64);
            if (v > best || (v == best && vy >= 0 && (bky < 0 || vy < bky))) {
                best = v;
                bky = vy;
                bkx = kx;
            }
        }
        if (KW == 0)
            for (int kx = 8; kx < kW; ++kx) {
                int srcl = lane_base + (int)c * dW + kx;
                srcl = srcl < 64 ? srcl : 63;
                const float v = __shfl(cv, srcl, 64);
                const int vy = __shfl(cky, srcl, 64);
                if (v > best || (v == best && vy >= 0 && (bky < 0 || vy < bky))) {
                    best = v;
                    bky = vy;
                    bkx = kx;
                }
            }
        const int j = j0 + (int)c;
        if (live && (int)c < p.CO && j < g.Wo) {
            const int o = ((int)pl * ni + (int)il) * g.Wo + j;
            res[o] = best;
            // a window that never updated the maximum (all NaN or -inf): the CPU code stores (1, 0)
            res[nout + o] = bky < 0 ? 1.0f : (float)(bky + 1);
            res[2 * nout + o] = bky < 0 ? 0.0f : (float)(bkx + 1);
        }
    }
    __syncthreads();
    // ---- the three result arrays leave as contiguous streams (grouped planes lie back to back; a strip is a run
    // of whole output rows) ------------------------------------------------------------------------------------
    const long obase = (long)plane0 * g.Ho * g.Wo + (p.G > 1 ? 0 : (long)i0 * g.Wo);
    float *const dsts[3] = {out + obase, indy + obase, indx + obase};
#pragma unroll
    for (int a = 0; a < 3; ++a) {
        float *dst = dsts[a];
        const float *src = res + a * nout;
        for (int e = tid; e < nout; e += 256) dst[e] = src[e];
    }
}

constexpr long kPoolLdsBytes = 32 * 1024;  // the most LDS a pooling tile may ask for

// Shape of the forward tile kernel; false when a window is wider than a wavefront or one strip row does not fit LDS.
bool plan_pool_fwd(const PoolGeom &g, long planes, PoolFwdPlan &p) {
    if (g.kW > 64 || g.kH > 64) return false;
    const long plane_floats = (long)g.H * g.W;
    auto strip_floats = [&](long SR) { return ((SR - 1) * g.dH + g.kH) * (long)g.W; };
    if (strip_floats(1) * 4 > kPoolLdsBytes) return false;
    const long want = 4096;  // floats per workgroup
    p.G = 1;
    if (plane_floats <= want / 2 && plane_floats * 4 <= kPoolLdsBytes) {
        p.SR = g.Ho;
        long G = want / plane_floats;
        if (G > planes) G = planes;
        while (G > 1 && G * plane_floats * 4 > kPoolLdsBytes) --G;
        p.G = (int)(G < 1 ? 1 : G);
    } else {
        long SR = g.Ho;
        while (SR > 1 && (strip_floats(SR) > want || strip_floats(SR) * 4 > kPoolLdsBytes)) --SR;
        const long strips = (g.Ho + SR - 1) / SR;
        p.SR = (int)((g.Ho + strips - 1) / strips);  // even strips
    }
    if (p.G == 1 && strip_floats(p.SR) * 4 > kPoolLdsBytes) return false;
    p.strips = (g.Ho + p.SR - 1) / p.SR;
    // staged rows plus three result arrays
    if (((long)p.G * (p.G > 1 ? g.H : (p.SR - 1) * g.dH + g.kH) * g.W + 4 + 3L * p.G * p.SR * g.Wo) * 4 > 2 * kPoolLdsBytes)
        return false;
    // column chunks: a wavefront's 64 lanes cover (CO-1)*dW + kW input columns
    if (g.W <= 64) {
        p.CO = g.Wo;
        p.chunks = 1;
        p.P = 64 / g.W;
    } else {
        p.CO = (64 - g.kW) / g.dW + 1;
        p.chunks = (g.Wo + p.CO - 1) / p.CO;
        p.P = 1;
    }
    if (p.P < 1) p.P = 1;
    p.divStrips = FastDiv((uint32_t)p.strips);
    p.divItemRows = FastDiv((uint32_t)(p.G > 1 ? g.Ho : p.SR));
    p.divChunks = FastDiv((uint32_t)p.chunks);
    p.divLaneW = FastDiv((uint32_t)(p.P > 1 ? g.W : 64));
    return true;
}

// ---- backward ----------------------------------------------------------------------------------------

// Launch shape of the backward tile kernel.
struct PoolBwdPlan {
    int G;      // planes per workgroup (more than one only when a strip is the whole plane)
    int PR;     // pixel rows per strip
    int tiles;  // strips per plane
    FastDiv divTiles, divWo;
};

constexpr int kPoolBwdWindowsPerLane = 4;  // windows a lane keeps in registers: a workgroup takes up to 1024
constexpr int kPoolBwdPixelsPerLane = 16;  // pixels a lane writes (and mask values it holds): up to 4096 a workgroup

__global__ __launch_bounds__(256) void maxpool_bwd_tile_kernel(const float *__restrict__ gout,
                                                               const float *__restrict__ indy,
                                                               const float *__restrict__ indx,
                                                               float *__restrict__ gin, const PoolGeom g,
                                                               const PoolBwdPlan p, unsigned planes, int TH, int TW,
                                                               const InputMask mask) {
    extern __shared__ float px[];  // [np][nh][W]: the strip's gradInput
    constexpr int U = kPoolBwdWindowsPerLane;
    const int tid = threadIdx.x;
    unsigned grp, strip;
    p.divTiles.divmod(blockIdx.x, grp, strip);
    const unsigned plane0 = grp * (unsigned)p.G;
    const int np = (int)(planes - plane0 < (unsigned)p.G ? planes - plane0 : (unsigned)p.G);
    const int h0 = (int)strip * p.PR;
    const int nh = g.H - h0 < p.PR ? g.H - h0 : p.PR;
    const int npix = np * nh * g.W;
    // window rows that can reach pixel rows [h0, h0 + nh): i*dH + kH - 1 >= h0 and i*dH <= h0 + nh - 1
    const int t0 = h0 - g.kH + g.dH;  // numerator of the ceiling
    const int i_first = t0 <= 0 ? 0 : (int)g.divDH.div((unsigned)t0);
    int i_last = (int)g.divDH.div((unsigned)(h0 + nh - 1));
    if (i_last > g.Ho - 1) i_last = g.Ho - 1;
    const int ni = i_last - i_first + 1;  // may be <= 0: rows no window reaches stay zero
    const int per_plane = ni > 0 ? ni * g.Wo : 0;
    const int nwin = np * per_plane;

    // ---- the mask values of the strip's pixels are requested first and used last ------------------------------
    constexpr int PX = kPoolBwdPixelsPerLane;
    const long base = (long)plane0 * g.H * g.W + (p.G > 1 ? 0 : (long)h0 * g.W);
    float mv[PX];
    if (mask.in) {
        const float *m = mask.in + base;
#pragma unroll
        for (int u = 0; u < PX; ++u) {
            const int e = tid + u * 256;
            mv[u] = e < npix ? m[e] : 0.0f;
        }
    }

    // ---- the windows: three contiguous reads, all in flight before the tile is touched -----------------------
    float wg[U];
    int wt[U], wphase[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int e = tid + u * 256;
        wphase[u] = -1;
        wt[u] = 0;
        wg[u] = 0.0f;
        if (e < nwin) {
            unsigned pl = 0, rem = (unsigned)e, il, j;
            if (p.G > 1) g.divHoWo.divmod((unsigned)e, pl, rem);  // grouped planes are whole: Ho*Wo windows each
            p.divWo.divmod(rem, il, j);
            const int i = i_first + (int)il;
            const long o = ((long)(plane0 + pl) * g.Ho + i) * g.Wo + j;
            const float fy = indy[o], fx = indx[o];
            wg[u] = gout[o];
            const int y = (int)fy - 1, x = (int)fx - 1;
            const int h = i * g.dH + y, w = (int)j * g.dW + x;
            // the argmax lies inside the window by construction; anything else (the (1, 0) a window of NaNs
            // stores) names no pixel and is skipped
            if (y >= 0 && y < g.kH && x >= 0 && x < g.kW && h >= h0 && h < h0 + nh && w < g.W) {
                const int a = (int)g.divDH.div((unsigned)y), b = (int)g.divDW.div((unsigned)x);  // h/dH - i, w/dW - j
                wphase[u] = (TH - 1 - a) * TW + (TW - 1 - b);  // both differences descending
                wt[u] = ((int)pl * nh + (h - h0)) * g.W + w;
            }
        }
    }
    for (int e = tid; e < npix; e += 256) px[e] = 0.0f;
    __syncthreads();

    // ---- scatter, phase by phase: inside one phase no two windows share a pixel ------------------------------
    const int nphase = TH * TW;
    for (int ph = 0; ph < nphase; ++ph) {
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (wphase[u] == ph) px[wt[u]] += wg[u];
        __syncthreads();
    }

    // ---- the tile leaves as one contiguous stream --------------------------------------------------------------
    float *dst = gin + base;
    if (mask.in) {
#pragma unroll
        for (int u = 0; u < PX; ++u) {
            const int e = tid + u * 256;
            if (e < npix) dst[e] = mv[u] > mask.threshold ? px[e] : 0.0f;
        }
    } else {
#pragma unroll
        for (int u = 0; u < PX; ++u) {
            const int e = tid + u * 256;
            if (e < npix) dst[e] = px[e];
        }
    }
}

// Strip shape of the backward tile kernel; false when one pixel row with its windows does not fit.
bool plan_pool_bwd(const PoolGeom &g, long planes, int TH, PoolBwdPlan &p) {
    const long max_win = 256L * kPoolBwdWindowsPerLane;
    auto win_rows = [&](long PR) { return (PR + g.dH - 1) / g.dH + TH; };  // an upper bound
    const long max_pix = 256L * kPoolBwdPixelsPerLane;
    auto fits = [&](long G, long PR) {
        return G * PR * (long)g.W <= max_pix && G * win_rows(PR) * (long)g.Wo <= max_win;
    };
    if (!fits(1, 1)) return false;
    const long want = 4096;  // pixels per workgroup
    p.G = 1;
    if (fits(1, g.H)) {
        p.PR = g.H;
        // whole planes: the window count is exact, Ho*Wo per plane
        long G = want / ((long)g.H * g.W);
        if (G > planes) G = planes;
        if (G < 1) G = 1;
        while (G > 1 && (G * (long)g.H * g.W > max_pix || G * (long)g.Ho * g.Wo > max_win)) --G;
        p.G = (int)G;
    } else {
        long PR = want / g.W;
        if (PR < 1) PR = 1;
        if (PR > g.H) PR = g.H;
        while (PR > 1 && !fits(1, PR)) --PR;
        const long tiles = (g.H + PR - 1) / PR;
        p.PR = (int)((g.H + tiles - 1) / tiles);
    }
    p.tiles = (g.H + p.PR - 1) / p.PR;
    p.divTiles = FastDiv((uint32_t)p.tiles);
    p.divWo = FastDiv((uint32_t)(g.Wo > 0 ? g.Wo : 1));
    return true;
}

// The cell kernel: the default for the window shapes of the benchmark stacks (3x3 stride 2, 2x2 stride 2).  A lane
// owns the DH x DW pixels of one stride cell (y, x) = (h / DH, w / DW) of a plane.  Only the TH x TW =
// ceil(KH/DH) x ceil(KW/DW) windows (y - a, x - b) can name one of them: window (y - a, x - b) reaches pixel
// (ph, pw) of the cell when its saved argmax is (ky, kx) = (ph + a*DH, pw + b*DW).  The lane requests the three
// window arrays of those windows and the mask of its pixels up front (lanes run along x, so every request is a
// contiguous run; neighbouring cells share windows through the vector cache, as the forward kernel's lanes share
// rows), then adds the gradients that hit each pixel with a and b descending, i.e. windows in (i ascending, j
// ascending) order: the float addition order of the CPU module's scatter (mcw_nn/generic/SpatialMaxPooling.c:165-174).
// A window that does not hit adds +0.0f, which leaves a sum that started from +0.0f unchanged bit for bit.  No LDS,
// no barrier, no atomics, no zero-fill pass; 3*TH*TW + DH*DW loads and DH*DW stores per DH*DW pixels.
struct __attribute__((packed, aligned(4))) pool_float2u {  // two floats at a 4-byte aligned address
    float x, y;
};

template <int KH, int KW, int DH, int DW>
__global__ __launch_bounds__(256) void maxpool_bwd_cell_kernel(const float *__restrict__ gout,
                                                               const float *__restrict__ indy,
                                                               const float *__restrict__ indx,
                                                               float *__restrict__ gin, const PoolGeom g,
                                                               const FastDiv divXc, const FastDiv divCells, int Xc,
                                                               unsigned total_cells, const InputMask mask,
                                                               const TwinOutput twin, const unsigned cell_blocks,
                                                               const WeightJob side) {
    // workgroups behind the cells' carry a job of the next layer's (side_jobs.h)
    if (blockIdx.x >= cell_blocks) {
        reorder_weight(side, (blockIdx.x - cell_blocks) * 256u + threadIdx.x);
        return;
    }
    constexpr int TH = (KH + DH - 1) / DH, TW = (KW + DW - 1) / DW;
    const unsigned cell = blockIdx.x * blockDim.x + threadIdx.x;
    if (cell >= total_cells) return;
    unsigned plane, rem, y, x;
    divCells.divmod(cell, plane, rem);
    divXc.divmod(rem, y, x);
    const int h0 = (int)y * DH, w0 = (int)x * DW;
    // ---- requests: the windows, then the mask -- every load unconditional, from an index clamped into its array
    // (a load under a lane condition becomes a branch with its own wait, and the requests would go out one after
    // the other); what a clamped index fetched is discarded by the selects below ------------------------------------
    float wg[TH][TW], wy[TH][TW], wx[TH][TW];
    bool win[TH][TW];
    const long obase = (long)plane * g.Ho * g.Wo;
#pragma unroll
    for (int a = 0; a < TH; ++a)
#pragma unroll
        for (int b = 0; b < TW; ++b) {
            const int i = (int)y - a, j = (int)x - b;
            win[a][b] = i >= 0 && i < g.Ho && j >= 0 && j < g.Wo;
            const int ic = i < 0 ? 0 : i < g.Ho ? i : g.Ho - 1, jc = j < 0 ? 0 : j < g.Wo ? j : g.Wo - 1;
            const long o = obase + (long)ic * g.Wo + jc;
            wg[a][b] = gout[o];
            wy[a][b] = indy[o];
            wx[a][b] = indx[o];
        }
    const long plane_px = (long)plane * g.H * g.W;
    float mv[DH][DW];
    if (mask.in) {
#pragma unroll
        for (int ph = 0; ph < DH; ++ph) {
            const int h = h0 + ph < g.H ? h0 + ph : g.H - 1;
            const float *m = mask.in + plane_px + (long)h * g.W;
            if (DW == 2) {  // (W >= KW >= 2)
                // one 64-bit load per row; the last cell of an odd row reads the pair that ends at its one pixel
                const int wb = w0 + 1 < g.W ? w0 : g.W - 2;
                const pool_float2u t = *reinterpret_cast<const pool_float2u *>(m + wb);
                mv[ph][0] = wb == w0 ? t.x : t.y;
                mv[ph][DW - 1] = t.y;
            } else {
#pragma unroll
                for (int pw = 0; pw < DW; ++pw) mv[ph][pw] = m[w0 + pw < g.W ? w0 + pw : g.W - 1];
            }
        }
    }
    // ---- the adds: windows in (i, j) ascending order --------------------------------------------------------------
    float acc[DH][DW];
#pragma unroll
    for (int ph = 0; ph < DH; ++ph)
#pragma unroll
        for (int pw = 0; pw < DW; ++pw) acc[ph][pw] = 0.0f;
#pragma unroll
    for (int a = TH - 1; a >= 0; --a)
#pragma unroll
        for (int b = TW - 1; b >= 0; --b) {
            // the tap as a pixel of this cell; a window outside the plane names none
            const int ky = win[a][b] ? (int)wy[a][b] - 1 - a * DH : -1, kx = (int)wx[a][b] - 1 - b * DW;
#pragma unroll
            for (int ph = 0; ph < DH; ++ph)
#pragma unroll
                for (int pw = 0; pw < DW; ++pw) {
                    // taps beyond the window ((ph + a*DH, pw + b*DW) outside KH x KW) are never saved, so they never match
                    if (ph + a * DH >= KH || pw + b * DW >= KW) continue;
                    acc[ph][pw] += (ky == ph && kx == pw) ? wg[a][b] : 0.0f;
                }
        }
    // ---- the cell's pixels leave row by row -----------------------------------------------------------------------
#pragma unroll
    for (int ph = 0; ph < DH; ++ph) {
        if (h0 + ph >= g.H) continue;
        float *dst = gin + plane_px + (long)(h0 + ph) * g.W + w0;
#pragma unroll
        for (int pw = 0; pw < DW; ++pw)
            if (mask.in) acc[ph][pw] = mv[ph][pw] > mask.threshold ? acc[ph][pw] : 0.0f;
        // the second copy (TwinOutput): the same row inside another buffer
        float *dst2 = twin.base ? twin.base + (long)plane * twin.plane + (long)(h0 + ph) * twin.pitch + w0 : nullptr;
        if (DW == 2 && w0 + 1 < g.W) {  // one 64-bit store per row: a wavefront writes whole runs of a row
            pool_float2u t;
            t.x = acc[ph][0];
            t.y = acc[ph][DW - 1];
            *reinterpret_cast<pool_float2u *>(dst) = t;
            if (dst2) *reinterpret_cast<pool_float2u *>(dst2) = t;
        } else {
#pragma unroll
            for (int pw = 0; pw < DW; ++pw)
                if (w0 + pw < g.W) {
                    dst[pw] = acc[ph][pw];
                    if (dst2) dst2[pw] = acc[ph][pw];
                }
        }
    }
}

// The staged kernel: the cell kernel's arithmetic with the tile kernel's memory streams, the default for the window
// shapes of the benchmark stacks.  The cell kernel's stores -- 8 bytes per lane, rows of W floats that start
// anywhere -- reach the L2 as requests of 29 bytes on average, 2.2 times as many as the data needs (counters), and
// on launches large enough to stream from memory that costs it 10 - 20 %.  Here a workgroup owns a contiguous range
// of pixels (a group of small planes, or a strip of rows of a large one), its lanes compute the range's cells exactly
// as the cell kernel does (every load requested up front, no zero-fill, no scatter phases), park the results in LDS,
// and after ONE barrier the range leaves as one contiguous stream of full-width requests, the mask (requested first,
// as a contiguous stream too) applied on the way.  A second copy (TwinOutput) leaves the same way, row gaps included
// when they are known to hold zeros, so that it is a contiguous stream as well.
constexpr int kStagedPixelsPerLane = 16;  // a workgroup stages up to 4096 pixels (16 KB of LDS)
constexpr int kStagedCellsPerLane = 4;    // ... computed as up to 4 passes of 256 / Xc cell rows

struct PoolStagedPlan {
    int G;         // planes per workgroup (more than one only when a strip is the whole plane)
    int PR;        // pixel rows per strip (a multiple of the row stride unless the strip is the whole plane)
    int strips;    // strips per plane
    int Xc;        // cells per cell row
    int pass_rows; // cell rows a workgroup's 256 lanes cover at once: 256 / Xc
    int twin_step_rows, twin_step_cols;  // 256 = twin_step_rows * (row pitch of the second copy) + twin_step_cols
    FastDiv divStrips, divXc, divYc, divTwinPitch;
};

// A float at a byte offset from a wavefront-uniform base: the address is scalar base + 32-bit lane offset, one
// instruction's worth of address arithmetic instead of a 64-bit multiply-add per access.
__device__ __forceinline__ float pool_ld(const float *base, unsigned byte_off) {
    return *reinterpret_cast<const float *>(reinterpret_cast<const char *>(base) + byte_off);
}
__device__ __forceinline__ void pool_st(float *base, unsigned byte_off, float v) {
    *reinterpret_cast<float *>(reinterpret_cast<char *>(base) + byte_off) = v;
}
// Quotient and remainder of a number below 2^24 (a lane or cell index within a workgroup's range): the remainder
// through the full-rate 24-bit multiply.
__device__ __forceinline__ void pool_divmod24(const FastDiv &d, unsigned n, unsigned &q, unsigned &r) {
    q = d.div(n);
    r = n - __umul24(q, d.d);
}

// The instruction count per pixel is what bounds this kernel once its streams are contiguous, so the indexing is
// arranged to be cheap: a lane keeps ONE cell column x for all its cells (cell row r0 + ci * pass_rows of the range),
// so column clamps and validity are computed once; every array is addressed as a uniform per-workgroup base plus a
// 32-bit byte offset; and a window's saved argmax is compared as one number, wy * 1024 + wx (both small integers
// held in floats, so the sum is exact), against the constant that names the pixel.
template <int KH, int KW, int DH, int DW>
__global__ __launch_bounds__(256) void maxpool_bwd_staged_kernel(const float *__restrict__ gout,
                                                                 const float *__restrict__ indy,
                                                                 const float *__restrict__ indx,
                                                                 float *__restrict__ gin, const PoolGeom g,
                                                                 const PoolStagedPlan p, unsigned planes,
                                                                 const InputMask mask, const TwinOutput twin,
                                                                 const bool twin_gaps, const unsigned pool_blocks,
                                                                 const WeightJob side) {
    extern __shared__ float px[];  // [np][nh][W]: the range's gradInput
    if (blockIdx.x >= pool_blocks) {  // workgroups behind the pooling's carry a job of the next layer's (side_jobs.h)
        reorder_weight(side, (blockIdx.x - pool_blocks) * 256u + threadIdx.x);
        return;
    }
    constexpr int TH = (KH + DH - 1) / DH, TW = (KW + DW - 1) / DW;
    constexpr int PXL = kStagedPixelsPerLane, CI = kStagedCellsPerLane;
    const unsigned tid = threadIdx.x;
    unsigned grp, strip;
    p.divStrips.divmod(blockIdx.x, grp, strip);
    const unsigned plane0 = grp * (unsigned)p.G;
    const int np = (int)(planes - plane0 < (unsigned)p.G ? planes - plane0 : (unsigned)p.G);
    const int h0 = (int)strip * p.PR;
    const int nh = g.H - h0 < p.PR ? g.H - h0 : p.PR;
    const unsigned npix = (unsigned)(np * nh * g.W);
    const long base = (long)plane0 * g.H * g.W + (long)h0 * g.W;  // (h0 = 0 when planes are grouped)

    // The write-out's lanes are shifted so that every wavefront store of 64 consecutive floats starts on a 64-byte
    // line of gradInput: a store leaves the vector cache in 64-byte requests, and a run that starts mid-line costs five
    // requests instead of four (the range starts wherever its plane does).  Lane t takes the floats t - shift + 256 u;
    // the plan leaves room for the up to 15 lanes that fall in front of the range.
    float *dst = gin + base;
    const unsigned shift = (unsigned)((reinterpret_cast<uintptr_t>(dst) >> 2) & 15u);

    // ---- the mask of the range: requested first, used last ---------------------------------------------------------
    float mv[PXL];
    if (mask.in) {
        const float *m = mask.in + base;
#pragma unroll
        for (int u = 0; u < PXL; ++u) {
            const unsigned e = tid + u * 256u - shift;  // (wraps to a huge number in front of the range)
            mv[u] = pool_ld(m, (e < npix ? e : 0u) * 4u);
        }
    }

    // ---- the range's cells: all window requests of a lane's cells go out before the first is used -------------------
    const long wbase = (long)plane0 * g.Ho * g.Wo;  // the group's first window
    const float *gb = gout + wbase, *yb = indy + wbase, *xb = indx + wbase;
    const int yc0 = h0 / DH;  // strips start on a cell row
    const int nyc = (nh + DH - 1) / DH;
    const unsigned nrows = (unsigned)(np * nyc);  // cell rows of the range
    unsigned r0, x;
    pool_divmod24(p.divXc, tid, r0, x);
    const bool lane_live = r0 < (unsigned)p.pass_rows;  // (the last 256 mod Xc lanes have no column of their own)
    // the lane's column: which of its TW window columns exist, where they are, which of its DW pixel columns exist
    bool cv[TW], pv[DW];
    unsigned jb[TW];  // byte offset of the window column within a row of windows
#pragma unroll
    for (int b = 0; b < TW; ++b) {
        const int j = (int)x - b;
        cv[b] = j >= 0 && j < g.Wo;
        jb[b] = (unsigned)(j < 0 ? 0 : j < g.Wo ? j : g.Wo - 1) * 4u;
    }
#pragma unroll
    for (int pw = 0; pw < DW; ++pw) pv[pw] = (int)x * DW + pw < g.W;
    float wg[CI][TH][TW], code[CI][TH][TW];
    bool win[CI][TH][TW], rowlive[CI];
    int cell_hl[CI];        // the cell's first row in the range
    unsigned cell_px[CI];   // LDS offset of the cell's first pixel
#pragma unroll
    for (int ci = 0; ci < CI; ++ci) {
        const unsigned r = r0 + (unsigned)(ci * p.pass_rows);
        rowlive[ci] = lane_live && r < nrows;
        const unsigned rr = rowlive[ci] ? r : 0u;
        unsigned pl = 0, yl = rr;
        if (p.G > 1) pool_divmod24(p.divYc, rr, pl, yl);  // grouped planes are whole: Yc cell rows each
        const int y = yc0 + (int)yl;
        cell_hl[ci] = (int)yl * DH;
        // (every product here is of numbers far below 2^24: the full-rate 24-bit multiply)
        cell_px[ci] = __umul24(__umul24(pl, (unsigned)nh) + yl * DH, (unsigned)g.W) + x * DW;
#pragma unroll
        for (int a = 0; a < TH; ++a) {
            const int i = y - a;
            const bool rv = rowlive[ci] && i >= 0 && i < g.Ho;
            const unsigned iclamp = (unsigned)(i < 0 ? 0 : i < g.Ho ? i : g.Ho - 1);
            const unsigned ib = __umul24(__umul24(pl, (unsigned)g.Ho) + iclamp, (unsigned)g.Wo * 4u);
#pragma unroll
            for (int b = 0; b < TW; ++b) {
                // every load unconditional, from an index clamped into the group's windows; what a clamped index
                // fetched is discarded through `win`
                const unsigned o = ib + jb[b];
                win[ci][a][b] = rv && cv[b];
                wg[ci][a][b] = pool_ld(gb, o);
                code[ci][a][b] = __fmaf_rn(pool_ld(yb, o), 1024.0f, pool_ld(xb, o));
            }
        }
    }
#pragma unroll
    for (int ci = 0; ci < CI; ++ci) {
        float acc[DH][DW];
#pragma unroll
        for (int ph = 0; ph < DH; ++ph)
#pragma unroll
            for (int pw = 0; pw < DW; ++pw) acc[ph][pw] = 0.0f;
        // windows in (i, j) ascending order: the float addition order of the CPU module's scatter
#pragma unroll
        for (int a = TH - 1; a >= 0; --a)
#pragma unroll
            for (int b = TW - 1; b >= 0; --b) {
                const float c = win[ci][a][b] ? code[ci][a][b] : 0.0f;  // (a saved argmax is 1-based: never 0)
#pragma unroll
                for (int ph = 0; ph < DH; ++ph)
#pragma unroll
                    for (int pw = 0; pw < DW; ++pw) {
                        // taps beyond the window ((ph + a*DH, pw + b*DW) outside KH x KW) are never saved
                        if (ph + a * DH >= KH || pw + b * DW >= KW) continue;
                        const float hit = (float)((ph + a * DH + 1) * 1024 + pw + b * DW + 1);
                        acc[ph][pw] += c == hit ? wg[ci][a][b] : 0.0f;
                    }
            }
#pragma unroll
        for (int ph = 0; ph < DH; ++ph)
#pragma unroll
            for (int pw = 0; pw < DW; ++pw)
                if (rowlive[ci] && cell_hl[ci] + ph < nh && pv[pw]) px[cell_px[ci] + ph * g.W + pw] = acc[ph][pw];
    }
    __syncthreads();

    // ---- the range leaves as one contiguous stream -------------------------------------------------------------------
    float v[PXL];
#pragma unroll
    for (int u = 0; u < PXL; ++u) {  // all LDS reads first (from a clamped index: no branch, no wait in between)
        const unsigned e = tid + u * 256u - shift;
        v[u] = px[e < npix ? e : 0u];
    }
    if (mask.in) {
#pragma unroll
        for (int u = 0; u < PXL; ++u) v[u] = mv[u] > mask.threshold ? v[u] : 0.0f;
        if (twin.base) {  // the second copy takes the masked values
#pragma unroll
            for (int u = 0; u < PXL; ++u) {
                const unsigned e = tid + u * 256u - shift;
                if (e < npix) px[e] = v[u];
            }
        }
    }
#pragma unroll
    for (int u = 0; u < PXL; ++u) {
        const unsigned e = tid + u * 256u - shift;
        if (e < npix) pool_st(dst, e * 4u, v[u]);
    }
    if (!twin.base) return;
    if (mask.in) __syncthreads();
    // The second copy: per plane the rows lie twin.pitch apart; with twin_gaps the floats between one row's end and
    // the next row's start (zeros by the buffer's contract) are stored too, which makes the plane's rows one run.
    // A lane walks the run in steps of 256 floats and keeps (row, column) by carrying, without a division per float.
    const bool more_rows = h0 + nh < g.H;  // the strip's last row is followed by another row of the plane
    const unsigned run = (unsigned)(twin_gaps && !more_rows ? (nh - 1) * twin.pitch + g.W : nh * twin.pitch);
    unsigned hl0, xq0;
    pool_divmod24(p.divTwinPitch, tid, hl0, xq0);
    for (int pl = 0; pl < np; ++pl) {
        float *t = twin.base + (long)(plane0 + pl) * twin.plane + (long)h0 * twin.pitch;
        const float *src = px + pl * nh * g.W;
        unsigned xq = xq0, srow = __umul24(hl0, (unsigned)g.W);  // column in the padded row, LDS offset of the source row
        for (unsigned e = tid; e < run; e += 256u) {
            if (xq < (unsigned)g.W) pool_st(t, e * 4u, src[srow + xq]);
            else if (twin_gaps) pool_st(t, e * 4u, 0.0f);
            xq += (unsigned)p.twin_step_cols;
            srow += (unsigned)(p.twin_step_rows * g.W);
            if (xq >= (unsigned)twin.pitch) {
                xq -= (unsigned)twin.pitch;
                srow += (unsigned)g.W;
            }
        }
    }
}

// Shape of the staged kernel's launch; false when a cell row of a plane does not fit a workgroup's lanes or its LDS.
bool plan_pool_staged(const PoolGeom &g, long planes, int dH, int dW, int twin_pitch, PoolStagedPlan &p) {
    long max_pix = 256L * kStagedPixelsPerLane - 16;  // (up to 15 lanes of the write-out fall in front of the range)
    const int want = tuning().pool_bwd_pixels;  // (a tuning aid: a smaller workgroup share)
    if (want >= 256 && want < max_pix) max_pix = want;
    const long Yc = (g.H + dH - 1) / dH, Xc = (g.W + dW - 1) / dW;
    p.Xc = (int)Xc;
    if ((long)dH * g.W > max_pix || Xc > 256) return false;
    p.pass_rows = (int)(256 / Xc);
    const long max_rows = (long)kStagedCellsPerLane * p.pass_rows;  // cell rows per workgroup
    if ((long)g.H * g.W <= max_pix && Yc <= max_rows) {
        long G = max_pix / ((long)g.H * g.W);
        if (G > max_rows / Yc) G = max_rows / Yc;
        if (G > planes) G = planes;
        p.G = (int)(G < 1 ? 1 : G);
        p.PR = g.H;
    } else {
        p.G = 1;
        long cell_rows = max_pix / ((long)dH * g.W);  // cell rows per strip
        if (cell_rows > max_rows) cell_rows = max_rows;
        if (cell_rows < 1) return false;
        const long strips = (Yc + cell_rows - 1) / cell_rows;
        cell_rows = (Yc + strips - 1) / strips;  // even strips
        p.PR = (int)(cell_rows * dH);
    }
    // the kernel addresses a group's windows by 32-bit byte offsets built with 24-bit multiplies
    if ((long)p.G * g.Ho >= (1L << 24) || (long)p.G * g.Ho * g.Wo >= (1L << 29)) return false;
    p.strips = (g.H + p.PR - 1) / p.PR;
    p.divStrips = FastDiv((uint32_t)p.strips);
    p.divXc = FastDiv((uint32_t)Xc);
    p.divYc = FastDiv((uint32_t)Yc);
    const int pitch = twin_pitch > 0 ? twin_pitch : 1;
    p.divTwinPitch = FastDiv((uint32_t)pitch);
    p.twin_step_rows = 256 / pitch;
    p.twin_step_cols = 256 % pitch;
    return true;
}

// The direct kernel, for geometries the tile kernel's plan does not take.  Every pixel visits the windows
// covering it in (i ascending, j ascending) order.
__global__ __launch_bounds__(256) void maxpool_bwd_direct_kernel(const float *__restrict__ gout,
                                                                 const float *__restrict__ indy,
                                                                 const float *__restrict__ indx,
                                                                 float *__restrict__ gin, const PoolGeom g,
                                                                 unsigned total, const InputMask mask) {
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
    for (int i = i_lo; i <= i_hi; ++i) {
        const float wy = (float)((int)h - i * g.dH + 1);  // 1-based ky that would hit this row
        for (int j = j_lo; j <= j_hi; ++j) {
            const int o = i * g.Wo + j;
            const float wx = (float)((int)w - j * g.dW + 1);
            if (iy[o] == wy && ix[o] == wx) acc += go[o];
        }
    }
    if (mask.in) acc = mask.in[p] > mask.threshold ? acc : 0.0f;
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
struct __attribute__((packed, aligned(4))) gb_float4u {  // four floats at a 4-byte aligned address
    float x, y, z, w;
};

__global__ __launch_bounds__(256) void gradbias_partial_kernel(const float *__restrict__ gout,
                                                               float *__restrict__ part, int B, int M, int N,
                                                               int imgs_per_slice, int nslices, const FastDiv divQ) {
    const int m = blockIdx.x, slice = blockIdx.y;
    const int b0 = slice * imgs_per_slice;
    const int b1 = b0 + imgs_per_slice < B ? b0 + imgs_per_slice : B;
    // The slice is (b1-b0) rows of N floats, M*N apart.  Lanes walk it in quads of four consecutive floats of
    // one row (one 128-bit load each; the last quad of a row is cut to the row's end), four quads in flight.
    const int Q = (N + 3) >> 2;  // quads per row
    const unsigned total = (unsigned)(b1 - b0) * (unsigned)Q;
    const float *base = gout + ((long)b0 * M + m) * N;
    const long row_stride = (long)M * N;
    float sum = 0.0f;
    for (unsigned f0 = threadIdx.x; f0 < total; f0 += 256 * 4) {
        float v[4][4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const unsigned f = f0 + 256u * u;
            unsigned row, q;
            divQ.divmod(f < total ? f : 0, row, q);
            const float *src = base + (long)row * row_stride + 4 * q;
            const int left = f < total ? N - 4 * (int)q : 0;  // floats of the row from this quad on
            if (left >= 4) {
                const gb_float4u t = *reinterpret_cast<const gb_float4u *>(src);
                v[u][0] = t.x; v[u][1] = t.y; v[u][2] = t.z; v[u][3] = t.w;
            } else {
                v[u][0] = left > 0 ? src[0] : 0.0f;
                v[u][1] = left > 1 ? src[1] : 0.0f;
                v[u][2] = left > 2 ? src[2] : 0.0f;
                v[u][3] = 0.0f;
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) sum += (v[u][0] + v[u][1]) + (v[u][2] + v[u][3]);
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
                       float *indices, long out_plane, int out_pitch) {
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
    const double bytes = 4.0 * (planes * (double)H * W + 3.0 * total);
    const bool dense_out = (out_plane == 0 || out_plane == (long)g.Ho * g.Wo) && (out_pitch == 0 || out_pitch == g.Wo);
    g.oplane = dense_out ? (long)g.Ho * g.Wo : out_plane;
    g.opitch = dense_out ? g.Wo : out_pitch;
    if (!dense_out && (out_pitch < g.Wo || out_plane < (long)(g.Ho - 1) * out_pitch + g.Wo))
        return fail("SpatialMaxPooling: output planes overlap");
    PoolFwdPlan plan;
    // The pool_fwd_wave switch selects the wavefront-level tile kernel where its plan applies (dense outputs only).
    if (tuning().pool_fwd_wave && dense_out && plan_pool_fwd(g, planes, plan)) {
        const long blocks = ((planes + plan.G - 1) / plan.G) * plan.strips;
        if (blocks < (1L << 31)) {
            const long rows = plan.G > 1 ? H : (long)(plan.SR - 1) * dH + kH;
            const long nres = (long)plan.G * (plan.G > 1 ? g.Ho : plan.SR) * g.Wo;
            const size_t lds = sizeof(float) * (size_t)(((plan.G * rows * W + 3) & ~3L) + 3 * nres);
            {
                LaunchScope scope(pool_label("maxpool_fwd", g, planes), 0.0, bytes);
                const dim3 grid((unsigned)blocks), block(256);
                float *iy = indices, *ix = indices + total;
#define THGPU_POOL_FWD(KH_, KW_, DH_, DW_)                                                                         \
    hipLaunchKernelGGL((maxpool_fwd_tile_kernel<KH_, KW_, DH_, DW_>), grid, block, lds, s, in, out, iy, ix, g, plan, \
                       (unsigned)planes)
                if (kH == 3 && kW == 3 && dH == 2 && dW == 2) THGPU_POOL_FWD(3, 3, 2, 2);
                else if (kH == 2 && kW == 2 && dH == 2 && dW == 2) THGPU_POOL_FWD(2, 2, 2, 2);
                else THGPU_POOL_FWD(0, 0, 0, 0);
#undef THGPU_POOL_FWD
            }
            return check_launch("maxpool_fwd");
        }
    }
    {
        LaunchScope scope(pool_label("maxpool_fwd", g, planes), 0.0, bytes);
        const dim3 grid((unsigned)((total + 255) / 256)), block(256);
        if (kH == 3 && kW == 3)
            hipLaunchKernelGGL((maxpool_fwd_direct_kernel<3, 3>), grid, block, 0, s, in, out, indices, indices + total, g,
                               (unsigned)total);
        else if (kH == 2 && kW == 2)
            hipLaunchKernelGGL((maxpool_fwd_direct_kernel<2, 2>), grid, block, 0, s, in, out, indices, indices + total, g,
                               (unsigned)total);
        else
            hipLaunchKernelGGL((maxpool_fwd_direct_kernel<0, 0>), grid, block, 0, s, in, out, indices, indices + total, g,
                               (unsigned)total);
    }
    return check_launch("maxpool_fwd");
}

// Host check of the tile planners: a strip's rows and windows must fit the LDS and register budgets the kernels
// assume, and the strips must cover the plane.
long pool_plan_selftest() {
    long bad = 0;
    const int sizes[] = {2, 3, 6, 7, 12, 13, 14, 24, 27, 28, 55, 56, 64, 65, 112, 224, 231, 1000, 5000};
    for (int H : sizes)
        for (int W : sizes)
            for (int k = 1; k <= 4; ++k)
                for (int kw : {k, 2})  // square windows, and every height against a width of 2
                    for (int d = 1; d <= 4; ++d)
                        for (int dw : {d, 2}) {
                    if (H < k || W < kw) continue;
                    const int th = (k + d - 1) / d;
                    PoolGeom g;
                    g.H = H; g.W = W; g.kH = k; g.kW = kw; g.dH = d; g.dW = dw;
                    g.Ho = (H - k) / d + 1;
                    g.Wo = (W - kw) / dw + 1;
                    for (long planes : {1L, 5L, 4096L}) {
                        PoolBwdPlan p;
                        if (plan_pool_bwd(g, planes, th, p)) {
                            bool ok = p.G >= 1 && p.G <= planes && p.PR >= 1 && p.PR <= H && (p.G == 1 || p.PR == H) &&
                                      (long)p.G * p.PR * W <= 256L * kPoolBwdPixelsPerLane && (long)p.tiles * p.PR >= H &&
                                      (long)(p.tiles - 1) * p.PR < H;
                            for (int t = 0; t < p.tiles && ok; ++t) {
                                const int h0 = t * p.PR, nh = (h0 + p.PR < H ? h0 + p.PR : H) - h0;
                                const int t0 = h0 - k + d;
                                const int i_first = t0 <= 0 ? 0 : t0 / d;
                                int i_last = (h0 + nh - 1) / d;
                                if (i_last > g.Ho - 1) i_last = g.Ho - 1;
                                const long nwin = (long)p.G * (i_last - i_first + 1 > 0 ? i_last - i_first + 1 : 0) * g.Wo;
                                ok = nwin <= 256L * kPoolBwdWindowsPerLane;
                            }
                            if (!ok) ++bad;
                        }
                        PoolStagedPlan sp;
                        if (plan_pool_staged(g, planes, d, dw, W + 3, sp)) {
                            const long Yc = (H + d - 1) / d, Xc = (W + dw - 1) / dw;
                            const long cell_rows = sp.G > 1 || sp.PR == H ? Yc : sp.PR / d;
                            const bool ok = sp.G >= 1 && sp.G <= planes && sp.PR >= 1 && sp.PR <= H &&
                                            (sp.G == 1 || sp.PR == H) && (sp.PR == H || sp.PR % d == 0) &&
                                            (long)sp.G * sp.PR * W <= 256L * kStagedPixelsPerLane - 16 &&
                                            Xc <= 256 && sp.pass_rows == 256 / Xc &&
                                            (long)sp.G * cell_rows <= (long)kStagedCellsPerLane * sp.pass_rows &&
                                            (long)sp.strips * sp.PR >= H && (long)(sp.strips - 1) * sp.PR < H &&
                                            sp.Xc == Xc;
                            if (!ok) ++bad;
                        }
                        PoolFwdPlan f;
                        if (plan_pool_fwd(g, planes, f)) {
                            const long rows = f.G > 1 ? H : (long)(f.SR - 1) * d + k;
                            bool ok = f.G >= 1 && f.G <= planes && f.SR >= 1 && f.SR <= g.Ho &&
                                      (f.G == 1 || f.SR == g.Ho) && (long)f.G * rows * W * 4 <= kPoolLdsBytes &&
                                      (long)f.strips * f.SR >= g.Ho && (long)(f.strips - 1) * f.SR < g.Ho &&
                                      (long)f.chunks * f.CO >= g.Wo && (f.CO - 1) * dw + kw <= (W <= 64 ? W : 64) &&
                                      f.P >= 1 && (f.P == 1 || f.P * W <= 64) && (f.P == 1 || f.chunks == 1);
                            // the last strip's rows end inside the plane
                            ok = ok && ((long)(g.Ho - 1) * d + k <= H);
                            if (!ok) ++bad;
                        }
                    }
                }
    return bad;
}

int maxpool_bwd_launch(const float *gout, const float *indices, long planes, int H, int W, int Ho, int Wo, int kH,
                       int kW, int dH, int dW, float *gin, InputMask mask, TwinOutput twin, bool *wrote_twin,
                       bool twin_gaps) {
    if (wrote_twin) *wrote_twin = false;
    hipStream_t s = stream();
    if (!s) return 1;
    PoolGeom g;
    g.H = H; g.W = W; g.kH = kH; g.kW = kW; g.dH = dH; g.dW = dW; g.Ho = Ho; g.Wo = Wo;
    g.oplane = (long)Ho * Wo;
    g.opitch = Wo;
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
    double bytes = 4.0 * ((mask.in ? 2.0 : 1.0) * (double)total + 3.0 * ototal);
    // The cell kernel takes the window shapes it is compiled for; the pool_bwd_tile and pool_bwd_direct switches force
    // the LDS tile kernel and the direct kernel (testing and tuning aids).
    const bool cell_shape = (kH == 3 && kW == 3 && dH == 2 && dW == 2) || (kH == 2 && kW == 2 && dH == 2 && dW == 2);
    // Staged or cell kernel: a launch of a few microseconds is over before the staged kernel's chain of requests,
    // barrier and write-out has paid for itself (measured cross-over: 13x13 planes at batch 128, 5.5 M pixels, run
    // 14 us on the cell kernel and 17.5 us staged; from some 20 M pixels on the staged kernel is ahead, by a third at
    // sizes that stream from memory).  pool_bwd_pixels > 0 pins the staged kernel.
    const bool small_launch = total < 12L * 1000 * 1000 && tuning().pool_bwd_pixels == 0;
    PoolStagedPlan sp;
    if (cell_shape && !tuning().pool_bwd_direct && !tuning().pool_bwd_tile && !tuning().pool_bwd_cell && !small_launch &&
        Ho > 0 && Wo > 0 && plan_pool_staged(g, planes, dH, dW, twin.base ? twin.pitch : 0, sp)) {
        const long blocks = ((planes + sp.G - 1) / sp.G) * sp.strips;
        if (blocks < (1L << 30)) {
            WeightJob side = {};
            unsigned side_blocks = 0;
            if (twin.base) {  // the second copy is part of the launch's traffic
                bytes += 4.0 * (double)total;
                if (wrote_twin) *wrote_twin = true;
                // ... and whoever reads that copy next may have a kernel bank to re-order: this launch carries it
                if (take_bank_job(side)) {
                    side_blocks = (side.count + 255u) / 256u;
                    bytes += 4.0 * (side.count + (double)side.M * side.C * side.kH * side.kW);
                }
            }
            {
                LaunchScope scope(pool_label("maxpool_bwd", g, planes), 0.0, bytes);
                const dim3 grid((unsigned)blocks + side_blocks), block(256);
                const size_t lds = sizeof(float) * (size_t)sp.G * sp.PR * W;
#define THGPU_POOL_BWD_STAGED(KH_, KW_, DH_, DW_)                                                                     \
    hipLaunchKernelGGL((maxpool_bwd_staged_kernel<KH_, KW_, DH_, DW_>), grid, block, lds, s, gout, indices,           \
                       indices + ototal, gin, g, sp, (unsigned)planes, mask, twin, twin_gaps, (unsigned)blocks, side)
                if (kH == 3) THGPU_POOL_BWD_STAGED(3, 3, 2, 2);
                else THGPU_POOL_BWD_STAGED(2, 2, 2, 2);
#undef THGPU_POOL_BWD_STAGED
            }
            return check_launch("maxpool_bwd");
        }
    }
    if (cell_shape && !tuning().pool_bwd_direct && !tuning().pool_bwd_tile && Ho > 0 && Wo > 0) {
        const long Yc = (H + dH - 1) / dH, Xc = (W + dW - 1) / dW;
        const long cells = planes * Yc * Xc;
        if (cells < (1L << 31)) {
            WeightJob side = {};
            unsigned side_blocks = 0;
            if (twin.base) {  // the second copy is part of the launch's traffic
                bytes += 4.0 * (double)total;
                if (wrote_twin) *wrote_twin = true;
                // ... and whoever reads that copy next may have a kernel bank to re-order: this launch carries it
                if (take_bank_job(side)) {
                    side_blocks = (side.count + 255u) / 256u;
                    bytes += 4.0 * (side.count + (double)side.M * side.C * side.kH * side.kW);
                }
            }
            {
                LaunchScope scope(pool_label("maxpool_bwd", g, planes), 0.0, bytes);
                const unsigned cell_blocks = (unsigned)((cells + 255) / 256);
                const dim3 grid(cell_blocks + side_blocks), block(256);
                const FastDiv divXc((uint32_t)Xc), divCells((uint32_t)(Yc * Xc));
#define THGPU_POOL_BWD_CELL(KH_, KW_, DH_, DW_)                                                                     \
    hipLaunchKernelGGL((maxpool_bwd_cell_kernel<KH_, KW_, DH_, DW_>), grid, block, 0, s, gout, indices,             \
                       indices + ototal, gin, g, divXc, divCells, (int)Xc, (unsigned)cells, mask, twin, cell_blocks, side)
                if (kH == 3) THGPU_POOL_BWD_CELL(3, 3, 2, 2);
                else THGPU_POOL_BWD_CELL(2, 2, 2, 2);
#undef THGPU_POOL_BWD_CELL
            }
            return check_launch("maxpool_bwd");
        }
    }
    PoolBwdPlan plan;
    if (!tuning().pool_bwd_direct && Ho > 0 && Wo > 0 && th * tw <= 64 && plan_pool_bwd(g, planes, th, plan)) {
        const long blocks = ((planes + plan.G - 1) / plan.G) * plan.tiles;
        if (blocks < (1L << 31)) {
            const size_t lds = sizeof(float) * (size_t)plan.G * plan.PR * W;
            {
                LaunchScope scope(pool_label("maxpool_bwd", g, planes), 0.0, bytes);
                hipLaunchKernelGGL(maxpool_bwd_tile_kernel, dim3((unsigned)blocks), dim3(256), lds, s, gout, indices,
                                   indices + ototal, gin, g, plan, (unsigned)planes, th, tw, mask);
            }
            return check_launch("maxpool_bwd");
        }
    }
    {
        LaunchScope scope(pool_label("maxpool_bwd", g, planes), 0.0, bytes);
        hipLaunchKernelGGL(maxpool_bwd_direct_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, gout,
                           indices, indices + ototal, gin, g, (unsigned)total, mask);
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
                           part, (int)B, M, (int)N, ips, (int)nslices, FastDiv((uint32_t)((N + 3) / 4)));
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

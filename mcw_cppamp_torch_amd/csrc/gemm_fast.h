// The fast fp32 MFMA GEMM kernel (see gemm_mfma.h for the problem statement).
// Included by one small translation unit per tile configuration.
//
// Structure
//   * A workgroup of WGM x WGN wavefronts owns a BM x BN tile of C, each
//     wavefront TM x TN blocks of 32x32 outputs, one v_mfma_f32_32x32x2_f32
//     accumulator (16 registers per lane) per block.
//   * No bounds checks in the main loop.  A tile at the lower/right edge is
//     shifted back so that it lies inside the matrix (needs M >= BM, J >= BN;
//     smaller problems take the bounds-checked generic kernel) and stores only
//     the rows/columns no other tile owns.  Only the last reduction step of an
//     image can be partial; it takes a separate, masked fetch.
//   * LDS holds both operand tiles as [x][r] (x the free index, r the
//     reduction index, 16 + 4 floats per row).  Each lane fetches its MFMA
//     operands with 128-bit LDS reads: lane (x, h) reads r = 8h .. 8h+7, and
//     MFMA step s takes r = s from the lower half-wave and r = 8 + s from the
//     upper one.  A and B use the same permutation of r, so the sum over r is
//     unchanged.  The row pitch of 20 floats makes 8 consecutive lanes hit 32
//     distinct banks.
//   * LDS is double buffered; the next tile's global loads are issued before
//     the current tile's MFMAs and written to the other buffer afterwards: one
//     barrier per reduction step.
#pragma once

#include <type_traits>

#include "gemm_mfma.h"

namespace thgpu {

constexpr int LDK = GEMM_BK + 4;  // LDS row pitch in floats

// Wavefronts per SIMD the register allocation must leave room for: the
// accumulators take (BM/WGM)*(BN/WGN)/64 registers of the 512 a lane has.
template <int BM, int BN, int WGM, int WGN>
constexpr int gemm_min_waves() {
    return (BM / WGM) * (BN / WGN) / 64 >= 128 ? 2 : 3;
}

template <int BM, int BN, int WGM, int WGN, int LA, int LB, bool RED>
__global__ __launch_bounds__(WGM *WGN * 64)
    __attribute__((amdgpu_waves_per_eu(gemm_min_waves<BM, BN, WGM, WGN>()))) void gemm_fast_kernel(const GemmArgs g) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int BK = GEMM_BK;
    constexpr int TM = BM / WGM / 32, TN = BN / WGN / 32;
    constexpr int NA = BM * BK / NT, NB = BN * BK / NT;
    static_assert(BM % (WGM * 32) == 0 && BN % (WGN * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(NT % 16 == 0 && NA >= 4 && NB >= 4 && NA % 4 == 0 && NB % 4 == 0, "loader shape");
    static_assert(NT % BM == 0 && NT % BN == 0, "x-contiguous loaders give every thread one row/column");
    static_assert(!RED || (LA != LD_XC_SCALAR && LB != LD_XC_SCALAR), "reduction batching needs r-contiguous operands");

    __shared__ __attribute__((aligned(16))) float As[2][BM][LDK];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN][LDK];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int half = lane >> 5, l32 = lane & 31;

    // ---- which tile, which part of the reduction --------------------------------
    unsigned pid = xcd_remap(blockIdx.x, g.total);
    unsigned ti, tj, split, rest;
    g.divTilesM.divmod(pid, rest, ti);
    g.divTilesJ.divmod(rest, split, tj);
    const int own_i0 = (int)ti * BM, own_j0 = (int)tj * BN;
    const int i0 = own_i0 + BM <= g.M ? own_i0 : g.M - BM;  // shifted back at the edge
    const int j0 = own_j0 + BN <= g.J ? own_j0 : g.J - BN;

    int step = (int)split * g.steps_per_split;
    int step_end = step + g.steps_per_split;
    if (step_end > g.steps_total) step_end = g.steps_total;
    const int nsteps = step_end - step;
    int ld_img = 0, ld_r0 = step * BK;
    if (RED) {
        unsigned im, st;
        g.divSpi.divmod((unsigned)step, im, st);
        ld_img = (int)im;
        ld_r0 = (int)st * BK;
    }

    // ---- loader set-up -------------------------------------------------------------
    // Per operand: a 64-bit per-thread base pointer (tile origin + thread part)
    // and compile-time multiples of the uniform stride for the thread's elements.
    const float *pA;
    int a_x, a_r;  // thread's first (x, r) inside the tile
    if (LA == LD_RC_VEC) {
        a_x = tid >> 2;
        a_r = (tid & 3) * 4;
        pA = g.A + (long)(i0 + a_x) * g.sA + a_r;
    } else if (LA == LD_RC_SCALAR) {
        a_x = tid >> 4;
        a_r = tid & 15;
        pA = g.A + (long)(i0 + a_x) * g.sA + a_r;
    } else {
        a_x = tid % BM;
        a_r = (tid / BM) * NA;  // NA consecutive r per thread (NT >= BM), or all 16 (NT < BM)
        pA = g.A + (long)(i0 + a_x);
    }
    const float *pB;
    int b_x, b_r;
    if (LB == LD_RC_VEC) {
        b_x = tid >> 2;
        b_r = (tid & 3) * 4;
        pB = g.B + (long)(j0 + b_x) * g.sB + b_r;
    } else if (LB == LD_RC_SCALAR) {
        b_x = tid >> 4;
        b_r = tid & 15;
        pB = g.B + (long)(j0 + b_x) * g.sB + b_r;
    } else {
        b_x = tid % BN;
        b_r = (tid / BN) * NB;
        unsigned img, n;
        g.divN.divmod((unsigned)(j0 + b_x), img, n);
        pB = g.B + (long)img * g.bsB + n;
    }
    floatx16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

    float ra[NA], rb[NB];

    // One operand's global loads for the step at (ld_img, ld_r0).  TAIL handles
    // a step that runs past R: addresses are clamped into the row and the
    // values past R are zeroed.
    auto fetch_one = [&](auto tail_tag, auto kind_tag, const float *base, long stride, int t_r, float *dst,
                         auto count_tag) {
        constexpr bool TAIL = decltype(tail_tag)::value;
        constexpr int KIND = decltype(kind_tag)::value;
        constexpr int CNT = decltype(count_tag)::value;
        const int r_base = ld_r0 + t_r;
        if (KIND == LD_RC_VEC) {
            // element q*4+e: row q*(NT/4), r = r_base + e
#pragma unroll
            for (int q = 0; q < CNT / 4; ++q) {
                const float *p = base + (long)(q * (NT / 4)) * stride + ld_r0;
                if (!TAIL) {
                    float4 v = *reinterpret_cast<const float4 *>(p);
                    dst[q * 4 + 0] = v.x;
                    dst[q * 4 + 1] = v.y;
                    dst[q * 4 + 2] = v.z;
                    dst[q * 4 + 3] = v.w;
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const int r = r_base + e;
                        const int back = r < g.R ? 0 : r - (g.R - 1);
                        const float v = p[e - back];
                        dst[q * 4 + e] = r < g.R ? v : 0.0f;
                    }
                }
            }
        } else if (KIND == LD_RC_SCALAR) {
            // element q: row q*(NT/16), r = r_base
            const int back = (!TAIL || r_base < g.R) ? 0 : r_base - (g.R - 1);
#pragma unroll
            for (int q = 0; q < CNT; ++q) {
                const float v = base[(long)(q * (NT / 16)) * stride + (ld_r0 - back)];
                dst[q] = (!TAIL || r_base < g.R) ? v : 0.0f;
            }
        } else {
            // element e: r = r_base + e, the thread's own row/column
#pragma unroll
            for (int e = 0; e < CNT; ++e) {
                const int r = r_base + e;
                const int rr = (!TAIL || r < g.R) ? r : g.R - 1;
                const float v = base[(long)rr * stride];
                dst[e] = (!TAIL || r < g.R) ? v : 0.0f;
            }
        }
    };

    auto fetch = [&]() {
        const float *a = pA + (RED ? (long)ld_img * g.rbA : 0L);
        const float *b = pB + (RED ? (long)ld_img * g.rbB : 0L);
        if (ld_r0 + BK <= g.R) {
            fetch_one(std::false_type{}, std::integral_constant<int, LA>{}, a, g.sA, a_r, ra,
                      std::integral_constant<int, NA>{});
            fetch_one(std::false_type{}, std::integral_constant<int, LB>{}, b, g.sB, b_r, rb,
                      std::integral_constant<int, NB>{});
        } else {
            fetch_one(std::true_type{}, std::integral_constant<int, LA>{}, a, g.sA, a_r, ra,
                      std::integral_constant<int, NA>{});
            fetch_one(std::true_type{}, std::integral_constant<int, LB>{}, b, g.sB, b_r, rb,
                      std::integral_constant<int, NB>{});
        }
        ld_r0 += BK;
        if (RED && ld_r0 >= g.R) {
            ld_r0 = 0;
            ++ld_img;
        }
    };

    auto stash_one = [&](auto kind_tag, float (*tile)[LDK], int t_x, int t_r, const float *src, auto count_tag) {
        constexpr int KIND = decltype(kind_tag)::value;
        constexpr int CNT = decltype(count_tag)::value;
        if (KIND == LD_RC_VEC) {
#pragma unroll
            for (int q = 0; q < CNT / 4; ++q)
                *reinterpret_cast<float4 *>(&tile[t_x + q * (NT / 4)][t_r]) =
                    make_float4(src[q * 4], src[q * 4 + 1], src[q * 4 + 2], src[q * 4 + 3]);
        } else if (KIND == LD_RC_SCALAR) {
#pragma unroll
            for (int q = 0; q < CNT; ++q) tile[t_x + q * (NT / 16)][t_r] = src[q];
        } else {
#pragma unroll
            for (int w = 0; w < CNT / 4; ++w)
                *reinterpret_cast<float4 *>(&tile[t_x][t_r + 4 * w]) =
                    make_float4(src[w * 4], src[w * 4 + 1], src[w * 4 + 2], src[w * 4 + 3]);
        }
    };

    auto stash = [&](int buf) {
        stash_one(std::integral_constant<int, LA>{}, As[buf], a_x, a_r, ra, std::integral_constant<int, NA>{});
        stash_one(std::integral_constant<int, LB>{}, Bs[buf], b_x, b_r, rb, std::integral_constant<int, NB>{});
    };

    if (nsteps > 0) {
        fetch();
        stash(0);
    }
    __syncthreads();

    for (int s = 0; s < nsteps; ++s) {
        const int buf = s & 1;
        if (s + 1 < nsteps) fetch();

        // MFMA operands: 8 reduction indices per lane and block, two 128-bit reads.
        float4 av[TM][2], bv[TN][2];
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
            for (int a = 0; a < TM; ++a)
                av[a][h2] = *reinterpret_cast<const float4 *>(&As[buf][wm * (TM * 32) + a * 32 + l32][8 * half + 4 * h2]);
#pragma unroll
            for (int b = 0; b < TN; ++b)
                bv[b][h2] = *reinterpret_cast<const float4 *>(&Bs[buf][wn * (TN * 32) + b * 32 + l32][8 * half + 4 * h2]);
        }
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
#pragma unroll
                for (int a = 0; a < TM; ++a) {
                    const float x = e == 0 ? av[a][h2].x : e == 1 ? av[a][h2].y : e == 2 ? av[a][h2].z : av[a][h2].w;
#pragma unroll
                    for (int b = 0; b < TN; ++b) {
                        const float y =
                            e == 0 ? bv[b][h2].x : e == 1 ? bv[b][h2].y : e == 2 ? bv[b][h2].z : bv[b][h2].w;
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(x, y, acc[a][b], 0, 0, 0);
                    }
                }
            }
        }
        if (s + 1 < nsteps) stash(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue ----------------------------------------------------------------------
    // Accumulator register v of lane l holds D[8*(v/4) + 4*(l/32) + v%4][l%32].
    const bool partial = g.nsplit > 1;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int jg = j0 + wn * (TN * 32) + b * 32 + l32;
        if (jg < own_j0) continue;  // owned by the neighbouring tile
        long coff;
        if (partial) {
            coff = (long)split * g.M * g.J + jg;
        } else if (!RED && g.N != g.J) {
            unsigned im, n;
            g.divN.divmod((unsigned)jg, im, n);
            coff = (long)im * g.bsC + n;
        } else {
            coff = jg;
        }
#pragma unroll
        for (int a = 0; a < TM; ++a) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = i0 + wm * (TM * 32) + a * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                if (i < own_i0) continue;
                float val = acc[a][b][v];
                if (partial) {
                    g.ws[coff + (long)i * g.J] = val;
                } else {
                    float *c = g.C + (long)i * g.sC + coff;
                    val *= g.alpha;
                    if (g.bias) val += g.bias[i];
                    if (g.beta != 0.0f) val += g.beta * *c;
                    *c = val;
                }
            }
        }
    }
}

template <int BM, int BN, int WGM, int WGN, int LA, int LB, bool RED>
int gemm_fast_go(const GemmArgs &g, hipStream_t s) {
    hipLaunchKernelGGL((gemm_fast_kernel<BM, BN, WGM, WGN, LA, LB, RED>), dim3(g.total), dim3(WGM * WGN * 64), 0, s, g);
    return 0;
}

// Dispatch over the loader kinds for one tile configuration.
template <int BM, int BN, int WGM, int WGN>
int gemm_fast_dispatch(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
#define THGPU_CASE(LA_, LB_)                                                          \
    if (la == LA_ && lb == LB_) {                                                     \
        if (red) {                                                                    \
            if constexpr (LA_ != LD_XC_SCALAR && LB_ != LD_XC_SCALAR)                 \
                return gemm_fast_go<BM, BN, WGM, WGN, LA_, LB_, true>(g, s);          \
            else                                                                      \
                return fail("gemm: reduction batching needs r-contiguous operands");  \
        }                                                                             \
        return gemm_fast_go<BM, BN, WGM, WGN, LA_, LB_, false>(g, s);                 \
    }
    THGPU_CASE(LD_RC_VEC, LD_RC_VEC)
    THGPU_CASE(LD_RC_VEC, LD_RC_SCALAR)
    THGPU_CASE(LD_RC_VEC, LD_XC_SCALAR)
    THGPU_CASE(LD_RC_SCALAR, LD_RC_VEC)
    THGPU_CASE(LD_RC_SCALAR, LD_RC_SCALAR)
    THGPU_CASE(LD_RC_SCALAR, LD_XC_SCALAR)
    THGPU_CASE(LD_XC_SCALAR, LD_RC_VEC)
    THGPU_CASE(LD_XC_SCALAR, LD_RC_SCALAR)
    THGPU_CASE(LD_XC_SCALAR, LD_XC_SCALAR)
#undef THGPU_CASE
    return fail("gemm: unknown loader combination (%d, %d)", la, lb);
}

}  // namespace thgpu

// Bounds-checked fp32 MFMA GEMM for gfx950 (see gemm_mfma.h for the problem
// statement): the fallback for problems with fewer rows or columns than the
// smallest tile of the fast kernel (gemm_fast.h).  Every global access is
// predicated, so any M, J, R work.
//
// Tiling: 2 x 2 wavefronts own a 64 x 64 tile of C, one v_mfma_f32_32x32x2_f32
// accumulator per wavefront.  Both operand tiles are staged in LDS in
// reduction-major order, As[r][i] and Bs[r][j], so that the per-lane MFMA
// operand fetch (lane l supplies A[i = l%32][k = l/32], B[k = l/32][j = l%32])
// is a conflict-free ds_read_b32.  LDS is double buffered, one barrier per step.
#include "gemm_mfma.h"

namespace thgpu {

namespace {

constexpr int BK = GEMM_BK;
constexpr int LDS_PAD = 2;

template <int BM, int BN, int WGM, int WGN, bool A_RC, bool B_RC, bool RED>
__global__ __launch_bounds__(WGM *WGN * 64) void gemm_generic_kernel(const GemmArgs g) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int TM = BM / WGM / 32, TN = BN / WGN / 32;
    constexpr int LDA = BM + LDS_PAD, LDB = BN + LDS_PAD;
    constexpr int NA = BM * BK / NT, NB = BN * BK / NT;
    static_assert(BM % (WGM * 32) == 0 && BN % (WGN * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(NT % BK == 0 && (BM * BK) % NT == 0 && (BN * BK) % NT == 0, "loader shape");
    static_assert(A_RC || NT % BM == 0, "i-contiguous A loader needs NT % BM == 0");
    static_assert(B_RC || NT % BN == 0, "j-contiguous B loader needs NT % BN == 0");
    static_assert(!RED || (A_RC && B_RC), "reduction batching needs r-contiguous operands");

    __shared__ float As[2][BK][LDA];
    __shared__ float Bs[2][BK][LDB];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;

    // ---- which tile ----------------------------------------------------------
    unsigned pid = xcd_remap(blockIdx.x, g.total);
    unsigned ti, tj, split, rest;
    g.divTilesM.divmod(pid, rest, ti);
    g.divTilesJ.divmod(rest, split, tj);
    const int i0 = (int)ti * BM, j0 = (int)tj * BN;

    // ---- loader set-up -------------------------------------------------------
    // A, r-contiguous: 16 consecutive lanes read 16 consecutive r of one row.
    // A, i-contiguous: consecutive lanes read consecutive rows i.
    const int a_r = A_RC ? (tid & 15) : (tid / BM);
    const int a_i = A_RC ? (tid >> 4) : (tid % BM);
    constexpr int A_STEP = A_RC ? NT / 16 : NT / BM;  // i step (RC) or r step (IC) between a thread's elements
    const int b_r = B_RC ? (tid & 15) : (tid / BN);
    const int b_j = B_RC ? (tid >> 4) : (tid % BN);
    constexpr int B_STEP = B_RC ? NT / 16 : NT / BN;

    const float *pA;
    if (A_RC)
        pA = g.A + (long)(i0 + a_i) * g.sA + a_r;
    else
        pA = g.A + (long)(i0 + a_i);  // the row offset (a_r and the step) is added per fetch

    const float *pB;
    bool b_col_ok = true;
    if (B_RC) {
        pB = g.B + (long)(j0 + b_j) * g.sB + b_r;
    } else {
        unsigned jg = (unsigned)(j0 + b_j), img, n;
        b_col_ok = (int)jg < g.J;
        g.divN.divmod(b_col_ok ? jg : 0u, img, n);
        pB = g.B + (long)img * g.bsB + n;  // the row offset (b_r and the step) is added per fetch
    }

    floatx16 acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int v = 0; v < 16; ++v) acc[a][b][v] = 0.0f;

    // ---- reduction range (steps of BK; in reduction batching a step is (image, r0)) ---
    int step = (int)split * g.steps_per_split;
    int step_end = step + g.steps_per_split;
    if (step_end > g.steps_total) step_end = g.steps_total;
    const int nsteps = step_end - step;
    int img = 0, r_first = step * BK;
    if (RED) {
        unsigned im, st;
        g.divSpi.divmod((unsigned)step, im, st);
        img = (int)im;
        r_first = (int)st * BK;
    }

    float ra[NA], rb[NB];
    int ld_img = img, ld_r0 = r_first;  // position of the next tile to fetch

    auto fetch = [&]() {
        const float *a = pA + (RED ? (long)ld_img * g.rbA : 0L);
        const float *b = pB + (RED ? (long)ld_img * g.rbB : 0L);
#pragma unroll
        for (int q = 0; q < NA; ++q) {
            if (A_RC) {
                bool ok = (i0 + a_i + q * A_STEP < g.M) && (ld_r0 + a_r < g.R);
                ra[q] = ok ? a[(long)(q * A_STEP) * g.sA + ld_r0] : 0.0f;
            } else {
                int r = ld_r0 + a_r + q * A_STEP;
                bool ok = (i0 + a_i < g.M) && (r < g.R);
                ra[q] = ok ? a[(long)r * g.sA] : 0.0f;
            }
        }
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            if (B_RC) {
                bool ok = (j0 + b_j + q * B_STEP < g.J) && (ld_r0 + b_r < g.R);
                rb[q] = ok ? b[(long)(q * B_STEP) * g.sB + ld_r0] : 0.0f;
            } else {
                int r = ld_r0 + b_r + q * B_STEP;
                bool ok = b_col_ok && (r < g.R);
                rb[q] = ok ? b[(long)r * g.sB] : 0.0f;
            }
        }
        ld_r0 += BK;
        if (RED && ld_r0 >= g.R) {
            ld_r0 = 0;
            ++ld_img;
        }
    };

    auto stash = [&](int buf) {
#pragma unroll
        for (int q = 0; q < NA; ++q) {
            if (A_RC)
                As[buf][a_r][a_i + q * A_STEP] = ra[q];
            else
                As[buf][a_r + q * A_STEP][a_i] = ra[q];
        }
#pragma unroll
        for (int q = 0; q < NB; ++q) {
            if (B_RC)
                Bs[buf][b_r][b_j + q * B_STEP] = rb[q];
            else
                Bs[buf][b_r + q * B_STEP][b_j] = rb[q];
        }
    };

    if (nsteps > 0) {
        fetch();
        stash(0);
    }
    __syncthreads();

    const int half = lane >> 5, l32 = lane & 31;
    for (int s = 0; s < nsteps; ++s) {
        const int buf = s & 1;
        if (s + 1 < nsteps) fetch();
        // Operand registers are double buffered: the LDS reads for the next
        // k-pair are issued before the MFMAs of the current one.
        float av[2][TM], bv[2][TN];
#pragma unroll
        for (int a = 0; a < TM; ++a) av[0][a] = As[buf][half][wm * (TM * 32) + a * 32 + l32];
#pragma unroll
        for (int b = 0; b < TN; ++b) bv[0][b] = Bs[buf][half][wn * (TN * 32) + b * 32 + l32];
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            const int cur = (kk >> 1) & 1, nxt = cur ^ 1;
            if (kk + 2 < BK) {
#pragma unroll
                for (int a = 0; a < TM; ++a) av[nxt][a] = As[buf][kk + 2 + half][wm * (TM * 32) + a * 32 + l32];
#pragma unroll
                for (int b = 0; b < TN; ++b) bv[nxt][b] = Bs[buf][kk + 2 + half][wn * (TN * 32) + b * 32 + l32];
            }
            __builtin_amdgcn_sched_barrier(0);  // keep the reads above the MFMAs below
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[cur][a], bv[cur][b], acc[a][b], 0, 0, 0);
        }
        if (s + 1 < nsteps) stash(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue --------------------------------------------------------------
    // Accumulator register v of lane l holds D[8*(v/4) + 4*(l/32) + v%4][l%32].
    const bool partial = g.nsplit > 1;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int jg = j0 + wn * (TN * 32) + b * 32 + l32;
        if (jg >= g.J) continue;
        long coff, moff = jg;
        if (partial) {
            coff = (long)split * g.M * g.J + jg;
        } else if (!RED && (g.N != g.J || g.c_pitch || g.mask_pitch)) {
            unsigned im, n, y, x;
            g.divN.divmod((unsigned)jg, im, n);
            g.divCW.divmod(n, y, x);
            coff = (long)im * g.bsC + (g.c_pitch ? (long)y * g.c_pitch + x : (long)n);
            moff = (long)im * g.mask_bsC + (g.mask_pitch ? (long)y * g.mask_pitch + x : (long)n);
        } else {
            coff = jg;
        }
#pragma unroll
        for (int a = 0; a < TM; ++a) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int i = i0 + wm * (TM * 32) + a * 32 + 8 * (v / 4) + 4 * half + (v % 4);
                if (i >= g.M) continue;
                float val = acc[a][b][v];
                if (partial) {
                    g.ws[coff + (long)i * g.J] = val;
                } else {
                    float *c = g.C + (long)i * g.sC + coff;
                    val *= g.alpha;
                    if (g.bias) val += g.bias[i];
                    if (g.beta != 0.0f) val += g.beta * *c;
                    if (g.act) val = val > g.act_threshold ? val : g.act_value;
                    if (g.mask) val = g.mask[(long)i * g.mask_sC + moff] > g.mask_threshold ? val : 0.0f;
                    *c = val;
                }
            }
        }
    }
}

}  // namespace

int gemm_generic_64x64(const GemmArgs &g, bool a_rc, bool b_rc, bool red, hipStream_t s) {
    dim3 grid(g.total), block(256);
    if (red) {
        if (!(a_rc && b_rc)) return fail("gemm: reduction batching needs r-contiguous operands");
        hipLaunchKernelGGL((gemm_generic_kernel<64, 64, 2, 2, true, true, true>), grid, block, 0, s, g);
    } else if (a_rc && !b_rc)
        hipLaunchKernelGGL((gemm_generic_kernel<64, 64, 2, 2, true, false, false>), grid, block, 0, s, g);
    else if (!a_rc && !b_rc)
        hipLaunchKernelGGL((gemm_generic_kernel<64, 64, 2, 2, false, false, false>), grid, block, 0, s, g);
    else if (a_rc && b_rc)
        hipLaunchKernelGGL((gemm_generic_kernel<64, 64, 2, 2, true, true, false>), grid, block, 0, s, g);
    else
        hipLaunchKernelGGL((gemm_generic_kernel<64, 64, 2, 2, false, true, false>), grid, block, 0, s, g);
    return 0;
}

}  // namespace thgpu

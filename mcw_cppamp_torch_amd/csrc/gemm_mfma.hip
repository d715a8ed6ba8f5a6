// fp32 MFMA GEMM for gfx950.  See gemm_mfma.h for the problem statement.
//
// Tiling: a workgroup of WGM x WGN wavefronts owns a BM x BN tile of C; each
// wavefront owns (BM/WGM) x (BN/WGN) outputs as TM x TN blocks of 32x32, one
// v_mfma_f32_32x32x2_f32 accumulator (16 VGPRs per lane) per block.  The
// reduction runs in steps of BK = 16.  Both operand tiles are staged in LDS
// in reduction-major order, As[r][i] and Bs[r][j], so that the per-lane MFMA
// operand fetch (lane l supplies A[i = l%32][k = l/32], B[k = l/32][j = l%32])
// is a conflict-free ds_read_b32: each half-wave reads 32 consecutive floats.
// LDS is double buffered and the next tile's global loads are issued before
// the current tile's MFMAs, so one barrier per step suffices.
//
// Replaces the four 16x16-tile C++ AMP kernels of the reference
// (gputorch/lib/THC/THCBlas.cpp:10-246).
#include "gemm_mfma.h"

namespace thgpu {

typedef float floatx16 __attribute__((ext_vector_type(16)));

namespace {

constexpr int BK = 16;
constexpr int LDS_PAD = 2;

struct GemmArgs {
    const float *A;
    const float *B;
    float *C;
    const float *bias;
    float *ws;
    int M, J, R, N;
    long sA, sB, sC, bsB, bsC, rbA, rbB;
    int nb, imgs_per_split, nsplit;
    unsigned tilesM, tilesJ, total;
    FastDiv divN, divTilesM, divTilesJ;
    float alpha, beta;
};

// Workgroups are handed to the 8 XCDs round-robin by linear id.  Remap so that
// each XCD walks a contiguous range of tiles: neighbours in that range share
// the same B tile (and the whole of A), which then stays in that XCD's L2.
__device__ inline unsigned xcd_remap(unsigned id, unsigned total) {
    constexpr unsigned XCDS = 8;
    unsigned q = total / XCDS, rem = total % XCDS;
    unsigned xcd = id % XCDS, slot = id / XCDS;
    unsigned base = xcd * q + (xcd < rem ? xcd : rem);
    return base + slot;
}

template <int BM, int BN, int WGM, int WGN, bool A_RC, bool B_RC, bool RED>
__global__ __launch_bounds__(WGM *WGN * 64) void gemm_kernel(const GemmArgs g) {
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

    // ---- reduction range -----------------------------------------------------
    const int steps_per_img = (g.R + BK - 1) / BK;
    int img = 0, img_end = 1;
    if (RED) {
        img = (int)split * g.imgs_per_split;
        img_end = img + g.imgs_per_split;
        if (img_end > g.nb) img_end = g.nb;
    }
    const int nsteps = (img_end - img) * steps_per_img;

    float ra[NA], rb[NB];
    int ld_img = img, ld_r0 = 0;  // position of the next tile to fetch

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
#pragma unroll
        for (int kk = 0; kk < BK; kk += 2) {
            float av[TM], bv[TN];
#pragma unroll
            for (int a = 0; a < TM; ++a) av[a] = As[buf][kk + half][wm * (TM * 32) + a * 32 + l32];
#pragma unroll
            for (int b = 0; b < TN; ++b) bv[b] = Bs[buf][kk + half][wn * (TN * 32) + b * 32 + l32];
#pragma unroll
            for (int a = 0; a < TM; ++a)
#pragma unroll
                for (int b = 0; b < TN; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[a], bv[b], acc[a][b], 0, 0, 0);
        }
        if (s + 1 < nsteps) stash(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue --------------------------------------------------------------
    // Accumulator register v of lane l holds D[8*(v/4) + 4*(l/32) + v%4][l%32].
    const bool partial = RED && g.nsplit > 1;
#pragma unroll
    for (int b = 0; b < TN; ++b) {
        const int jg = j0 + wn * (TN * 32) + b * 32 + l32;
        if (jg >= g.J) continue;
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
                if (i >= g.M) continue;
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

// C(i,j) = beta*C(i,j) + alpha * sum_s ws[s][i][j], s ascending.
__global__ void split_reduce_kernel(const float *__restrict__ ws, float *__restrict__ C, int M, int J, long sC,
                                    int nsplit, float alpha, float beta) {
    long idx = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long total = (long)M * J;
    if (idx >= total) return;
    float sum = 0.0f;
    for (int s = 0; s < nsplit; ++s) sum += ws[(long)s * total + idx];
    long i = idx / J, j = idx - i * J;
    float *c = C + i * sC + j;
    float val = alpha * sum;
    if (beta != 0.0f) val += beta * *c;
    *c = val;
}

template <int BM, int BN, int WGM, int WGN>
int launch_cfg(const GemmProblem &p, GemmArgs &g, hipStream_t s) {
    g.tilesM = (unsigned)((p.M + BM - 1) / BM);
    g.tilesJ = (unsigned)((p.J + BN - 1) / BN);
    g.divTilesM = FastDiv(g.tilesM);
    g.divTilesJ = FastDiv(g.tilesJ);
    const bool red = p.nb > 1;
    g.nsplit = 1;
    g.imgs_per_split = p.nb;
    if (red) {
        // Enough workgroups to fill the chip a few times over, whole images per split.
        long tiles = (long)g.tilesM * g.tilesJ;
        long want = (4L * num_cus() + tiles - 1) / tiles;
        if (want < 1) want = 1;
        if (want > p.nb) want = p.nb;
        g.imgs_per_split = (int)((p.nb + want - 1) / want);
        g.nsplit = (p.nb + g.imgs_per_split - 1) / g.imgs_per_split;
        if (g.nsplit > 1) {
            g.ws = workspace(sizeof(float) * (size_t)g.nsplit * p.M * p.J);
            if (!g.ws) return 1;
        }
    }
    long total = (long)g.tilesM * g.tilesJ * g.nsplit;
    if (total <= 0 || total >= (1L << 31)) return fail("gemm: tile count %ld out of range", total);
    g.total = (unsigned)total;
    dim3 grid(g.total), block(WGM * WGN * 64);
    {
        LaunchScope scope(p.tag, 2.0 * p.M * p.J * (double)p.R * (red ? p.nb : 1), 0.0);
        if (red)
            hipLaunchKernelGGL((gemm_kernel<BM, BN, WGM, WGN, true, true, true>), grid, block, 0, s, g);
        else if (p.a_rc && !p.b_rc)
            hipLaunchKernelGGL((gemm_kernel<BM, BN, WGM, WGN, true, false, false>), grid, block, 0, s, g);
        else if (!p.a_rc && !p.b_rc)
            hipLaunchKernelGGL((gemm_kernel<BM, BN, WGM, WGN, false, false, false>), grid, block, 0, s, g);
        else if (p.a_rc && p.b_rc)
            hipLaunchKernelGGL((gemm_kernel<BM, BN, WGM, WGN, true, true, false>), grid, block, 0, s, g);
        else
            hipLaunchKernelGGL((gemm_kernel<BM, BN, WGM, WGN, false, true, false>), grid, block, 0, s, g);
    }
    if (check_launch(p.tag)) return 1;
    if (red && g.nsplit > 1) {
        long n = (long)p.M * p.J;
        {
            LaunchScope scope("gemm_split_reduce", 0.0, 4.0 * n * (g.nsplit + 2));
            hipLaunchKernelGGL(split_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, g.ws, p.C,
                               p.M, p.J, p.sC, g.nsplit, p.alpha, p.beta);
        }
        if (check_launch("gemm_split_reduce")) return 1;
    }
    return 0;
}

long padded(long x, long t) { return (x + t - 1) / t * t; }

}  // namespace

int gemm_launch(const GemmProblem &p) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (p.M <= 0 || p.J <= 0) return 0;
    if ((long)p.M * p.J >= (1L << 31) && p.N == p.J) return fail("gemm: output too large for 32-bit tile indexing");

    GemmArgs g{};
    g.A = p.A;
    g.B = p.B;
    g.C = p.C;
    g.bias = p.bias;
    g.ws = nullptr;
    g.M = p.M;
    g.J = p.J;
    g.R = p.R;
    g.N = p.N > 0 ? p.N : p.J;
    g.sA = p.sA;
    g.sB = p.sB;
    g.sC = p.sC;
    g.bsB = p.bsB;
    g.bsC = p.bsC;
    g.rbA = p.rbA;
    g.rbB = p.rbB;
    g.nb = p.nb;
    g.divN = FastDiv((uint32_t)g.N);
    g.alpha = p.alpha;
    g.beta = p.beta;

    // Tile shape: least padded work; ties go to the squarer, larger tile.
    const long w128 = padded(p.M, 128) * padded(p.J, 128);
    const long w64x256 = padded(p.M, 64) * padded(p.J, 256);
    const long w64 = padded(p.M, 64) * padded(p.J, 64);
    const long tiles128 = (padded(p.M, 128) / 128) * (padded(p.J, 128) / 128);
    if (w64 < w128 && w64 < w64x256 && (w64 * 10 < w128 * 9 || tiles128 < 2L * num_cus()))
        return launch_cfg<64, 64, 2, 2>(p, g, s);
    if (w64x256 < w128) return launch_cfg<64, 256, 1, 4>(p, g, s);
    return launch_cfg<128, 128, 2, 2>(p, g, s);
}

}  // namespace thgpu

using namespace thgpu;

extern "C" void THGPUBlas_gemm(char transa, char transb, long m, long n, long k, float alpha, float *a, long lda,
                               float *b, long ldb, float beta, float *c, long ldc) {
    const bool ta = (transa == 't' || transa == 'T');
    const bool tb = (transb == 't' || transb == 'T');
    // Quick returns of the reference dispatcher (gputorch/lib/THC/THCBlas.cpp:257).
    if (!m || !n || ((alpha == 0 || !k) && beta == 1)) return;
    // Degenerate leading dimensions as TH fixes them up (TH/generic/THBlas.c:275-298).
    if (n == 1) ldc = m;
    if (ta) {
        if (m == 1) lda = k;
    } else {
        if (k == 1) lda = m;
    }
    if (tb) {
        if (k == 1) ldb = n;
    } else {
        if (n == 1) ldb = k;
    }
    if (m >= (1L << 31) || n >= (1L << 31) || k >= (1L << 31)) {
        raise("THGPUBlas_gemm: dimension exceeds 2^31");
        return;
    }
    // Column-major C(m x n) is the row-major n x m matrix C'(i', j') =
    // c[j' + i'*ldc]; C' = op(B)' * op(A)' with
    //   A'(i', r) = op(B)(r, i'),  B'(r, j') = op(A)(j', r).
    GemmProblem p;
    p.A = b;
    p.B = a;
    p.C = c;
    p.M = (int)n;
    p.J = (int)m;
    p.R = alpha == 0 ? 0 : (int)k;  // empty sum: C = beta*C, whatever A and B hold
    p.N = (int)m;
    p.a_rc = !tb;  // 'n': b[r + i'*ldb]
    p.sA = ldb;
    p.b_rc = ta;  // 't': a[r + j'*lda]
    p.sB = lda;
    p.sC = ldc;
    p.alpha = alpha;
    p.beta = beta;
    p.tag = "gemm_blas";
    if (gemm_launch(p)) raise("%s", thgpu_last_error());
}

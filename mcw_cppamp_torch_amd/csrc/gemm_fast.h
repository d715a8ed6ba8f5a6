// The fast fp32 MFMA GEMM kernel (see gemm_mfma.h for the problem statement).
// Included by one small translation unit per tile configuration.
//
// Structure
//   * A workgroup of WGM x WGN wavefronts owns a BM x BN tile of C, each
//     wavefront TM x TN blocks of 32x32 outputs, one v_mfma_f32_32x32x2_f32
//     accumulator (16 registers per lane) per block.
//   * No bounds checks and no branches around loads.  A tile at the lower/right
//     edge is shifted back so that it lies inside the matrix and stores only the
//     rows/columns no other tile owns; a reduction step that would run past R is
//     shifted back to end at R and the part the previous step already covered
//     is zeroed on its way to LDS.  Needs M >= BM, J >= BN, R >= 16; smaller
//     problems take the bounds-checked generic kernel.
//   * LDS holds both operand tiles as [x][r] (x the free index, r the
//     reduction index).  Each lane fetches its MFMA operands with 128-bit LDS
//     reads: lane (x, h) reads r = 8h .. 8h+7, and MFMA step s takes r = s from
//     the lower half-wave and r = 8 + s from the upper one.  A and B use the
//     same permutation of r, so the sum over r is unchanged.  The row layout
//     follows the operand's loader, so that its 128-bit LDS writes and the
//     operand reads are both free of bank conflicts (the LDS conflict counter
//     reads zero for either): a tile written a column at a time (consecutive
//     lanes = consecutive rows) has rows of 16 + 4 floats; a tile written a row
//     at a time (four lanes per row) has rows of 16 floats whose four 16-byte
//     quarters are stored at quarter (r/4) xor ((x/4) mod 4).
//   * LDS is double buffered; the next tile's global loads are issued between
//     the current tile's MFMAs and written to the other buffer afterwards: one
//     barrier per reduction step.
//   * Two variants for row counts the 32-row blocks fit badly: ROWS16 (16x16 blocks over the first 48 rows of a
//     64-row tile, scattered products only) and the 96-row tile, whose first-operand loads the threads do not divide.
//   * Between the MFMAs of a step there are memory and scalar instructions only.
//     fp32 MFMAs and ordinary vector instructions share the SIMD's ALU (a v_add
//     between two MFMAs costs 6 to 13 cycles of matrix time, measured), and a
//     wavefront with MFMAs to issue keeps the other wavefronts of its SIMD from
//     issuing anything, so nothing the loop does is hidden by another wavefront:
//     operands are fetched with buffer loads (descriptor and offsets in scalar
//     registers, a constant lane offset), and the loop is unrolled by two so
//     that the LDS buffer folds into the offset field of the LDS instructions.
#pragma once

#include <type_traits>

#include "gemm_mfma.h"

namespace thgpu {

// Loader kind used inside the kernel only: an x-contiguous first operand whose row count the thread
// count does not divide (192 rows, 256 threads).  Wavefront w takes r = 4w .. 4w+3 of every block of
// 64 consecutive rows; lanes run along the rows.
constexpr int LD_XC_BLOCK = 3;

// LDS row layout by loader kind: pitch in floats, and the column at which element r of row x is stored.
//
// Measured on this hardware with eight wavefronts issuing nothing else: a conflict-free ds_read_b128 takes 4 cycles
// per wavefront and is served sixteen lanes at a time, where the sixteen are lanes 0-3, 12-15, 20-23, 24-27, then
// 4-7, 8-11, 16-19, 28-31 (likewise in the upper half-wave), over 64 banks; a ds_write_b128 is served eight
// consecutive lanes at a time, whose 16-byte units must differ modulo 128 bytes.  Hence:
//   * 32x32 blocks (lane l reads row l%32, quarter pair l/32): rows written a column at a time (consecutive lanes =
//     consecutive rows) are padded to 20 floats; rows written four lanes to a row keep 16 floats, quarter q of row x
//     stored at q xor (x/4)%4.  Reads and writes of both are conflict-free (the conflict counter reads zero).
//   * 16x16 blocks (SMALL16: lane l reads row l%16, quarter l/16): the row-written tile stores quarter q of row x
//     at p(q) xor (x/4)%4 with p = (0, 3, 1, 2), conflict-free both ways (the plain xor puts rows 0-3 and rows 4-7
//     of two lane quarters on the same banks).  The column-written tile keeps its 20-float rows: its writes need
//     an odd pitch in 16-byte units, and no placement of four quarters in such a row also frees these reads of
//     conflicts; they take 8 cycles instead of 4, two of a step's five operand reads.
template <int KIND, bool SMALL16 = false>
struct LdsRow {
    static constexpr bool kSwizzled = KIND == LD_RC_VEC;
    static constexpr int kPitch = kSwizzled ? GEMM_BK : GEMM_BK + 4;
    __device__ static __forceinline__ int col(int x, int r) {
        if (!kSwizzled) return r;
        const int q = SMALL16 ? (0x9C >> (2 * (r >> 2))) & 3 : r >> 2;
        return (r & 3) | (((q ^ (x >> 2)) & 3) << 2);
    }
};

// Four floats at a 4-byte aligned address: the hardware handles the
// misalignment of a 128-bit global load; the type only keeps the compiler from
// assuming 16-byte alignment.
struct __attribute__((packed, aligned(4))) float4u {
    float x, y, z, w;
};

// Wavefronts per SIMD the register allocation must leave room for: the
// accumulators take (BM/WGM)*(BN/WGN)/64 registers of the 512 a lane has.
template <int BM, int BN, int WGM, int WGN>
constexpr int gemm_min_waves() {
    return (BM / WGM) * (BN / WGN) / 64 >= 96 ? 2 : 3;
}

// ROWS16 > 0 selects the short-row variant: the workgroup still loads BM = 64 rows of the first operand, but its
// wavefronts multiply only the first 16*ROWS16 of them, in 16x16 blocks (v_mfma_f32_16x16x4_f32, four registers per
// lane and block).  It exists for scattered products whose row count is 48 (three planes at stride 4 x 4), which
// would otherwise spend a quarter of their MFMAs on padding; it has the scattered store only.
template <int BM, int BN, int WGM, int WGN, int LA, int LB, bool RED, int ROWS16 = 0>
__global__ __launch_bounds__(WGM *WGN * 64)
    __attribute__((amdgpu_waves_per_eu(gemm_min_waves<BM, BN, WGM, WGN>()))) void gemm_fast_kernel(const GemmArgs g) {
    constexpr int NT = WGM * WGN * 64;
    constexpr int BK = GEMM_BK;
    constexpr bool SMALL = ROWS16 > 0;
    constexpr int TM = SMALL ? ROWS16 : BM / WGM / 32, TN = SMALL ? BN / WGN / 16 : BN / WGN / 32;
    static_assert(!SMALL || (WGM == 1 && BM == 64 && ROWS16 <= 4 && LB == LD_XC_GATHER && !RED && TN % 2 == 0),
                  "the short-row variant: one row of wavefronts over a 64-row tile, gathered B, scattered store");
    // A first operand along r whose 128-bit loads the threads do not divide (96 rows: 384 loads, 256 threads): the
    // last round of loads is made by the leading wavefronts only (a uniform branch; wavefront w loads rows
    // 16w .. 16w+15 of every 64).
    constexpr bool PART_A = LA == LD_RC_VEC && (BM * BK) % (NT * 4) != 0;
    constexpr int NA = PART_A ? (BM * BK + NT * 4 - 1) / (NT * 4) * 4 : BM * BK / NT, NB = BN * BK / NT;
    static_assert(!PART_A || (NT == 256 && BM % 16 == 0), "partial loader shape");
    static_assert(BM % (WGM * 32) == 0 && BN % (WGN * 32) == 0, "wave tile must be whole 32x32 blocks");
    static_assert(NT % 16 == 0 && NA >= 4 && NB >= 4 && NA % 4 == 0 && NB % 4 == 0, "loader shape");
    // The kind the A loader really uses: x-contiguous with 192 rows goes block-wise.
    constexpr int KA = (LA == LD_XC_SCALAR && NT % BM != 0) ? LD_XC_BLOCK : LA;
    static_assert(KA != LD_XC_BLOCK || (NT == 256 && BM % 64 == 0 && NA == BM / 16), "block loader shape");
    static_assert((LB != LD_XC_SCALAR && LB != LD_XC_GATHER) || NT % BN == 0,
                  "x-contiguous loaders give every thread one row/column");
    static_assert(LB != LD_XC_GATHER || BN % 64 == 0, "a wavefront of the gathering loader shares its reduction indices");
    static_assert(LA != LD_XC_GATHER, "only the second operand is gathered");
    static_assert(!RED || (LA != LD_XC_SCALAR && LB != LD_XC_SCALAR),
                  "reduction batching needs r-contiguous or gathered operands");

    using RowA = LdsRow<KA, SMALL>;
    using RowB = LdsRow<LB, SMALL>;
    __shared__ __attribute__((aligned(16))) float As[2][BM][RowA::kPitch];
    __shared__ __attribute__((aligned(16))) float Bs[2][BN][RowB::kPitch];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // scalar: row bases stay uniform
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
    // Thread -> (x, r) of its first element inside an operand tile:
    //   LD_RC_VEC     x = tid/4 (+64 per load), r = 4*(tid%4) .. +3   (one 128-bit load each)
    //   LD_RC_SCALAR  x = tid/16 (+16 per load), r = tid%16
    //   LD_XC_SCALAR  x = tid % X, r = (tid / X) * CNT .. + CNT-1     (CNT loads down the column)
    //   LD_XC_BLOCK   x = lane (+64 per block of rows), r = 4*wave .. +3
    // A load address is a wave-uniform base (tile, image, step, load number: all
    // scalar) plus a per-thread byte offset that never changes, so the loop
    // spends no vector ALU work on addressing.
    int a_x, a_r, b_x, b_r;
    unsigned voffA, voffB;
    const char *tileA, *tileB;
    if (KA == LD_XC_BLOCK) {
        a_x = lane;
        a_r = 4 * wave;
        voffA = (unsigned)(((long)a_r * g.sA + a_x) * 4);
        tileA = reinterpret_cast<const char *>(g.A + i0);
    } else if (LA == LD_XC_SCALAR) {
        a_x = tid % BM;
        a_r = (tid / BM) * NA;
        voffA = (unsigned)(((long)a_r * g.sA + a_x) * 4);
        tileA = reinterpret_cast<const char *>(g.A + i0);
    } else {
        a_x = LA == LD_RC_VEC ? tid >> 2 : tid >> 4;
        a_r = LA == LD_RC_VEC ? (tid & 3) * 4 : tid & 15;
        voffA = (unsigned)(((long)a_x * g.sA + a_r) * 4);
        tileA = reinterpret_cast<const char *>(g.A + (long)i0 * g.sA);
    }
    if (LB == LD_XC_GATHER) {
        b_x = tid % BN;
        b_r = (wave * 64 / BN) * NB;  // = (tid / BN) * NB, kept uniform: the row offsets are scalar loads
        unsigned img0, n0, img, n;
        g.divN.divmod((unsigned)j0, img0, n0);
        g.divN.divmod((unsigned)(j0 + b_x), img, n);
        voffB = (unsigned)(((long)(img - img0) * g.bsB + g.coltab[n]) * 4);
        tileB = reinterpret_cast<const char *>(g.B + (long)img0 * g.bsB);
    } else if (LB == LD_XC_SCALAR) {
        b_x = tid % BN;
        b_r = (tid / BN) * NB;
        unsigned img0, n0, img, n;
        g.divN.divmod((unsigned)j0, img0, n0);
        g.divN.divmod((unsigned)(j0 + b_x), img, n);
        voffB = (unsigned)(((long)b_r * g.sB + (long)(img - img0) * g.bsB + n) * 4);
        tileB = reinterpret_cast<const char *>(g.B + (long)img0 * g.bsB);
    } else {
        b_x = LB == LD_RC_VEC ? tid >> 2 : tid >> 4;
        b_r = LB == LD_RC_VEC ? (tid & 3) * 4 : tid & 15;
        voffB = (unsigned)(((long)b_x * g.sB + b_r) * 4);
        tileB = reinterpret_cast<const char *>(g.B + (long)j0 * g.sB);
    }
    constexpr int UA = LA == LD_RC_VEC ? NA / 4 : NA;  // load instructions per step and operand
    constexpr int UB = LB == LD_RC_VEC ? NB / 4 : NB;

    // One accumulator per block: 16 registers (32x32 blocks) or 4 (16x16 blocks of the short-row variant).
    using Acc = std::conditional_t<SMALL, floatx4, floatx16>;
    constexpr int ACCV = SMALL ? 4 : 16;
    Acc acc[TM][TN];
#pragma unroll
    for (int a = 0; a < TM; ++a)
#pragma unroll
        for (int b = 0; b < TN; ++b)
#pragma unroll
            for (int v = 0; v < ACCV; ++v) acc[a][b][v] = 0.0f;

    // Row sums of the first operand (GemmProblem::rowsum), reduction batching only.  The column tiles of a row of
    // tiles all load the same first-operand tiles, so they share the work: the workgroup of column tile tj sums the
    // steps whose index is tj modulo the number of column tiles, from the MFMA operands its first column of
    // wavefronts holds in registers anyway (lane (x, h) holds r = 8h .. 8h+7 of row x).  A handful of vector adds
    // every tilesJ-th step; the partial sums go to rowsum_ws[row][split * tilesJ + tj].
    float bsum[TM];
#pragma unroll
    for (int a = 0; a < TM; ++a) bsum[a] = 0.0f;
    const bool rs_on = RED && !SMALL && g.rowsum_ws != nullptr && wn == 0;
    int rs_next = 0;
    if (rs_on) rs_next = (int)(((unsigned)tj + g.tilesJ - (unsigned)step % g.tilesJ) % g.tilesJ);

    float ra[NA], rb[NB];
    auto a_unit_live = [&](int u) { return !PART_A || u * (NT / 4) + 16 * wave < BM; };
    auto always_live = [](int) { return true; };
    if (PART_A) {
#pragma unroll
        for (int q = 0; q < NA; ++q) ra[q] = 0.0f;
    }
    // Gathered B: float offsets of the rows of the step being loaded (uniform), and of the step after it.  The
    // latter are fetched (scalar loads) in the middle of a step, a whole step before they turn into addresses,
    // so that no step starts by waiting for its row offsets.
    int roff[LB == LD_XC_GATHER ? NB : 1], roff_nx[LB == LD_XC_GATHER ? NB : 1];

    // Load number u of an operand for the step whose uniform base is `base`.  Buffer loads: the address is a
    // descriptor in scalar registers (the step's base) plus a scalar offset (which load) plus the lane's constant
    // 32-bit offset, so the loop spends no vector ALU instruction on addressing.  That matters more than its
    // instruction count suggests: fp32 MFMAs and ordinary vector instructions share the SIMD's ALU (a v_add
    // between two MFMAs costs 6 to 13 cycles of matrix-pipe time, measured), while scalar instructions and the
    // issue of memory instructions run beside the matrix pipe.
    typedef float float4v __attribute__((ext_vector_type(4)));
    auto descriptor = [](const char *base) {
        // raw buffer, no bounds (every offset below 2^32 passes), dword format
        return __builtin_amdgcn_make_buffer_rsrc(const_cast<char *>(base), 0, -1, 0x00020000);
    };
    auto load_unit = [&](auto kind_tag, const char *base, long stride, unsigned voff, float *dst, int u) {
        constexpr int KIND = decltype(kind_tag)::value;
        const __amdgpu_buffer_rsrc_t rsrc = descriptor(base);
        const int st = (int)stride * 4;
        if (KIND == LD_RC_VEC) {
            const float4v v = __builtin_bit_cast(
                float4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)voff, u * (NT / 4) * st, 0));
            dst[u * 4 + 0] = v.x;
            dst[u * 4 + 1] = v.y;
            dst[u * 4 + 2] = v.z;
            dst[u * 4 + 3] = v.w;
        } else {
            const int so = KIND == LD_RC_SCALAR  ? u * (NT / 16) * st
                           : KIND == LD_XC_BLOCK ? (u & 3) * st + (u >> 2) * 256
                           : KIND == LD_XC_GATHER ? roff[u] * 4
                                                  : u * st;
            dst[u] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(rsrc, (int)voff, so, 0));
        }
    };

    // Uniform bases of the step at (ld_img, ld_r0).  A step that would run past
    // R is moved back to end at R (every address stays inside the operand;
    // needs R >= BK); `shift` says how many of its leading reduction indices the
    // previous step already covered -- those are zeroed before they reach LDS.
    auto step_bases = [&](const char *&ga, const char *&gb, int &shift) {
        const int r0 = ld_r0 + BK <= g.R ? ld_r0 : g.R - BK;
        shift = ld_r0 - r0;
        ga = tileA + ((RED ? (long)ld_img * g.rbA : 0L) + (LA == LD_XC_SCALAR ? (long)r0 * g.sA : (long)r0)) * 4;
        if (LB == LD_XC_GATHER) {
            gb = tileB + (RED ? (long)ld_img * g.rbB : 0L) * 4;
#pragma unroll
            for (int u = 0; u < NB; ++u) roff[u] = roff_nx[u];
        } else {
            gb = tileB + ((RED ? (long)ld_img * g.rbB : 0L) + (LB == LD_XC_SCALAR ? (long)r0 * g.sB : (long)r0)) * 4;
        }
    };
    // Row offsets of the step whose reduction window starts at `pos` (moved back like the step itself).
    auto fetch_rows = [&](int pos) {
        if (LB == LD_XC_GATHER) {
            const int r0 = pos + BK <= g.R ? pos : g.R - BK;
            const int *rt = g.rowtab + r0 + b_r;
#pragma unroll
            for (int u = 0; u < NB; ++u) roff_nx[u] = rt[u];
        }
    };
    // Takes delivery of them (an empty statement that names the values keeps the compiler from postponing the
    // loads to the point of first use).
    auto pin_rows = [&]() {
        if (LB == LD_XC_GATHER) {
#pragma unroll
            for (int u = 0; u < NB; ++u) {
                int t = __builtin_amdgcn_readfirstlane(roff_nx[u]);
                asm("" : "+s"(t));
                roff_nx[u] = t;
            }
        }
    };
    auto advance = [&]() {
        ld_r0 += BK;
        if (RED && ld_r0 >= g.R) {
            ld_r0 = 0;
            ++ld_img;
        }
    };
    // Zero the elements whose position inside the step window is below `shift`.
    auto mask_one = [&](auto kind_tag, int t_r, float *v, auto count_tag, int shift) {
        constexpr int KIND = decltype(kind_tag)::value;
        constexpr int CNT = decltype(count_tag)::value;
#pragma unroll
        for (int q = 0; q < CNT; ++q) {
            const int rel = (KIND == LD_RC_VEC || KIND == LD_XC_BLOCK) ? t_r + (q & 3)
                            : KIND == LD_RC_SCALAR                          ? t_r
                                                                            : t_r + q;
            v[q] = rel < shift ? 0.0f : v[q];
        }
    };

    auto stash_one = [&](auto kind_tag, auto tile, int t_x, int t_r, const float *src, auto count_tag, auto live) {
        constexpr int KIND = decltype(kind_tag)::value;
        using Row = LdsRow<KIND, SMALL>;
        constexpr int CNT = decltype(count_tag)::value;
        if (KIND == LD_RC_VEC) {
#pragma unroll
            for (int q = 0; q < CNT / 4; ++q)
                if (live(q))
                    *reinterpret_cast<float4 *>(&tile[t_x + q * (NT / 4)][Row::col(t_x + q * (NT / 4), t_r)]) =
                        make_float4(src[q * 4], src[q * 4 + 1], src[q * 4 + 2], src[q * 4 + 3]);
        } else if (KIND == LD_RC_SCALAR) {
#pragma unroll
            for (int q = 0; q < CNT; ++q) tile[t_x + q * (NT / 16)][Row::col(t_x + q * (NT / 16), t_r)] = src[q];
        } else if (KIND == LD_XC_BLOCK) {
#pragma unroll
            for (int w = 0; w < CNT / 4; ++w)
                *reinterpret_cast<float4 *>(&tile[t_x + 64 * w][Row::col(t_x + 64 * w, t_r)]) =
                    make_float4(src[w * 4], src[w * 4 + 1], src[w * 4 + 2], src[w * 4 + 3]);
        } else {
#pragma unroll
            for (int w = 0; w < CNT / 4; ++w)
                *reinterpret_cast<float4 *>(&tile[t_x][Row::col(t_x, t_r + 4 * w)]) =
                    make_float4(src[w * 4], src[w * 4 + 1], src[w * 4 + 2], src[w * 4 + 3]);
        }
    };
    auto stash = [&](int buf, int shift) {
        if (shift > 0) {  // uniform: only the last step of an image can be partial
            mask_one(std::integral_constant<int, KA>{}, a_r, ra, std::integral_constant<int, NA>{}, shift);
            mask_one(std::integral_constant<int, LB>{}, b_r, rb, std::integral_constant<int, NB>{}, shift);
        }
        stash_one(std::integral_constant<int, KA>{}, As[buf], a_x, a_r, ra, std::integral_constant<int, NA>{}, a_unit_live);
        stash_one(std::integral_constant<int, LB>{}, Bs[buf], b_x, b_r, rb, std::integral_constant<int, NB>{}, always_live);
    };

    // ---- prologue: first step ---------------------------------------------------------
    const char *ga = tileA, *gb = tileB;
    int shift = 0;
    if (nsteps > 0) {
        fetch_rows(ld_r0);
        step_bases(ga, gb, shift);
#pragma unroll
        for (int u = 0; u < UA; ++u)
            if (a_unit_live(u)) load_unit(std::integral_constant<int, KA>{}, ga, g.sA, voffA, ra, u);
#pragma unroll
        for (int u = 0; u < UB; ++u) load_unit(std::integral_constant<int, LB>{}, gb, g.sB, voffB, rb, u);
        stash(0, shift);
        advance();
        fetch_rows(ld_r0);
    }
    __syncthreads();

    // ---- main loop ----------------------------------------------------------------------
    // Step s computes from LDS buffer s&1 while the loads of step s+1 are issued
    // in slices between its MFMAs (a steady trickle of requests; a burst at the
    // head of the step would hold the wavefront, and with it its MFMAs, in the
    // memory pipeline's queue) and written to the other buffer afterwards.
    // Two steps per trip, one per LDS buffer, so that the buffer is a compile-time constant and folds into the
    // offset field of every LDS instruction instead of costing vector adds per step.
    auto one_step = [&](auto buf_tag, int s) {
        constexpr int buf = decltype(buf_tag)::value;
        const bool more = s + 1 < nsteps;
        const bool rs_hit = rs_on && s == rs_next;  // uniform
        if (rs_hit) rs_next += (int)g.tilesJ;
        // The last step has nothing to fetch; it re-reads the previous addresses
        // (valid, cached) rather than branching around the loads.
        if (more) step_bases(ga, gb, shift);

        // What every slice of a step does besides its MFMAs: its share of the next step's loads, and the row
        // offsets of the step after that (requested once every LDS operand of this step has arrived, so that the
        // scalar loads share the wait counter with no outstanding LDS read; taken delivery of two slices later,
        // still under this step's MFMAs).
        constexpr int SLICES = 8;
        auto slice_tail = [&](auto slice_tag) {
            constexpr int slice = decltype(slice_tag)::value;
#pragma unroll
            for (int u = 0; u < UA; ++u)
                if (u * SLICES / UA == slice && a_unit_live(u))
                    load_unit(std::integral_constant<int, KA>{}, ga, g.sA, voffA, ra, u);
#pragma unroll
            for (int u = 0; u < UB; ++u)
                if (u * SLICES / UB == slice) load_unit(std::integral_constant<int, LB>{}, gb, g.sB, voffB, rb, u);
            if (slice == 5) {
                int pos = ld_r0 + BK;
                if (RED && pos >= g.R) pos = 0;
                fetch_rows(pos);
            }
            if (!RED && slice == 7) pin_rows();
            __builtin_amdgcn_sched_barrier(0);
        };
        auto component = [](const float4 &v, int e) { return e == 0 ? v.x : e == 1 ? v.y : e == 2 ? v.z : v.w; };

        if constexpr (SMALL) {
            // 16x16 blocks: lane (x, q) reads r = 4q .. 4q+3 of its row and column with one 128-bit read each, and
            // MFMA e takes r = 4q + e from quarter-wave q.
            const int q4 = lane >> 4, l16 = lane & 15;
            float4 av[TM], bv[TN];
#pragma unroll
            for (int a = 0; a < TM; ++a)
                av[a] = *reinterpret_cast<const float4 *>(&As[buf][a * 16 + l16][RowA::col(l16, 4 * q4)]);
#pragma unroll
            for (int b = 0; b < TN; ++b)
                bv[b] = *reinterpret_cast<const float4 *>(&Bs[buf][wn * (TN * 16) + b * 16 + l16][RowB::col(l16, 4 * q4)]);
            auto half_slice = [&](auto e_tag, auto bh_tag) {
                constexpr int e = decltype(e_tag)::value, bh = decltype(bh_tag)::value;
#pragma unroll
                for (int a = 0; a < TM; ++a)
#pragma unroll
                    for (int b = bh * (TN / 2); b < (bh + 1) * (TN / 2); ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x4f32(component(av[a], e), component(bv[b], e),
                                                                         acc[a][b], 0, 0, 0);
                slice_tail(std::integral_constant<int, e * 2 + bh>{});
            };
            using std::integral_constant;
            half_slice(integral_constant<int, 0>{}, integral_constant<int, 0>{});
            half_slice(integral_constant<int, 0>{}, integral_constant<int, 1>{});
            half_slice(integral_constant<int, 1>{}, integral_constant<int, 0>{});
            half_slice(integral_constant<int, 1>{}, integral_constant<int, 1>{});
            half_slice(integral_constant<int, 2>{}, integral_constant<int, 0>{});
            half_slice(integral_constant<int, 2>{}, integral_constant<int, 1>{});
            half_slice(integral_constant<int, 3>{}, integral_constant<int, 0>{});
            half_slice(integral_constant<int, 3>{}, integral_constant<int, 1>{});
        } else {
            // MFMA operands: 8 reduction indices per lane and block, two 128-bit reads.
            float4 av[TM][2], bv[TN][2];
#pragma unroll
            for (int h2 = 0; h2 < 2; ++h2) {
#pragma unroll
                for (int a = 0; a < TM; ++a)
                    av[a][h2] = *reinterpret_cast<const float4 *>(
                        &As[buf][wm * (TM * 32) + a * 32 + l32][RowA::col(l32, 8 * half + 4 * h2)]);
#pragma unroll
                for (int b = 0; b < TN; ++b)
                    bv[b][h2] = *reinterpret_cast<const float4 *>(
                        &Bs[buf][wn * (TN * 32) + b * 32 + l32][RowB::col(l32, 8 * half + 4 * h2)]);
            }
            auto slice_of = [&](auto slice_tag) {
                constexpr int slice = decltype(slice_tag)::value;
                constexpr int h2 = slice / 4, e = slice % 4;
#pragma unroll
                for (int a = 0; a < TM; ++a)
#pragma unroll
                    for (int b = 0; b < TN; ++b)
                        acc[a][b] = __builtin_amdgcn_mfma_f32_32x32x2f32(component(av[a][h2], e), component(bv[b][h2], e),
                                                                         acc[a][b], 0, 0, 0);
                if constexpr (RED && (slice == 3 || slice == 7)) {
                    if (rs_hit) {
#pragma unroll
                        for (int a = 0; a < TM; ++a)
                            bsum[a] += (av[a][h2].x + av[a][h2].y) + (av[a][h2].z + av[a][h2].w);
                    }
                }
                slice_tail(slice_tag);
            };
            using std::integral_constant;
            slice_of(integral_constant<int, 0>{});
            slice_of(integral_constant<int, 1>{});
            slice_of(integral_constant<int, 2>{});
            slice_of(integral_constant<int, 3>{});
            slice_of(integral_constant<int, 4>{});
            slice_of(integral_constant<int, 5>{});
            slice_of(integral_constant<int, 6>{});
            slice_of(integral_constant<int, 7>{});
        }
        if (more) {
            stash(buf ^ 1, shift);
            advance();
        }
        __syncthreads();
    };
    for (int s = 0; s < nsteps; s += 2) {
        one_step(std::integral_constant<int, 0>{}, s);
        if (s + 1 < nsteps) one_step(std::integral_constant<int, 1>{}, s + 1);
    }

    // ---- epilogue ----------------------------------------------------------------------
    // Accumulator register v of lane l holds D[8*(v/4) + 4*(l/32) + v%4][l%32].
    // A store address is a wave-uniform row base plus a constant per-lane byte
    // offset (column, image and the lane half's four rows), as for the loads.
    // MODE 0: partial sums to the workspace; 1: alpha*acc (+bias); 2: also + beta*C.
    const bool edge_tile = i0 != own_i0 || j0 != own_j0;  // an edge tile: some rows or columns belong to its neighbour
    auto write_out = [&](auto mode_tag, auto check_tag) {
        constexpr int MODE = decltype(mode_tag)::value;
        constexpr bool CHECK = decltype(check_tag)::value;
        const long row_bytes = (MODE == 0 ? (long)g.J : g.sC) * 4;
        char *const out0 = MODE == 0 ? reinterpret_cast<char *>(g.ws + (long)split * g.M * g.J)
                                     : reinterpret_cast<char *>(g.C);
        // Fused threshold / mask of the final value (uniform conditions; both off for partial sums).
        const bool act = MODE != 0 && g.act != 0;
        const bool masked = MODE != 0 && g.mask != nullptr;
        const long mask_row_bytes = g.mask_sC * 4;
        unsigned img0 = 0, n0 = 0;
        // columns are (image, position) pairs, or positions of an image plane whose rows are kept apart
        const bool twin = MODE != 0 && !RED && g.C2 != nullptr;  // a second copy of the result (GemmProblem::C2)
        const long twin_row_bytes = g.c2_sC * 4;
        const bool per_image = MODE != 0 && !RED && (g.N != g.J || g.c_pitch != 0 || g.mask_pitch != 0 || twin);
        if (per_image) g.divN.divmod((unsigned)j0, img0, n0);
        char *const out = out0 + (per_image ? (long)img0 * g.bsC : (long)j0) * 4;
        const char *const msk = reinterpret_cast<const char *>(g.mask) + (per_image ? (long)img0 * g.mask_bsC : (long)j0) * 4;
        char *const out2 = reinterpret_cast<char *>(g.C2) + (long)img0 * g.c2_bsC * 4;
        // Per 32-column block of the wavefront: the lane's byte offset (into C, into the mask) and whether this tile
        // owns the column.
        unsigned voff[TN], mvoff[TN], tvoff[TN];
        bool own[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int jg = j0 + wn * (TN * 32) + b * 32 + l32;
            own[b] = jg >= own_j0;  // else the neighbouring tile stores it
            long col = jg - j0, mcol = jg - j0, tcol = 0;
            if (per_image) {
                unsigned im, n, y, x;
                g.divN.divmod((unsigned)jg, im, n);
                g.divCW.divmod(n, y, x);
                col = (long)(im - img0) * g.bsC + (g.c_pitch ? (long)y * g.c_pitch + x : (long)n);
                mcol = (long)(im - img0) * g.mask_bsC + (g.mask_pitch ? (long)y * g.mask_pitch + x : (long)n);
                tcol = (long)(im - img0) * g.c2_bsC + (long)y * g.c2_pitch + x;
            }
            voff[b] = (unsigned)(col * 4 + 4 * half * row_bytes);
            mvoff[b] = (unsigned)(mcol * 4 + 4 * half * mask_row_bytes);
            tvoff[b] = (unsigned)(tcol * 4 + 4 * half * twin_row_bytes);
        }
        // Rows outermost, the wavefront's column blocks innermost: the stores of one output row follow each other
        // directly, so a cache line that two neighbouring 128-byte segments share (rows are rarely 128-byte aligned)
        // is completed while it is still in L2 instead of going out to memory twice.
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const int iu = i0 + wm * (TM * 32) + a * 32;  // uniform
            float bias_v[16];
            if (MODE != 0 && g.bias) {
#pragma unroll
                for (int v = 0; v < 16; ++v)
                    bias_v[v] = *reinterpret_cast<const float *>(
                        reinterpret_cast<const char *>(g.bias + iu + 8 * (v / 4) + (v % 4)) + 16 * half);
            } else {
#pragma unroll
                for (int v = 0; v < 16; ++v) bias_v[v] = 0.0f;
            }
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int ir = iu + 8 * (v / 4) + (v % 4);  // uniform; the lane's row is ir + 4*half
                if (CHECK && ir + 4 * half < own_i0) continue;
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    if (CHECK && !own[b]) continue;
                    float *c = reinterpret_cast<float *>(out + (long)ir * row_bytes + voff[b]);
                    float val = acc[a][b][v];
                    if (MODE != 0) val = val * g.alpha + bias_v[v];
                    if (MODE == 2) val += g.beta * *c;
                    if (act) val = val > g.act_threshold ? val : g.act_value;
                    if (masked) {
                        const float mv = *reinterpret_cast<const float *>(msk + (long)ir * mask_row_bytes + mvoff[b]);
                        val = mv > g.mask_threshold ? val : 0.0f;
                    }
                    *c = val;
                    if (twin) *reinterpret_cast<float *>(out2 + (long)ir * twin_row_bytes + tvoff[b]) = val;
                }
            }
        }
    };
    // The scattered store (see GemmProblem::scatter): rows are (plane, row phase, column phase) triples, columns
    // cells of a per-image grid; an element lands at a strided position of the image or is dropped.
    // Block geometry of the accumulators: 32x32 blocks keep D[8*(v/4) + 4*(l/32) + v%4][l%32] in register v of lane
    // l, 16x16 blocks D[4*(l/16) + v][l%16].
    constexpr int BLK = SMALL ? 16 : 32;
    auto write_scatter = [&]() {
        const bool masked = g.mask != nullptr;
        const int lcol = lane & (BLK - 1);
        long cbase[TN];  // float offset of the cell's phase-(0,0) pixel; may lie before the image (pH, pW)
        int hy[TN], wx[TN];
        bool own[TN];
#pragma unroll
        for (int b = 0; b < TN; ++b) {
            const int jg = j0 + wn * (TN * BLK) + b * BLK + lcol;
            own[b] = jg >= own_j0;
            unsigned im, n, y, x;
            g.divN.divmod((unsigned)jg, im, n);
            g.divCW.divmod(n, y, x);
            hy[b] = (int)y * g.scat_sH - g.scat_pH;
            wx[b] = (int)x * g.scat_sW - g.scat_pW;
            cbase[b] = (long)im * g.bsC + (long)hy[b] * g.scat_W + wx[b];
        }
        const long plane = (long)g.scat_H * g.scat_W;
#pragma unroll
        for (int a = 0; a < TM; ++a) {
            const int iu = i0 + wm * (TM * BLK) + a * BLK;
#pragma unroll
            for (int v = 0; v < ACCV; ++v) {
                const int row = SMALL ? iu + 4 * (lane >> 4) + v : iu + 8 * (v / 4) + (v % 4) + 4 * half;
                if (row < own_i0 || row >= g.scat_rows) continue;
                unsigned c, rem, ph, pw;
                g.divScatS.divmod((unsigned)row, c, rem);
                g.divScatW.divmod(rem, ph, pw);
                const long roff = (long)c * plane + (long)ph * g.scat_W + pw;
#pragma unroll
                for (int b = 0; b < TN; ++b) {
                    const int h = hy[b] + (int)ph, w = wx[b] + (int)pw;
                    if (!own[b] || h < 0 || h >= g.scat_H || w < 0 || w >= g.scat_W) continue;
                    const long off = cbase[b] + roff;
                    float val = acc[a][b][v] * g.alpha;
                    if (masked) val = g.mask[off] > g.mask_threshold ? val : 0.0f;
                    g.C[off] = val;
                }
            }
        }
    };
    if constexpr (RED && !SMALL) {
        if (rs_on) {  // all of a wavefront or none
            const long slots = (long)g.nsplit * g.tilesJ;
            float *dst = g.rowsum_ws + ((long)split * g.tilesJ + tj);
#pragma unroll
            for (int a = 0; a < TM; ++a) {
                const float total = bsum[a] + __shfl_xor(bsum[a], 32);  // the two halves hold different r
                const int row = i0 + wm * (TM * 32) + a * 32 + l32;
                if (half == 0 && row >= own_i0) dst[row * slots] = total;
            }
        }
    }
    using std::integral_constant;
    if constexpr (LB == LD_XC_GATHER && !RED) {
        if (SMALL || g.scatter) {
            write_scatter();
            return;
        }
    }
    if constexpr (!SMALL) {
        if (g.nsplit > 1) {
            if (edge_tile) write_out(integral_constant<int, 0>{}, integral_constant<bool, true>{});
            else write_out(integral_constant<int, 0>{}, integral_constant<bool, false>{});
        } else if (g.beta == 0.0f) {
            if (edge_tile) write_out(integral_constant<int, 1>{}, integral_constant<bool, true>{});
            else write_out(integral_constant<int, 1>{}, integral_constant<bool, false>{});
        } else {
            write_out(integral_constant<int, 2>{}, integral_constant<bool, true>{});
        }
    }
}

// The short-row variant (see the kernel's ROWS16): first operand along r, gathered B, scattered store, unsplit.
template <int BN, int WGN, int ROWS16>
int gemm_fast_short_rows_go(const GemmArgs &g, hipStream_t s) {
    if (!g.scatter || g.nsplit != 1 || g.M != 64 || g.scat_rows > 16 * ROWS16)
        return fail("gemm: the short-row kernel takes an unsplit scattered product of 64 padded rows, at most %d used",
                    16 * ROWS16);
    hipLaunchKernelGGL((gemm_fast_kernel<64, BN, 1, WGN, LD_RC_VEC, LD_XC_GATHER, false, ROWS16>), dim3(g.total),
                       dim3(WGN * 64), 0, s, g);
    return 0;
}

template <int BM, int BN, int WGM, int WGN, int LA, int LB, bool RED>
int gemm_fast_go(const GemmArgs &g, hipStream_t s) {
    hipLaunchKernelGGL((gemm_fast_kernel<BM, BN, WGM, WGN, LA, LB, RED>), dim3(g.total), dim3(WGM * WGN * 64), 0, s, g);
    return 0;
}

// Dispatch over the loader kinds for one tile configuration.
template <int BM, int BN, int WGM, int WGN>
int gemm_fast_dispatch(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
#define THGPU_CASE(LA_, LB_)                                                           \
    if (la == LA_ && lb == LB_) {                                                      \
        if constexpr ((LA_ == LD_XC_SCALAR && (WGM * WGN * 64) % BM != 0 &&            \
                       !((WGM * WGN * 64) == 256 && BM % 64 == 0)) ||                  \
                      ((LB_ == LD_XC_SCALAR || LB_ == LD_XC_GATHER) && (WGM * WGN * 64) % BN != 0)) { \
            return fail("gemm: this tile has no x-contiguous loader for that side");   \
        } else {                                                                       \
            if (red) {                                                                 \
                if constexpr (LA_ != LD_XC_SCALAR && LB_ != LD_XC_SCALAR)              \
                    return gemm_fast_go<BM, BN, WGM, WGN, LA_, LB_, true>(g, s);       \
                else                                                                   \
                    return fail("gemm: reduction batching needs r-contiguous operands"); \
            }                                                                          \
            return gemm_fast_go<BM, BN, WGM, WGN, LA_, LB_, false>(g, s);              \
        }                                                                              \
    }
    THGPU_CASE(LD_RC_VEC, LD_RC_VEC)
    THGPU_CASE(LD_RC_VEC, LD_RC_SCALAR)
    THGPU_CASE(LD_RC_VEC, LD_XC_SCALAR)
    THGPU_CASE(LD_RC_VEC, LD_XC_GATHER)
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

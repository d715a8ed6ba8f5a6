// Host side of the fp32 MFMA GEMM: picks a tile configuration, the operand
// loaders and a reduction split for a GemmProblem, launches the kernel and,
// when the reduction was split, the fixed-order reduction of the partial sums.
// Also the THGPUBlas_gemm entry point.
#include "gemm_mfma.h"
#include "side_jobs.h"

#include <cstring>

namespace thgpu {

namespace {

// C(i, j) = beta*C + alpha * sum_s ws[s][i][j] (+ bias[i]), s ascending; j is
// mapped through (image, n) when the output is column batched.
// The second job of a reduction launch: out[i] += alpha * sum over slots of ws[i][slot].  One wavefront per row:
// lane l adds slots l, l + 64, ... in ascending order, then the lanes are added pairwise in a fixed tree, so the
// result is reproducible.
struct RowSumJob {
    const float *ws;
    float *out;
    int M, slots;
    float alpha;
    unsigned first_block;  // workgroups from this one on work on the row sums, four rows each
};

__device__ __forceinline__ void rowsum_reduce(const RowSumJob &j, unsigned block) {
    const int lane = threadIdx.x & 63;
    const int row = (int)block * 4 + (int)(threadIdx.x >> 6);
    if (row >= j.M) return;  // a whole wavefront
    const float *src = j.ws + (long)row * j.slots;
    float sum = 0.0f;
    for (int s = lane; s < j.slots; s += 64) sum += src[s];
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) sum += __shfl_down(sum, d);
    if (lane == 0) j.out[row] += j.alpha * sum;
}

template <bool quarters>
__global__ __launch_bounds__(256) void split_reduce_kernel(const RowSumJob rs, const float *__restrict__ ws, float *__restrict__ C,
                                                           const float *__restrict__ bias, int M, int J, int N,
                                                           long sC, long bsC, FastDiv divJ, FastDiv divN, int nsplit,
                                                           float alpha, float beta, int act, float act_threshold,
                                                           float act_value, const float *__restrict__ mask,
                                                           float mask_threshold, int c_pitch, int mask_pitch,
                                                           long mask_sC, long mask_bsC, FastDiv divCW,
                                                           float *__restrict__ C2, long c2_sC, long c2_bsC, int c2_pitch,
                                                           const unsigned side_first_block, const WeightJob side,
                                                           const unsigned j_store) {
    // workgroups behind the reduction's carry a job of the next layer's (side_jobs.h)
    if (blockIdx.x >= side_first_block) {
        reorder_weight(side, (blockIdx.x - side_first_block) * 256u + threadIdx.x);
        return;
    }
    if (rs.out && blockIdx.x >= rs.first_block) {
        rowsum_reduce(rs, blockIdx.x - rs.first_block);
        return;
    }
    // With `quarters` the four wavefronts of a workgroup share 64 outputs, each adding a contiguous quarter of the
    // partial sums (for few outputs and many splits: one lane per output would leave the GPU idle behind a long
    // chain of loads); the quarters are then added in order.  Either way the order of the adds is fixed.
    const unsigned total = (unsigned)M * (unsigned)J;
    const unsigned wave = threadIdx.x >> 6;
    unsigned idx = quarters ? blockIdx.x * 64u + (threadIdx.x & 63u) : blockIdx.x * blockDim.x + threadIdx.x;
    const bool valid = idx < total;
    if (!quarters && !valid) return;
    const int per = quarters ? (nsplit + 3) / 4 : nsplit;
    const int s_begin = quarters ? (int)wave * per : 0;
    const int s_end = s_begin + per < nsplit ? s_begin + per : nsplit;
    // Eight partials are requested before the first is added; the adds stay in split order.
    float sum = 0.0f;
    const float *src = ws + (valid ? idx : 0);
    for (int s0 = s_begin; s0 < s_end; s0 += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = s0 + u < s_end ? src[(long)(s0 + u) * total] : 0.0f;
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (s0 + u < s_end) sum += v[u];
    }
    if (quarters) {
        __shared__ float part[4][64];
        part[wave][threadIdx.x & 63u] = sum;
        __syncthreads();
        if (wave != 0 || !valid) return;
        sum = ((part[0][threadIdx.x] + part[1][threadIdx.x]) + part[2][threadIdx.x]) + part[3][threadIdx.x];
    }
    unsigned i, j;
    divJ.divmod(idx, i, j);
    if (j >= j_store) return;  // a scratch column of a product run wider than its result (GemmProblem::j_store)
    long coff = j, moff = j, toff = 0;
    if (N != J || c_pitch || mask_pitch || C2) {
        unsigned im, n, y, x;
        divN.divmod(j, im, n);
        divCW.divmod(n, y, x);
        coff = (long)im * bsC + (c_pitch ? (long)y * c_pitch + x : (long)n);
        moff = (long)im * mask_bsC + (mask_pitch ? (long)y * mask_pitch + x : (long)n);
        toff = (long)im * c2_bsC + (long)y * c2_pitch + x;
    }
    float *c = C + (long)i * sC + coff;
    float val = alpha * sum;
    if (bias) val += bias[i];
    if (beta != 0.0f) val += beta * *c;
    if (act) val = val > act_threshold ? val : act_value;
    if (mask) val = mask[(long)i * mask_sC + moff] > mask_threshold ? val : 0.0f;
    *c = val;
    if (C2) C2[(long)i * c2_sC + toff] = val;  // the second copy (GemmProblem::C2)
}

struct TileCfg {
    const char *name;
    int bm, bn;
    int resident;  // workgroups that fit a CU at once (registers / LDS)
    // Fraction of the MFMA rate the inner loop sustains with a full CU, by operand layout (measured
    // on the AlexNet layer shapes): [0] A along r, B along j (forward); [1] both along their free
    // index (gradInput); [2] both along r (gradWeight); [3] A along i, B along r; [4] A along r, B gathered
    // (the 64-row tiles: narrow gathered products run faster on the small tile, products on columns do not).  The figures are fitted to
    // measured launch times together with the occupancy factors of model_cycles.
    double eff[5];
    int (*launch)(const GemmArgs &, int, int, bool, hipStream_t);
    // Fraction of that rate kept with k = 1..4 workgroups resident per CU (nullptr: the tables of model_cycles), and
    // the row count from which the tile is no longer considered (0: no limit).
    const double *occ;
    int below_rows;
    // Short-row variant: the rows of the tile its wavefronts multiply (0: all of them).  It takes scattered products
    // of exactly one tile of rows, of which no more than this many are in use.
    int rows_used;
    // The tile has no loader for a first operand contiguous along its rows.
    bool a_rc_only;
};

// The 64 x 128 tile's wavefronts own 64 x 32 outputs, half the MFMAs per reduction step of the large tiles: it needs all
// four workgroups on a CU to keep the matrix pipe busy (measured on the 64-row products of the AlexNet-style stack: the
// 64 x 4800 gathered gradInput runs 10 % faster in seven splits that fill every round than unsplit with three
// workgroups per CU).  Taller tiles re-read the second operand less often, so it only stands in where they do not fit.
const double kOccNarrow[5] = {0.0, 0.50, 0.75, 0.88, 1.0};

const TileCfg kCfgs[] = {
    {"128x128", 128, 128, 4, {0.90, 0.90, 0.88, 0.86, 0.90}, gemm_fast_128x128, nullptr, 0, 0, false},
    {"192x128", 192, 128, 3, {0.90, 0.90, 0.90, 0.86, 0.90}, gemm_fast_192x128, nullptr, 0, 0, false},
    {"64x256", 64, 256, 3, {0.76, 0.74, 0.90, 0.74, 0.70}, gemm_fast_64x256, nullptr, 0, 0, false},
    {"128x256", 128, 256, 2, {0.85, 0.87, 0.95, 0.85, 0.85}, gemm_fast_128x256, nullptr, 0, 0, false},
    {"256x128", 256, 128, 2, {0.90, 0.75, 0.95, 0.75, 0.90}, gemm_fast_256x128, nullptr, 0, 0, false},
    {"64x64", 64, 64, 4, {0.68, 0.60, 0.74, 0.60, 0.72}, gemm_fast_64x64, nullptr, 0, 0, false},
    {"64x128", 64, 128, 4, {0.84, 0.78, 0.84, 0.78, 0.86}, gemm_fast_64x128, kOccNarrow, 128, 0, false},
    {"48x128", 64, 128, 4, {0, 0, 0, 0, 0.84}, gemm_fast_48x128, kOccNarrow, 128, 48, false},
    {"48x256", 64, 256, 3, {0, 0, 0, 0, 0.70}, gemm_fast_48x256, nullptr, 0, 48, false},
    {"96x128", 96, 128, 4, {0.84, 0, 0.84, 0, 0.86}, gemm_fast_96x128, kOccNarrow, 128, 0, true},
};

inline long cdiv(long a, long b) { return (a + b - 1) / b; }

// Rough time model (in CU-cycles) used only to rank (tile, split) candidates.
// A CU retires 256 flops per cycle at best; with fewer workgroups resident it
// hides less of their latencies (kOcc); workgroups beyond what fits at once
// run in further rounds; every round pays a prologue/epilogue; a split adds
// the traffic of writing and re-reading the partial sums.
double model_cycles(const TileCfg &c, int layout, long M, long J, long steps_total, int nsplit, int cus) {
    // With both operands along r (layout 2) two resident workgroups already keep the MFMA pipe as
    // busy as three: measured on the 192 x 1600 gradWeight product, 39 splits (two per CU) beat 59.
    static const double kOccDefault[5] = {0.0, 0.70, 0.88, 0.96, 1.0};
    static const double kOccBothR[5] = {0.0, 0.70, 0.98, 0.96, 1.0};
    const double *kOcc = c.occ ? c.occ : layout == 2 ? kOccBothR : kOccDefault;
    const long tiles = cdiv(M, c.bm) * cdiv(J, c.bn);
    const long wgs = tiles * nsplit;
    const long steps = cdiv(steps_total, nsplit);
    const double per_step = 2.0 * (c.rows_used ? c.rows_used : c.bm) * c.bn * GEMM_BK / 256.0 / c.eff[layout];
    const double ovh = 3000.0 + 6.0 * c.bm * c.bn / 64.0;
    const long slots = (long)cus * c.resident;
    const long full = wgs / slots, rest = wgs - full * slots;
    double t = full * (c.resident * steps * per_step / kOcc[c.resident] + ovh);
    if (rest > 0) {
        const long on_busiest = cdiv(rest, cus);
        const int k = (int)(on_busiest < c.resident ? on_busiest : c.resident);
        t += on_busiest * steps * per_step / kOcc[k] + ovh * (k > 1 ? 1.0 : 1.5);
    }
    if (nsplit > 1) t += (double)(nsplit + 2) * M * J * 4.0 / (4.5e12 / 2.4e9);  // bytes / (bytes per cycle)
    return t;
}

// The tile configuration and reduction split for a problem; cfg == nullptr when no tiled kernel takes it.
struct GemmPlan {
    const TileCfg *cfg = nullptr;
    int nsplit = 1;
};

GemmPlan plan_gemm(const GemmProblem &p, int steps_total) {
    GemmPlan plan;
    const bool gather = p.rowtab != nullptr;
    const int cus = num_cus();
    double best_t = 0;
    // Tuning aids: the gemm_tile switch forces a configuration by name, gemm_split a split count.
    const Tuning &tune = tuning();
    const char *force = tune.gemm_tile[0] ? tune.gemm_tile : nullptr;
    const int fsplit = tune.gemm_split;
    // The fast kernel addresses each operand as a uniform base plus a 32-bit
    // per-thread byte offset and moves a partial last step back by up to 15
    // reduction indices: it needs R >= 16 and tile-local offsets below 2^30 floats.
    // The output is addressed the same way (four rows and a tile's columns per lane).
    const long n_img = p.N > 0 ? p.N : p.J;
    auto offsets_fit = [&](int bm, int bn) {
        const long offA = p.a_rc ? (long)(bm - 1) * p.sA + GEMM_BK : (long)(GEMM_BK - 1) * p.sA + bm;
        const long span = (bn - 1) / n_img + 2;  // images a tile's columns can touch
        const long offB = gather ? p.b_extent
                          : p.b_rc ? (long)(bn - 1) * p.sB + GEMM_BK
                                   : (long)(GEMM_BK - 1) * p.sB + span * p.bsB + n_img;
        const long offC = 4 * (p.sC > p.J ? p.sC : (long)p.J) + span * p.bsC + n_img;
        const long offC2 = p.C2 ? 4 * p.c2_sC + span * p.c2_bsC + (p.c_w > 0 ? n_img / p.c_w : 0) * p.c2_pitch + p.c_w : 0;
        return offA < (1L << 30) && offB < (1L << 30) && offC < (1L << 30) && offC2 < (1L << 30);
    };
    const bool fast_ok = p.R == 0 || p.R >= GEMM_BK;
    const int layout = gather ? 4 : p.a_rc ? (p.b_rc ? 2 : 0) : (p.b_rc ? 3 : 1);
    for (const TileCfg &c : kCfgs) {
        if (!fast_ok || p.M < c.bm || p.J < c.bn || !offsets_fit(c.bm, c.bn)) continue;
        if (force && std::strcmp(force, c.name) != 0) continue;
        if (!force && c.below_rows > 0 && p.M >= c.below_rows) continue;
        if (c.a_rc_only && !p.a_rc) continue;
        if (c.rows_used > 0 && !(p.scatter && layout == 4 && p.M == c.bm && p.scat_rows <= c.rows_used)) continue;
        const long tiles = cdiv(p.M, c.bm) * cdiv(p.J, c.bn);
        // (a product run wider than its result has one narrow tile per row block: it may split further to fill the GPU)
        const int split_cap = p.j_store > 0 ? 1024 : 256;
        int max_split = (int)(steps_total / 8 > 0 ? (steps_total / 8 < split_cap ? steps_total / 8 : split_cap) : 1);
        if (p.scatter) max_split = 1;  // the scattered store has no partial-sum form
        const int min_split = p.j_store > 0 ? 2 : 1;  // scratch columns never reach C unsplit
        int want = fsplit > 0 ? (fsplit < max_split ? fsplit : max_split) : 0;
        if (want > 0 && want < min_split) want = min_split;
        for (int ns = min_split; ns <= max_split; ++ns) {
            if (want > 0 && ns != want) continue;
            if (tiles * ns > 8L * cus * c.resident && ns > 1 && fsplit <= 0) break;
            if (ns > 1 && p.ws_fixed && (long)ns * p.M * p.J > p.ws_fixed_floats) break;  // partial sums must fit
            const int sps = (int)cdiv(steps_total, ns);
            if ((int)cdiv(steps_total, sps) != ns) continue;  // would leave an empty split
            const double t = model_cycles(c, layout, p.M, p.J, steps_total, ns, cus);
            if (!plan.cfg || t < best_t) {
                plan.cfg = &c;
                plan.nsplit = ns;
                best_t = t;
            }
        }
    }
    return plan;
}

inline int steps_of(const GemmProblem &p) {
    return (p.R + GEMM_BK - 1) / GEMM_BK * (p.nb > 1 ? p.nb : 1);
}

}  // namespace

bool gemm_tiled_fits(const GemmProblem &p) {
    if (p.M <= 0 || p.J <= 0 || (long)p.M * p.J >= (1L << 31)) return false;
    return plan_gemm(p, steps_of(p)).cfg != nullptr;
}

int gemm_launch(const GemmProblem &p) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (p.M <= 0 || p.J <= 0) return 0;
    if ((long)p.M * p.J >= (1L << 31)) return fail("gemm: output of %d x %d exceeds 32-bit tile indexing", p.M, p.J);

    const bool red = p.nb > 1;
    const bool gather = p.rowtab != nullptr;
    if (gather && (!p.coltab || p.b_rc || !p.a_rc)) return fail("gemm: a gathered B needs both tables and an r-contiguous A");
    if (red && !(p.a_rc && (p.b_rc || gather))) return fail("gemm: reduction batching needs r-contiguous operands");

    GemmArgs g;
    std::memset(&g, 0, sizeof(g));
    g.A = p.A;
    g.B = p.B;
    g.C = p.C;
    g.bias = p.bias;
    g.rowtab = p.rowtab;
    g.coltab = p.coltab;
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
    g.act = p.act ? 1 : 0;
    g.act_threshold = p.act_threshold;
    g.act_value = p.act_value;
    g.mask = p.mask;
    g.mask_threshold = p.mask_threshold;
    if ((p.c_pitch || p.mask_pitch) && (p.c_w <= 0 || red || g.N % p.c_w != 0))
        return fail("gemm: pitched rows need column batching and a plane width that divides the columns of an image");
    g.c_w = p.c_w > 0 ? p.c_w : 1;
    g.c_pitch = p.c_pitch;
    g.mask_pitch = p.mask_pitch;
    g.mask_sC = p.mask_sC ? p.mask_sC : p.sC;
    g.mask_bsC = p.mask_bsC ? p.mask_bsC : p.bsC;
    g.divCW = FastDiv((uint32_t)g.c_w);
    // (reduction batching or one image: either way every column of the product is a column of C or scratch)
    if (p.j_store > 0 && (p.N != p.J || p.j_store > p.J || p.sC < p.j_store || p.C2 || p.scatter))
        return fail("gemm: scratch columns need an unbatched column index and a row pitch of C that holds the stored ones");
    if (p.C2) {
        if (red || p.scatter || p.c_w <= 0 || g.N % p.c_w != 0 || p.c2_pitch < p.c_w || p.c2_sC <= 0 || p.c2_bsC <= 0)
            return fail("gemm: a second copy of the result needs column batching, a plane width and the copy's strides");
        g.C2 = p.C2;
        g.c2_sC = p.c2_sC;
        g.c2_bsC = p.c2_bsC;
        g.c2_pitch = p.c2_pitch;
    }
    if (p.scatter) {
        if (!gather || red || p.bias || p.beta != 0.0f || p.c_pitch || p.mask_pitch || p.c_w <= 0 || g.N % p.c_w != 0 ||
            p.scat_sH <= 0 || p.scat_sW <= 0 || p.scat_H <= 0 || p.scat_W <= 0 || p.scat_rows <= 0 || p.scat_rows > p.M ||
            p.scat_pH < 0 || p.scat_pW < 0)
            return fail("gemm: a scattered store needs a gathered B, column batching, no bias and beta = 0");
        g.scatter = 1;
        g.scat_sH = p.scat_sH;
        g.scat_sW = p.scat_sW;
        g.scat_pH = p.scat_pH;
        g.scat_pW = p.scat_pW;
        g.scat_H = p.scat_H;
        g.scat_W = p.scat_W;
        g.scat_rows = p.scat_rows;
        g.divScatS = FastDiv((uint32_t)(p.scat_sH * p.scat_sW));
        g.divScatW = FastDiv((uint32_t)p.scat_sW);
    }
    g.steps_per_img = (p.R + GEMM_BK - 1) / GEMM_BK;
    g.steps_total = g.steps_per_img * (red ? p.nb : 1);
    g.divSpi = FastDiv((uint32_t)(g.steps_per_img > 0 ? g.steps_per_img : 1));

    const int cus = num_cus();
    const GemmPlan plan = plan_gemm(p, g.steps_total);
    const TileCfg *best = plan.cfg;
    const int best_split = plan.nsplit;

    g.nsplit = best ? best_split : 1;
    const int bm = best ? best->bm : 64, bn = best ? best->bn : 64;
    if (!best && red) {
        // The generic kernel splits too: enough workgroups to fill the chip.
        const long tiles = cdiv(p.M, 64) * cdiv(p.J, 64);
        long want = cdiv(2L * cus, tiles);
        const long cap = g.steps_total / 8 > 0 ? g.steps_total / 8 : 1;
        if (want > cap) want = cap;
        if (want < 1) want = 1;
        if (p.ws_fixed && want * p.M * p.J > p.ws_fixed_floats) want = p.ws_fixed_floats / ((long)p.M * p.J);
        if (want < 1) want = 1;
        const int sps = (int)cdiv(g.steps_total, want);
        g.nsplit = (int)cdiv(g.steps_total, sps);
    }
    g.steps_per_split = (int)cdiv(g.steps_total, g.nsplit);
    g.tilesM = (unsigned)cdiv(p.M, bm);
    g.tilesJ = (unsigned)cdiv(p.J, bn);
    g.divTilesM = FastDiv(g.tilesM);
    g.divTilesJ = FastDiv(g.tilesJ);
    const long total = (long)g.tilesM * g.tilesJ * g.nsplit;
    if (total <= 0 || total >= (1L << 31)) return fail("gemm: tile count %ld out of range", total);
    g.total = (unsigned)total;
    // Row sums of A ride along with a tiled reduction-batched product (never with the fixed workspace of the
    // entry point that may not allocate: nothing there asks for them).
    const bool rowsum = p.rowsum && best && red && !p.ws_fixed;
    if (p.rowsum_done) *p.rowsum_done = rowsum;
    const size_t rowsum_floats = rowsum ? (size_t)g.nsplit * g.tilesJ * p.M : 0;
    if (g.nsplit > 1 || rowsum) {
        const size_t need = (g.nsplit > 1 ? (size_t)g.nsplit * p.M * p.J : 0) + rowsum_floats;
        if (p.ws_fixed) {
            if ((long)need > p.ws_fixed_floats)
                return fail("gemm: %zu floats of partial sums exceed the fixed workspace of %ld", need, p.ws_fixed_floats);
            g.ws = p.ws_fixed;
        } else {
            g.ws = workspace(sizeof(float) * need);
        }
        if (!g.ws) return 1;
        if (rowsum) g.rowsum_ws = g.ws + (need - rowsum_floats);
    }

    // ---- loaders: r-contiguous operands use 128-bit loads (4-byte alignment suffices) --------
    const int la = p.a_rc ? LD_RC_VEC : LD_XC_SCALAR;
    const int lb = p.b_rc ? LD_RC_VEC : gather ? LD_XC_GATHER : LD_XC_SCALAR;
    if (gather && !best) return fail("gemm: a gathered B needs a shape the tiled kernel takes (M, J >= 64, R >= 16)");
    if (p.C2 && !best) return fail("gemm: a second copy of the result needs a shape the tiled kernel takes");
    if (p.j_store > 0 && (!best || g.nsplit < 2))
        return fail("gemm: scratch columns need a tiled kernel and a split reduction");

    int rc;
    {
        const char *label = p.tag;
        if (prof_enabled())
            label = prof_label("%s M=%d J=%d R=%ld tile=%s split=%d", p.tag, p.M, p.J, (long)p.R * (red ? p.nb : 1),
                               best ? best->name : "generic", g.nsplit);
        LaunchScope scope(label, p.flops > 0 ? p.flops : 2.0 * p.M * p.J * (double)p.R * (red ? p.nb : 1), 0.0);
        rc = best ? best->launch(g, la, lb, red, s) : gemm_generic_64x64(g, p.a_rc, p.b_rc, red, s);
    }
    if (rc) return rc;
    if (check_launch(p.tag)) return 1;
    if (g.nsplit > 1 || rowsum) {
        const long n = g.nsplit > 1 ? (long)p.M * p.J : 0;  // an unsplit product has stored its own result
        RowSumJob rs;
        std::memset(&rs, 0, sizeof(rs));
        // few outputs, many splits: four wavefronts per 64 outputs
        const int quarters = (n > 0 && n < 128 * 1024 && g.nsplit >= 32) ? 1 : 0;
        unsigned blocks = (unsigned)cdiv(n, quarters ? 64 : 256);
        if (rowsum) {
            rs.ws = g.rowsum_ws;
            rs.out = p.rowsum;
            rs.M = p.M;
            rs.slots = (int)(g.nsplit * g.tilesJ);
            rs.alpha = p.alpha;
            rs.first_block = blocks;
            blocks += (unsigned)cdiv(p.M, 4);
        }
        // A product that stores a second copy of its result for the next layer's gradInput product also carries that
        // layer's pending kernel-bank job, if there is one.
        WeightJob side = {};
        const unsigned side_first = blocks;
        double side_bytes = 0.0;
        if (g.C2 && n > 0 && take_bank_job(side)) {
            blocks += (side.count + 255u) / 256u;
            side_bytes = 4.0 * (side.count + (double)side.M * side.C * side.kH * side.kW);
        }
        {
            LaunchScope scope("gemm_split_reduce", 0.0,
                              4.0 * n * (g.nsplit + 2 + (g.C2 ? 1 : 0)) + 4.0 * rowsum_floats + side_bytes);
            auto kernel = quarters ? split_reduce_kernel<true> : split_reduce_kernel<false>;
            hipLaunchKernelGGL(kernel, dim3(blocks), dim3(256), 0, s, rs, g.ws, p.C, p.bias,
                               p.M, p.J, g.N, p.sC, p.bsC, FastDiv((uint32_t)p.J), g.divN, g.nsplit, p.alpha,
                               p.beta, g.act, g.act_threshold, g.act_value, g.mask, g.mask_threshold, g.c_pitch,
                               g.mask_pitch, g.mask_sC, g.mask_bsC, g.divCW, g.C2, g.c2_sC, g.c2_bsC, g.c2_pitch,
                               side_first, side, (unsigned)(p.j_store > 0 ? p.j_store : p.J));
        }
        if (check_launch("gemm_split_reduce")) return 1;
    }
    return 0;
}

}  // namespace thgpu

using namespace thgpu;

namespace {

// Column-major BLAS arguments as a GemmProblem.  Returns 1 for the quick returns of the reference
// dispatcher (nothing to do), -1 for a dimension the kernels cannot index, -2 for a null operand, 0 otherwise.
int blas_problem(GemmProblem &p, char transa, char transb, long m, long n, long k, float alpha, const float *a,
                 long lda, const float *b, long ldb, float beta, float *c, long ldc) {
    const bool ta = (transa == 't' || transa == 'T');
    const bool tb = (transb == 't' || transb == 'T');
    // Quick returns of the reference dispatcher (gputorch/lib/THC/THCBlas.cpp:257).
    if (!m || !n || ((alpha == 0 || !k) && beta == 1)) return 1;
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
    if (m < 0 || n < 0 || k < 0 || m >= (1L << 31) || n >= (1L << 31) || k >= (1L << 31)) return -1;
    // a product that will touch memory needs its operands: a null pointer here would fault on the GPU
    if (!c || (alpha != 0 && k > 0 && (!a || !b))) return -2;
    // Column-major C(m x n) is the row-major n x m matrix C'(i', j') =
    // c[j' + i'*ldc]; C' = op(B)' * op(A)' with
    //   A'(i', r) = op(B)(r, i'),  B'(r, j') = op(A)(j', r).
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
    return 0;
}

}  // namespace

extern "C" void THGPUBlas_gemm(char transa, char transb, long m, long n, long k, float alpha, float *a, long lda,
                               float *b, long ldb, float beta, float *c, long ldc) {
    GemmProblem p;
    const int rc = blas_problem(p, transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
    if (rc > 0) return;
    if (rc < 0) {
        raise(rc == -2 ? "THGPUBlas_gemm: null operand" : "THGPUBlas_gemm: dimension exceeds 2^31");
        return;
    }
    if (gemm_launch(p)) raise("%s", thgpu_last_error());
}

extern "C" int thgpu_gemm_noalloc(char transa, char transb, long m, long n, long k, float alpha, const float *a,
                                  long lda, const float *b, long ldb, float beta, float *c, long ldc) {
    // Nothing here may allocate, so neither may a lazy initialisation: the stream and the address of the
    // static array exist only after thgpu_init.
    size_t cap = 0;
    float *ws = static_scratch(&cap);
    if (!ws) return fail("thgpu_gemm_noalloc: call thgpu_init() first (this entry point sets nothing up itself)");
    // (dimensions are range-checked before they are multiplied)
    if (m >= (1L << 31) || n >= (1L << 31) || k >= (1L << 31))
        return fail("thgpu_gemm_noalloc: dimension exceeds 2^31");
    if (m > 0 && n > 0 && m * n > (long)cap)
        return fail("thgpu_gemm_noalloc: a result of %ld x %ld elements exceeds the limit of %zu elements (%zu MiB)", m,
                    n, cap, cap * sizeof(float) >> 20);
    GemmProblem p;
    const int rc = blas_problem(p, transa, transb, m, n, k, alpha, a, lda, b, ldb, beta, c, ldc);
    if (rc > 0) return 0;
    if (rc < 0) return fail(rc == -2 ? "thgpu_gemm_noalloc: null operand" : "thgpu_gemm_noalloc: dimension exceeds 2^31");
    p.ws_fixed = ws;
    p.ws_fixed_floats = (long)cap;
    p.tag = "gemm_blas_noalloc";
    return gemm_launch(p);
}

extern "C" int thgpu_gemm_strided_batched(char transa, char transb, long m, long n, long k, float alpha, const float *a,
                                          long lda, long stride_a, const float *b, long ldb, long stride_b, float beta,
                                          float *c, long ldc, long stride_c, long batch) {
    const bool ta = (transa == 't' || transa == 'T');
    const bool tb = (transb == 't' || transb == 'T');
    if (batch <= 0 || !m || !n) return 0;
    if (m >= (1L << 31) || n >= (1L << 31) || k >= (1L << 31)) return fail("gemm_strided_batched: dimension exceeds 2^31");
    if (stride_c == 0 && batch > 1) return fail("gemm_strided_batched: the results of a batch must not overlap");
    if (!c || (alpha != 0 && k > 0 && (!a || !b))) return fail("gemm_strided_batched: null operand");
    // One launch for the whole batch when op(B) is shared, op(A) = A and the batch's columns fit the
    // kernel's 32-bit tile indexing: the batch index then simply extends the columns of the (row-major,
    // transposed) product, as in the convolution's forward and gradInput GEMMs.
    if (!ta && stride_b == 0 && batch > 1 && m * batch < (1L << 31) && n * m * batch < (1L << 31)) {
        GemmProblem p;
        p.A = b;
        p.B = a;
        p.C = c;
        p.M = (int)n;
        p.J = (int)(m * batch);
        p.R = alpha == 0 ? 0 : (int)k;
        p.N = (int)m;
        p.a_rc = !tb;
        p.sA = ldb;
        p.b_rc = false;
        p.sB = lda;
        p.sC = ldc;
        p.bsB = stride_a;
        p.bsC = stride_c;
        p.alpha = alpha;
        p.beta = beta;
        p.tag = "gemm_blas_batched";
        return gemm_launch(p);
    }
    for (long i = 0; i < batch; ++i) {
        GemmProblem p;
        p.A = b + i * stride_b;
        p.B = a + i * stride_a;
        p.C = c + i * stride_c;
        p.M = (int)n;
        p.J = (int)m;
        p.R = alpha == 0 ? 0 : (int)k;
        p.N = (int)m;
        p.a_rc = !tb;
        p.sA = ldb;
        p.b_rc = ta;
        p.sB = lda;
        p.sC = ldc;
        p.alpha = alpha;
        p.beta = beta;
        p.tag = "gemm_blas_batched";
        if (gemm_launch(p)) return 1;
    }
    return 0;
}

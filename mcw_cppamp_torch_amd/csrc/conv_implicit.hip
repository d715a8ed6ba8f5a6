// nn.SpatialConvolutionMM without the column buffer: the GEMM's second operand is gathered straight
// from a zero-padded copy of the image, element (r, x) at rowtab[r] + coltab[x] (gemm_mfma.h), so
// im2col, col2im and the K x N column buffers (kH*kW times the image) drop out.
//
//   forward     output[b][m][n]   = bias[m] + sum_k weight[m][k] * P[b][tap(k) + pixel(n)]
//   gradWeight  gradWeight[m][k] += scale * sum_b sum_n gradOutput[b][m][n] * P[b][pixel(n) + tap(k)]
//   gradInput   gradInput[b][c][p] = sum_{m,kh,kw} Wt[c][(m,kh,kw)] * Q[b][tap'(m,kh,kw) + pixel'(p)]   (stride 1)
//
// P is the input padded by (padH, padW); tap(c,kh,kw) = c*Hp*Wp + kh*Wp + kw and pixel(ho,wo) =
// ho*dH*Wp + wo*dW.  Q is gradOutput padded by (kH-1-padH, kW-1-padW) and Wt[c][(m,kh,kw)] =
// weight[m][c][kH-1-kh][kW-1-kw]: a unit-stride convolution's gradInput is the correlation of the
// padded gradOutput with the flipped kernels.  The sums run over the same products as
// gpunn-impl/SpatialConvolutionMM.cpp:110-429 (im2col + sgemm + col2im), in a different order for
// gradInput.
//
// gradInput of a strided layer, by residue class of the pixel coordinates: write h + padH = dH*y + ph and
// w + padW = dW*x + pw.  Pixel (h, w) only meets the taps kh = ph + dH*a, kw = pw + dW*b, through the output
// positions (y - a, x - b), so each of the dH*dW classes is a unit-stride correlation of gradOutput with a
// sub-sampled kernel of at most A x Bk = ceil(kH/dH) x ceil(kW/dW) taps:
//   gradInput[b][c][h][w] = sum_{m,a,b} weight[m][c][ph + dH*a][pw + dW*b] * gradOutput[b][m][y - a][x - b].
// One GEMM does all classes: row (c, ph, pw), reduction index (m, a, b) (taps beyond the kernel carry zero
// weights), column (image, y, x), second operand gathered from gradOutput padded by (A-1, Bk-1), and a
// scattered store (GemmProblem::scatter) that puts element ((c,ph,pw), (y,x)) at pixel (dH*y+ph-padH,
// dW*x+pw-padW).  No zero-dilated gradOutput, no column buffer, no col2im; the work is that of the layer's
// other products times (A*dH/kH)*(Bk*dW/kW) (taps rounded up to whole strides).
#include "gemm_mfma.h"
#include "kernels.h"
#include "side_jobs.h"

#include <array>
#include <cstdlib>
#include <cstring>
#include <map>

namespace thgpu {

namespace {

// out[plane][y][x] = in[plane][y - pH][x - pW], zero outside.  A lane produces four consecutive
// output elements (one 128-bit store; single stores at the end of an odd-sized buffer or into an unaligned one).
struct PadJob {
    const float *in;
    float *out;
    unsigned total;
    int H, W, pH, pW, Hp, Wp;
    FastDiv divWp, divHp;
    bool aligned;
};

__device__ __forceinline__ void pad_four(const PadJob &j, unsigned block) {
    const unsigned idx = (block * 256u + threadIdx.x) * 4u;
    if (idx >= j.total) return;
    unsigned rest, x, plane, y;
    j.divWp.divmod(idx, rest, x);
    j.divHp.divmod(rest, plane, y);
    float v[4];
#pragma unroll
    for (int q = 0; q < 4; ++q) {
        const int h = (int)y - j.pH, w = (int)x - j.pW;
        v[q] = 0.0f;
        if (h >= 0 && h < j.H && w >= 0 && w < j.W && idx + q < j.total) v[q] = j.in[((long)plane * j.H + h) * j.W + w];
        if (++x == (unsigned)j.Wp) {
            x = 0;
            if (++y == (unsigned)j.Hp) {
                y = 0;
                ++plane;
            }
        }
    }
    if (j.aligned && idx + 4 <= j.total) {
        *reinterpret_cast<float4 *>(j.out + idx) = make_float4(v[0], v[1], v[2], v[3]);
    } else {
        for (unsigned q = 0; idx + q < j.total; ++q) j.out[idx + q] = v[q];
    }
}

__global__ __launch_bounds__(256) void pad_planes_kernel(const PadJob j) { pad_four(j, blockIdx.x); }

// Both preparations of a gradInput product in one launch (they are independent, and the kernel bank alone is a
// launch of a few microseconds of work): the first pad_blocks workgroups pad gradOutput, the rest re-order the bank.
__global__ __launch_bounds__(256) void pad_planes_and_weights_kernel(const PadJob pad, unsigned pad_blocks,
                                                                      const WeightJob wj) {
    if (blockIdx.x < pad_blocks) pad_four(pad, blockIdx.x);
    else reorder_weight(wj, (blockIdx.x - pad_blocks) * 256u + threadIdx.x);
}

// t[(c, kh, kw)] = c*plane + kh*pitch + kw
__global__ __launch_bounds__(256) void tap_table_kernel(int *__restrict__ t, int planes, int kH, int kW, int plane,
                                                        int pitch) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= planes * kH * kW) return;
    const int kw = idx % kW, kh = (idx / kW) % kH, c = idx / (kW * kH);
    t[idx] = c * plane + kh * pitch + kw;
}

// The tap table padded to `count` entries: the entries beyond the taps repeat tap 0 (any valid offset would do: they
// address the scratch columns of a product run wider than its result, GemmProblem::j_store).
__global__ __launch_bounds__(256) void tap_table_padded_kernel(int *__restrict__ t, int planes, int kH, int kW, int plane,
                                                               int pitch, int count) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= count) return;
    const int k = idx < planes * kH * kW ? idx : 0;
    const int kw = k % kW, kh = (k / kW) % kH, c = k / (kW * kH);
    t[idx] = c * plane + kh * pitch + kw;
}

// t[(y, x)] = y*row_step + x*col_step
__global__ __launch_bounds__(256) void pixel_table_kernel(int *__restrict__ t, int Hn, int Wn, int row_step,
                                                          int col_step) {
    const int idx = blockIdx.x * 256 + threadIdx.x;
    if (idx >= Hn * Wn) return;
    t[idx] = (idx / Wn) * row_step + (idx % Wn) * col_step;
}

// Offset tables by geometry, built once on the device and kept for the life of the process (a few
// KB each).  Everything runs on the one library stream, so a table is complete before its first use.
using TableKey = std::array<int, 6>;
std::map<TableKey, int *> g_tables;

const int *table(int kind, int a, int b, int c, int d, int e, long count) {
    const TableKey key{kind, a, b, c, d, e};
    auto it = g_tables.find(key);
    if (it != g_tables.end()) return it->second;
    hipStream_t s = stream();
    if (!s) return nullptr;
    int *t = nullptr;
    hipError_t err = device_malloc(reinterpret_cast<void **>(&t), sizeof(int) * (size_t)count);
    if (err != hipSuccess) {
        (void)hipGetLastError();
        if (drop_cached_blocks()) err = device_malloc(reinterpret_cast<void **>(&t), sizeof(int) * (size_t)count);
    }
    if (err != hipSuccess) {
        (void)hipGetLastError();
        fail("offset table allocation of %ld entries failed", count);
        return nullptr;
    }
    const unsigned blocks = (unsigned)((count + 255) / 256);
    if (kind == 0)
        hipLaunchKernelGGL(tap_table_kernel, dim3(blocks), dim3(256), 0, s, t, a, b, c, d, e);
    else if (kind == 2)
        hipLaunchKernelGGL(tap_table_padded_kernel, dim3(blocks), dim3(256), 0, s, t, a, b, c, d, e, (int)count);
    else
        hipLaunchKernelGGL(pixel_table_kernel, dim3(blocks), dim3(256), 0, s, t, a, b, c, d);
    if (check_launch("conv offset table")) {
        device_free(t);
        return nullptr;
    }
    g_tables[key] = t;
    return t;
}

// Called once at the start of a convolution pass, before it takes its two tables: a caller cycling
// through many geometries starts the cache over (never between the two look-ups of one pass, which
// would free the first table under the pass that is about to use it).
int trim_tables() {
    if (g_tables.size() < 512) return 0;
    hipStream_t s = stream();
    if (!s) return 1;
    THGPU_HIP_TRY(hipStreamSynchronize(s));
    for (auto &kv : g_tables) device_free(kv.second);
    g_tables.clear();
    return 0;
}

const int *tap_table(int planes, int kH, int kW, int plane, int pitch) {
    return table(0, planes, kH, kW, plane, pitch, (long)planes * kH * kW);
}
const int *tap_table_padded(int planes, int kH, int kW, int plane, int pitch, int count) {
    // (the padded length is a function of the taps, so the key of kind 2 need not hold it)
    return table(2, planes, kH, kW, plane, pitch, count);
}
const int *pixel_table(int Hn, int Wn, int row_step, int col_step) {
    return table(1, Hn, Wn, row_step, col_step, 0, (long)Hn * Wn);
}

constexpr long kMaxExtent = 1L << 30;  // floats: the loaders address with 32-bit byte offsets

int g_mode = -1;

// The three products as GEMM problems, without pointers and tables (those are filled in by the launchers; a
// problem with `gathered` set is enough for the planner to say whether a tiled kernel takes it).
const int kNoTable = 0;  // stands in for a table where only the planner looks at the problem
constexpr int kNarrowestTile = 64;  // columns of the narrowest GEMM tile

GemmProblem forward_problem(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW) {
    const int Hp = H + 2 * pH, Wp = W + 2 * pW;
    const int Ho = (Hp - kH) / sH + 1, Wo = (Wp - kW) / sW + 1;
    const long N = (long)Ho * Wo;
    GemmProblem p;
    p.a_rc = true;
    p.sA = (long)C * kH * kW;
    p.rowtab = p.coltab = &kNoTable;
    p.bsB = (long)C * Hp * Wp;
    p.b_extent = B * p.bsB;
    p.sC = N;
    p.bsC = (long)M * N;
    p.M = M;
    p.J = (int)(B * N);
    p.N = (int)N;
    p.R = C * kH * kW;
    p.flops = 2.0 * M * (double)N * p.R * B;
    p.tag = "gemm_conv_fwd";
    return p;
}

GemmProblem gradweight_problem(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW) {
    const int Hp = H + 2 * pH, Wp = W + 2 * pW;
    const int Ho = (Hp - kH) / sH + 1, Wo = (Wp - kW) / sW + 1;
    const long N = (long)Ho * Wo;
    const int K = C * kH * kW;
    GemmProblem p;
    p.a_rc = true;
    p.sA = N;
    p.rbA = (long)M * N;
    p.rowtab = p.coltab = &kNoTable;
    p.rbB = (long)C * Hp * Wp;
    p.b_extent = B * p.rbB;
    p.sC = K;
    p.M = M;
    p.J = K;
    p.N = K;
    if (K < kNarrowestTile) {  // fewer taps than the narrowest tile has columns: run it that wide, store K of them
        p.J = p.N = kNarrowestTile;
        p.j_store = K;
    }
    p.R = (int)N;
    p.nb = (int)B;
    p.beta = 1.0f;
    p.flops = 2.0 * M * (double)N * K * B;
    p.tag = "gemm_conv_gradweight";
    return p;
}

// Unit stride only: one column per input pixel, one reduction index per (output plane, tap).
GemmProblem gradinput_problem(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW) {
    const int Ho = H + 2 * pH - kH + 1, Wo = W + 2 * pW - kW + 1;
    const int Hq = H + kH - 1, Wq = W + kW - 1;
    GemmProblem p;
    p.a_rc = true;
    p.sA = (long)M * kH * kW;
    p.rowtab = p.coltab = &kNoTable;
    p.bsB = (long)M * Hq * Wq;
    p.b_extent = B * p.bsB;
    p.sC = (long)H * W;
    p.bsC = (long)C * H * W;
    p.M = C;
    p.J = (int)(B * H * W);
    p.N = H * W;
    p.R = M * kH * kW;
    p.flops = 2.0 * M * (double)Ho * Wo * C * kH * kW * B;  // the convolution's own count: Ho*Wo <= H*W columns
    p.tag = "gemm_conv_gradinput";
    return p;
}

// Geometry of a strided layer's gradInput product (see the top of the file).
struct PhaseGeom {
    int A, Bk;     // taps per residue class: ceil(kH/sH), ceil(kW/sW)
    int Yn, Xn;    // cells per image: y = (h + pH) / sH over the image rows, likewise x
    int Hq, Wq;    // gradOutput padded by (A-1, Bk-1) in front and up to Yn + A - 1, Xn + Bk - 1 behind
    int rows, rows_pad;
};

PhaseGeom phase_geom(int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW) {
    PhaseGeom q;
    q.A = (kH + sH - 1) / sH;
    q.Bk = (kW + sW - 1) / sW;
    q.Yn = (H - 1 + pH) / sH + 1;
    q.Xn = (W - 1 + pW) / sW + 1;
    q.Hq = q.Yn + q.A - 1;
    q.Wq = q.Xn + q.Bk - 1;
    q.rows = C * sH * sW;
    q.rows_pad = q.rows < 64 ? 64 : q.rows;
    return q;
}

GemmProblem gradinput_strided_problem(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH,
                                      int sW) {
    const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
    const int Ho = (H + 2 * pH - kH) / sH + 1, Wo = (W + 2 * pW - kW) / sW + 1;
    GemmProblem p;
    p.a_rc = true;
    p.sA = (long)M * q.A * q.Bk;
    p.rowtab = p.coltab = &kNoTable;
    p.bsB = (long)M * q.Hq * q.Wq;
    p.b_extent = B * p.bsB;
    p.bsC = (long)C * H * W;
    p.M = q.rows_pad;
    p.J = (int)(B * q.Yn * q.Xn);
    p.N = q.Yn * q.Xn;
    p.R = M * q.A * q.Bk;
    p.c_w = q.Xn;
    p.scatter = true;
    p.scat_sH = sH;
    p.scat_sW = sW;
    p.scat_pH = pH;
    p.scat_pW = pW;
    p.scat_H = H;
    p.scat_W = W;
    p.scat_rows = q.rows;
    p.flops = 2.0 * M * (double)Ho * Wo * C * kH * kW * B;
    p.tag = "gemm_conv_gradinput";
    return p;
}

WeightJob bank_job(const float *weight, float *wt, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH,
                   int sW) {
    WeightJob wj;
    wj.w = weight;
    wj.wt = wt;
    wj.M = M;
    wj.C = C;
    wj.kH = kH;
    wj.kW = kW;
    if (sH != 1 || sW != 1) {
        const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
        wj.sH = sH;
        wj.sW = sW;
        wj.A = q.A;
        wj.Bk = q.Bk;
        wj.rows = q.rows;
        wj.rows_pad = q.rows_pad;
        wj.count = (unsigned)((long)q.rows_pad * M * q.A * q.Bk);
    } else {
        wj.sH = wj.sW = wj.A = wj.Bk = wj.rows = wj.rows_pad = 0;
        wj.count = (unsigned)((long)M * C * kH * kW);
    }
    return wj;
}

// The pending bank job, and the bank that the last carrier re-ordered (see side_jobs.h).  Two records: a convolution
// that consumes a carried job is, in the same call, the producer whose launch carries the next layer's.
WeightJob g_bank_job = {};
bool g_bank_pending = false;
const float *g_bank_carried = nullptr;

}  // namespace

void offer_bank_job(const WeightJob &job) {
    g_bank_job = job;
    g_bank_pending = job.count > 0;
    if (g_bank_carried == job.wt) g_bank_carried = nullptr;  // a record left over from a pass that never reached its product
}

bool take_bank_job(WeightJob &job) {
    if (!g_bank_pending) return false;
    job = g_bank_job;
    g_bank_pending = false;
    g_bank_carried = job.wt;
    return true;
}

bool bank_job_done(const float *wt) {
    const bool done = g_bank_carried == wt && wt != nullptr;
    g_bank_carried = nullptr;
    if (g_bank_pending && g_bank_job.wt == wt) g_bank_pending = false;  // nobody carried it: the product does it itself
    return done;
}

void conv_implicit_offer_bank(const float *weight, float *scratch, long B, int C, int H, int W, int M, int kH, int kW,
                              int pH, int pW, int sH, int sW) {
    int top, left, Hq, Wq;
    conv_implicit_q_layout(C, H, W, kH, kW, pH, pW, sH, sW, &top, &left, &Hq, &Wq);
    long nw = (long)M * C * kH * kW;
    if (sH != 1 || sW != 1) {
        const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
        nw = (long)q.rows_pad * M * q.A * q.Bk;
    }
    if (nw >= (1L << 31)) return;  // the product itself will refuse
    offer_bank_job(bank_job(weight, scratch + B * M * (long)Hq * Wq, C, H, W, M, kH, kW, pH, pW, sH, sW));
}

int conv_mode() {
    if (g_mode < 0) {
        const char *e = std::getenv("THGPU_CONV");
        g_mode = !e ? 1 : std::strcmp(e, "columns") == 0 ? 0 : std::strcmp(e, "gathered") == 0 ? 2 : 1;
    }
    return g_mode;
}

void conv_set_mode(int mode) { g_mode = mode; }

// Shapes the gathered GEMMs take: the padded batch must stay within 32-bit byte offsets and a tile of the fast
// kernel must take both products that share finput (the GEMM's own planner answers that: M, J >= 64, R >= 16,
// offsets of operands and output below 2^30 floats, a tile the tuning switches allow).
// Forward and gradWeight share finput (the padded input), so a layer takes both or neither.  K >= 16 is the GEMM's
// shortest reduction (forward); a gradWeight product with fewer than 64 taps runs 64 columns wide (gradweight_problem).
static bool forward_fits(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW) {
    const long Hp = H + 2L * pH, Wp = W + 2L * pW;
    const long Ho = (Hp - kH) / sH + 1, Wo = (Wp - kW) / sW + 1;
    const long K = (long)C * kH * kW, N = Ho * Wo;
    if (!(M >= 64 && K >= 16 && N >= 16 && B * N >= 64 && B * N < (1L << 31) && B * C * Hp * Wp < kMaxExtent)) return false;
    return gemm_tiled_fits(forward_problem(B, C, H, W, M, kH, kW, pH, pW, sH, sW)) &&
           gemm_tiled_fits(gradweight_problem(B, C, H, W, M, kH, kW, pH, pW, sH, sW));
}

static bool gradinput_fits(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW) {
    if (sH != 1 || sW != 1) {
        // by residue class of the pixel coordinates: any padding, rows padded to a whole tile
        const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
        const long cols = B * (long)q.Yn * q.Xn;
        if (!(cols >= 64 && cols < (1L << 31) && (long)M * q.A * q.Bk >= 16 && B * M * (long)q.Hq * q.Wq < kMaxExtent &&
              (long)q.rows_pad * cols < (1L << 31)))
            return false;
        return gemm_tiled_fits(gradinput_strided_problem(B, C, H, W, M, kH, kW, pH, pW, sH, sW));
    }
    if (kH - 1 - pH < 0 || kW - 1 - pW < 0) return false;
    const long Hq = H + kH - 1, Wq = W + kW - 1;
    if (!(C >= 64 && B * H * W >= 64 && (long)M * kH * kW >= 16 && B * M * Hq * Wq < kMaxExtent &&
          B * (long)H * W < (1L << 31)))
        return false;
    return gemm_tiled_fits(gradinput_problem(B, C, H, W, M, kH, kW, pH, pW));
}

// Where the gathered route pays (measured on the AlexNet-, OverFeat- and VGG-style layers and the reference's
// benchmark set).  Forward and gradWeight: wherever a tiled kernel takes the product -- the gathered products run at
// the rate of those on columns (0.84 - 0.92 of the matrix peak on the 512- and 1024-plane layers, either way), and
// the columns' trip through memory is saved.  gradInput: the gathered product has one row per input plane, so it
// wants C to fill its 64-row tiles, and one column per input pixel, so it wants the layer padded (see below).
bool conv_use_gathered(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW) {
    const int mode = conv_mode();
    if (mode == 0 || !forward_fits(B, C, H, W, M, kH, kW, pH, pW, sH, sW)) return false;
    return true;
}

bool conv_use_gathered_gradinput(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW) {
    const int mode = conv_mode();
    if (mode == 0 || !gradinput_fits(B, C, H, W, M, kH, kW, pH, pW, sH, sW)) return false;
    if (mode == 2) return true;
    if (sH != 1 || sW != 1) {
        // The product by residue class executes rows_pad*A*Bk*sH*sW / (C*kH*kW) times the layer's flops (rows
        // padded to a tile, taps rounded up to whole strides) but saves the gradient columns, kH*kW/(sH*sW) times
        // the input written and read back: it pays while that excess stays small.
        const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
        const double excess = (double)q.rows_pad * q.A * q.Bk / ((double)C * kH * kW);
        return excess <= 2.0;
    }
    const long rows = (C + 63L) / 64 * 64;
    // An unpadded (or lightly padded) layer has fewer output positions than input pixels, and the gathered
    // product computes one column per input pixel: it executes H*W / (Ho*Wo) times the layer's flops, where the
    // column route pays the algorithmic flops plus the gradient columns' trip through memory (8*K*N bytes per
    // image).  At the measured rates (120 TFLOP/s, 4.5 TB/s) the columns win once (H*W/(Ho*Wo) - 1) * M exceeds
    // about 100; measured on the reference benchmark's unpadded layers, the switch-over lies between 100 (gathered
    // still 9 % ahead) and 150 (columns 19 % ahead).
    const long Ho = H + 2L * pH - kH + 1, Wo = W + 2L * pW - kW + 1;
    const bool inflation_ok = ((long)H * W - Ho * Wo) * M <= 110 * Ho * Wo;
    return rows * 8 <= C * 9L && inflation_ok;
}

long conv_implicit_gradinput_scratch(long B, int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH,
                                     int sW) {
    if (sH != 1 || sW != 1) {
        const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
        return B * M * (long)q.Hq * q.Wq + (long)q.rows_pad * M * q.A * q.Bk;
    }
    return B * M * (H + kH - 1L) * (W + kW - 1L) + (long)C * M * kH * kW;
}

// out[plane][y][x] = in[plane][y - top][x - left], zero outside the H x W source; out planes are Hp x Wp.  With a
// weight job the same launch also re-orders the kernel bank.
static int pad_planes_into(const float *in, long planes, int H, int W, int top, int left, long Hp, long Wp, float *out,
                           const WeightJob *wj = nullptr) {
    hipStream_t s = stream();
    if (!s) return 1;
    const long total = planes * Hp * Wp;
    if (total <= 0 && !wj) return 0;
    if (total >= (1L << 31)) return fail("pad: %ld elements exceed 32-bit indexing", total);
    {
        const char *label = planes == 0 ? "kernel_bank_reorder"
                            : prof_enabled() ? prof_label("pad_planes planes=%ld %dx%d p=%dx%d", planes, H, W, top, left)
                                             : "pad_planes";
        const double wbytes = wj ? 4.0 * (wj->count + (double)wj->M * wj->C * wj->kH * wj->kW) : 0.0;
        LaunchScope scope(label, 0.0, 4.0 * (total + planes * H * W) + wbytes);
        PadJob pj;
        pj.in = in;
        pj.out = out;
        pj.total = (unsigned)total;
        pj.H = H;
        pj.W = W;
        pj.pH = top;
        pj.pW = left;
        pj.Hp = (int)Hp;
        pj.Wp = (int)Wp;
        pj.divWp = FastDiv((uint32_t)Wp);
        pj.divHp = FastDiv((uint32_t)Hp);
        pj.aligned = (reinterpret_cast<uintptr_t>(out) & 15) == 0;
        const unsigned pad_blocks = (unsigned)((total + 1023) / 1024);
        if (wj) {
            const unsigned wblocks = (wj->count + 255u) / 256u;
            hipLaunchKernelGGL(pad_planes_and_weights_kernel, dim3(pad_blocks + wblocks), dim3(256), 0, s, pj, pad_blocks,
                               *wj);
        } else {
            hipLaunchKernelGGL(pad_planes_kernel, dim3(pad_blocks), dim3(256), 0, s, pj);
        }
    }
    return check_launch("pad_planes");
}

void conv_implicit_q_layout(int C, int H, int W, int kH, int kW, int pH, int pW, int sH, int sW, int *top, int *left,
                            int *Hq, int *Wq) {
    if (sH != 1 || sW != 1) {
        const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
        *top = q.A - 1;
        *left = q.Bk - 1;
        *Hq = q.Hq;
        *Wq = q.Wq;
        return;
    }
    *top = kH - 1 - pH;
    *left = kW - 1 - pW;
    *Hq = H + kH - 1;
    *Wq = W + kW - 1;
}

int pad_planes_launch(const float *in, long planes, int H, int W, int pH, int pW, float *out) {
    return pad_planes_into(in, planes, H, W, pH, pW, H + 2L * pH, W + 2L * pW, out);
}

int conv_implicit_forward(const float *padded, const float *weight, const float *bias, float *output, long B, int C,
                          int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW, OutputThreshold act,
                          OutputLayout out) {
    const int Hp = H + 2 * pH, Wp = W + 2 * pW;
    const int Ho = (Hp - kH) / sH + 1, Wo = (Wp - kW) / sW + 1;
    if (trim_tables()) return 1;
    GemmProblem p = forward_problem(B, C, H, W, M, kH, kW, pH, pW, sH, sW);
    p.A = weight;
    p.B = padded;
    p.rowtab = tap_table(C, kH, kW, Hp * Wp, Wp);
    p.coltab = pixel_table(Ho, Wo, sH * Wp, sW);
    if (!p.rowtab || !p.coltab) return 1;
    if (conv_narrow_forward_fits(B, M, (long)C * kH * kW, Wo, (long)Ho * Wo, sW, out))
        return conv_narrow_forward(padded, (long)C * Hp * Wp, weight, bias, output, B, M, C * kH * kW, Ho, Wo, sH * Wp,
                                   p.rowtab, act);
    p.C = output;
    p.bias = bias;
    p.act = act.on;
    p.act_threshold = act.threshold;
    p.act_value = act.value;
    if (out.plane > 0) {
        p.sC = out.plane;
        p.bsC = (long)M * out.plane;
    }
    if (out.pitch > 0) {
        p.c_pitch = out.pitch;
        p.c_w = Wo;
    }
    return gemm_launch(p);
}

int conv_implicit_gradweight(const float *padded, const float *gradOutput, float *gradWeight, long B, int C, int H,
                             int W, int M, int kH, int kW, int pH, int pW, int sH, int sW, float scale, float *gradBias,
                             bool *bias_done) {
    const int Hp = H + 2 * pH, Wp = W + 2 * pW;
    const int Ho = (Hp - kH) / sH + 1, Wo = (Wp - kW) / sW + 1;
    if (trim_tables()) return 1;
    if (conv_narrow_gradweight_fits(B, M, (long)C * kH * kW, Wo, (long)Ho * Wo, sW)) {
        const int *taps = tap_table(C, kH, kW, Hp * Wp, Wp);
        if (!taps) return 1;
        if (bias_done) *bias_done = gradBias != nullptr;
        return conv_narrow_gradweight(padded, (long)C * Hp * Wp, gradOutput, gradWeight, gradBias, B, M, C * kH * kW, Ho,
                                      Wo, sH * Wp, taps, scale);
    }
    GemmProblem p = gradweight_problem(B, C, H, W, M, kH, kW, pH, pW, sH, sW);
    p.A = gradOutput;
    p.B = padded;
    p.rowtab = pixel_table(Ho, Wo, sH * Wp, sW);
    p.coltab = p.j_store > 0 ? tap_table_padded(C, kH, kW, Hp * Wp, Wp, p.J) : tap_table(C, kH, kW, Hp * Wp, Wp);
    if (!p.rowtab || !p.coltab) return 1;
    p.C = gradWeight;
    p.alpha = scale;
    p.rowsum = gradBias;  // gradBias[m] += scale * sum of gradOutput[.][m][.]: the row sums of this product's A
    p.rowsum_done = bias_done;
    return gemm_launch(p);
}

// gradInput of a strided layer as one product over the residue classes of the pixel coordinates.
static int conv_implicit_gradinput_strided(const float *gradOutput, const float *weight, float *scratch,
                                           float *gradInput, long B, int C, int H, int W, int M, int kH, int kW, int pH,
                                           int pW, int sH, int sW, InputMask mask, bool q_ready) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (mask.in && (mask.pitch > 0 || (mask.plane > 0 && mask.plane != (long)H * W)))
        return fail("SpatialConvolutionMM: the strided gradInput product takes a densely packed mask only");
    const PhaseGeom q = phase_geom(C, H, W, kH, kW, pH, pW, sH, sW);
    const int Ho = (H + 2 * pH - kH) / sH + 1, Wo = (W + 2 * pW - kW) / sW + 1;
    float *Q = scratch;
    float *Wt = scratch + B * M * (long)q.Hq * q.Wq;
    const long nw = (long)q.rows_pad * M * q.A * q.Bk;
    if (nw >= (1L << 31)) return fail("SpatialConvolutionMM: kernel bank too large for the strided gradInput product");
    const WeightJob wj = bank_job(weight, Wt, C, H, W, M, kH, kW, pH, pW, sH, sW);
    // With gradOutput already in place only the kernel bank is re-ordered (zero planes to pad), unless a launch before
    // this one has carried that job along.
    const bool bank_done = bank_job_done(Wt);
    if (!(q_ready && bank_done) &&
        pad_planes_into(gradOutput, q_ready ? 0 : B * M, Ho, Wo, q.A - 1, q.Bk - 1, q.Hq, q.Wq, Q, &wj))
        return 1;
    if (trim_tables()) return 1;
    GemmProblem p = gradinput_strided_problem(B, C, H, W, M, kH, kW, pH, pW, sH, sW);
    p.A = Wt;
    p.B = Q;
    p.rowtab = tap_table(M, q.A, q.Bk, q.Hq * q.Wq, q.Wq);
    p.coltab = pixel_table(q.Yn, q.Xn, q.Wq, 1);
    if (!p.rowtab || !p.coltab) return 1;
    p.C = gradInput;
    p.mask = mask.in;
    p.mask_threshold = mask.threshold;
    return gemm_launch(p);
}

int conv_implicit_gradinput(const float *gradOutput, const float *weight, float *scratch, float *gradInput, long B,
                            int C, int H, int W, int M, int kH, int kW, int pH, int pW, int sH, int sW, InputMask mask,
                            bool q_ready, TwinOutput twin, bool *wrote_twin) {
    if (wrote_twin) *wrote_twin = false;
    if (sH != 1 || sW != 1)  // (the scattered store keeps no second copy)
        return conv_implicit_gradinput_strided(gradOutput, weight, scratch, gradInput, B, C, H, W, M, kH, kW, pH, pW, sH,
                                               sW, mask, q_ready);
    hipStream_t s = stream();
    if (!s) return 1;
    const int Ho = H + 2 * pH - kH + 1, Wo = W + 2 * pW - kW + 1;
    const int qH = kH - 1 - pH, qW = kW - 1 - pW;
    const int Hq = Ho + 2 * qH, Wq = Wo + 2 * qW;  // = H + kH - 1, W + kW - 1
    float *Q = scratch;
    float *Wt = scratch + B * M * (long)Hq * Wq;
    const long nw = (long)M * C * kH * kW;
    if (nw >= (1L << 31)) return fail("SpatialConvolutionMM: kernel bank too large for the gradInput product");
    const WeightJob wj = bank_job(weight, Wt, C, H, W, M, kH, kW, pH, pW, sH, sW);
    const bool bank_done = bank_job_done(Wt);
    if (!(q_ready && bank_done) && pad_planes_into(gradOutput, q_ready ? 0 : B * M, Ho, Wo, qH, qW, Hq, Wq, Q, &wj))
        return 1;
    if (trim_tables()) return 1;
    GemmProblem p = gradinput_problem(B, C, H, W, M, kH, kW, pH, pW);
    p.A = Wt;
    p.B = Q;
    p.rowtab = tap_table(M, kH, kW, Hq * Wq, Wq);
    p.coltab = pixel_table(H, W, Wq, 1);
    if (!p.rowtab || !p.coltab) return 1;
    p.C = gradInput;
    p.mask = mask.in;
    p.mask_threshold = mask.threshold;
    if (mask.in && mask.plane > 0) {
        p.mask_sC = mask.plane;
        p.mask_bsC = (long)C * mask.plane;
    }
    if (mask.in && mask.pitch > 0) {
        p.mask_pitch = mask.pitch;
        p.c_w = W;
    }
    if (twin.base) {
        p.C2 = twin.base;
        p.c2_sC = twin.plane;
        p.c2_bsC = (long)C * twin.plane;
        p.c2_pitch = twin.pitch;
        p.c_w = W;
        if (!gemm_tiled_fits(p)) p.C2 = nullptr;  // the copy's offsets exceed the kernels' addressing: do without
        if (wrote_twin) *wrote_twin = p.C2 != nullptr;
    }
    return gemm_launch(p);
}

}  // namespace thgpu

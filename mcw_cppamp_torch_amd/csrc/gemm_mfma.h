// fp32 GEMM on CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), shared by
// THGPUBlas_gemm and the three GEMMs of nn.SpatialConvolutionMM.
//
// The kernels compute, in row-major terms with the output contiguous along j,
//     C(i, j) = alpha * sum_r A(i, r) * B(r, j)  [+ beta * C(i, j)]  [+ bias(i)]
// with each operand contiguous either along the reduction index r or along
// its free index.  Two batching schemes cover the convolution:
//   * column batching: j enumerates (image, n) pairs, j = image*N + n; B and C
//     take a per-image stride, A is shared (forward and gradInput);
//   * reduction batching: r enumerates (image, n) pairs and both operands
//     take a per-image stride (gradWeight).
// The reduction can be split over several workgroups; the partial sums go to a
// workspace and a second kernel adds them in a fixed order, so results are
// reproducible run to run (no atomics anywhere).
#pragma once

#include "common.h"

namespace thgpu {

struct GemmProblem {
    const float *A = nullptr;
    const float *B = nullptr;
    float *C = nullptr;
    const float *bias = nullptr;  // added per output row i when non-null
    int M = 0;                    // rows of C
    int J = 0;                    // columns of C (all images together in column batching)
    int R = 0;                    // reduction length (per image in reduction batching)
    bool a_rc = true;             // A contiguous along r (else along i)
    bool b_rc = false;            // B contiguous along r (else along j)
    // Gathered B (implicit im2col): B(r, j) = B[image(j)*bsB + rowtab[r] + coltab[n(j)]] (with reduction batching:
    // B[image*rbB + rowtab[r] + coltab[j]]).  Needs !b_rc, a_rc and a shape the tiled kernel takes; sB is unused.
    const int *rowtab = nullptr;  // R entries (floats)
    const int *coltab = nullptr;  // N entries (floats)
    long b_extent = 0;            // floats addressable from B (gathered B only; checked against 32-bit offsets)
    long sA = 0;                  // the non-unit stride of A
    long sB = 0;                  // the non-unit stride of B
    long sC = 0;                  // row stride of C
    // column batching (N = columns per image; N == J means a single image)
    int N = 0;
    long bsB = 0, bsC = 0;        // per-image strides of B and C
    // reduction batching (nb images, per-image strides of A and B)
    int nb = 1;
    long rbA = 0, rbB = 0;
    float alpha = 1.0f, beta = 0.0f;
    // Fused into the store of the final value (after alpha, bias and beta), in this order:
    //   act:  C = C > act_threshold ? C : act_value          (nn.Threshold applied to a convolution's output)
    //   mask: C = mask[same offset as C] > mask_threshold ? C : 0
    //         (nn.Threshold's backward applied to a convolution's gradInput; mask is laid out exactly like C)
    bool act = false;
    float act_threshold = 0.0f, act_value = 0.0f;
    const float *mask = nullptr;
    float mask_threshold = 0.0f;
    // Column batching only: the N columns of an image are an image plane of width c_w, and C / mask keep it with
    // rows c_pitch / mask_pitch floats apart (0: densely, column n at offset n): a result written into the
    // interior of a zero-bordered buffer, a mask read from one.  The mask takes its own row and image strides
    // (0: those of C).
    int c_w = 0, c_pitch = 0, mask_pitch = 0;
    long mask_sC = 0, mask_bsC = 0;
    // Column batching with c_w set: a second copy of every final value (after alpha, bias, beta, act and mask) goes to
    // C2, element (row i, image, y, x) at C2[image*c2_bsC + i*c2_sC + y*c2_pitch + x] -- the same image planes kept
    // in another layout, e.g. the interior of a zero-bordered buffer that the next product gathers from, so that no
    // padded copy of C has to be made afterwards.  nullptr: off.  Not with a scattered store.
    float *C2 = nullptr;
    long c2_sC = 0, c2_bsC = 0;
    int c2_pitch = 0;
    // Scattered store (column batching, no bias, beta = 0, never split): row i of the product is a (plane, row
    // phase, column phase) triple, i = (c*scat_sH + ph)*scat_sW + pw, column n of an image a cell (y, x) of a grid
    // c_w wide, and element (i, (image, y, x)) goes to
    //     C[image*bsC + c*scat_H*scat_W + h*scat_W + w],   h = y*scat_sH + ph - scat_pH,  w = x*scat_sW + pw - scat_pW,
    // when 0 <= h < scat_H, 0 <= w < scat_W and i < scat_rows; every other element is dropped.  This is how the
    // gradInput of a strided convolution leaves its GEMM: one row per residue class of the pixel coordinates modulo
    // the strides.  A mask is read at the same offsets (it is laid out exactly like C).  sC is unused.
    bool scatter = false;
    int scat_sH = 1, scat_sW = 1, scat_pH = 0, scat_pW = 0, scat_H = 0, scat_W = 0, scat_rows = 0;
    // Reduction batching only: rowsum[i] += alpha * sum over the whole reduction of A(i, r), computed by the product's
    // own workgroups from the first-operand tiles they load anyway (the bias gradient of a convolution is this sum
    // over gradOutput).  *rowsum_done tells whether the launch took it on (a tiled reduction-batched kernel ran);
    // when it is false the caller computes the sums itself.
    float *rowsum = nullptr;
    bool *rowsum_done = nullptr;
    // Products whose columns are not batched over images (N == J: gradWeight): computed J columns wide, but only the
    // first j_store of them exist in C (rows of C are sC >= j_store floats apart); the rest are scratch.  This is how a product with fewer columns than
    // the narrowest tile runs on the tiled kernels: its column table is padded with entries that repeat a valid one.
    // The reduction is always split (the partial sums are J wide, the final pass stores j_store).  0: all J columns.
    int j_store = 0;
    const char *tag = "gemm";     // name used by per-kernel timing
    // Flops the per-kernel timing credits the launch with; 0 means the product's own 2*M*J*R*nb.  A
    // convolution pass sets its algorithmic 2*M*N*K*B here, which a gathered gradInput product (one
    // column per input pixel) can exceed.
    double flops = 0.0;
    // When non-null the split reduction keeps its partial sums in this caller-provided device buffer of
    // ws_fixed_floats floats instead of the library's grow-only workspace, and only splits that fit it
    // are considered: the launch then allocates nothing.
    float *ws_fixed = nullptr;
    long ws_fixed_floats = 0;
};

// Enqueues the GEMM on the library stream.  Returns 0 or a recorded error.
int gemm_launch(const GemmProblem &p);
// Whether one of the tiled kernels takes the problem (shape at least a tile, operand and output offsets
// within the kernels' 32-bit addressing, a tile the tuning switches allow): the test a gathered second
// operand, which has no generic kernel, must pass before it is launched.
bool gemm_tiled_fits(const GemmProblem &p);

// ---- shared between the kernel translation units ------------------------------

constexpr int GEMM_BK = 16;  // reduction step of every kernel

struct GemmArgs {
    const float *A;
    const float *B;
    float *C;
    const float *bias;
    float *ws;  // partial sums [nsplit][M][J] when nsplit > 1
    const int *rowtab, *coltab;  // gathered B
    int M, J, R, N;
    long sA, sB, sC, bsB, bsC, rbA, rbB;
    int nb;
    int steps_per_img;    // ceil(R / GEMM_BK)
    int steps_per_split;  // reduction steps one workgroup walks
    int steps_total;      // nb * steps_per_img
    int nsplit;
    unsigned tilesM, tilesJ, total;
    FastDiv divN, divTilesM, divTilesJ, divSpi;
    float alpha, beta;
    int act;  // see GemmProblem
    float act_threshold, act_value;
    const float *mask;
    float mask_threshold;
    int c_w, c_pitch, mask_pitch;
    long mask_sC, mask_bsC;
    FastDiv divCW;
    float *C2;  // see GemmProblem
    long c2_sC, c2_bsC;
    int c2_pitch;
    int scatter;  // see GemmProblem
    int scat_sH, scat_sW, scat_pH, scat_pW, scat_H, scat_W, scat_rows;
    FastDiv divScatS, divScatW;  // a row index by sH*sW and its remainder by sW
    float *rowsum_ws;            // partial row sums of A, [M][nsplit * tilesJ], or null
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

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

// How an operand tile travels from global memory to LDS.
enum Loader {
    LD_RC_VEC = 0,     // contiguous along r: 128-bit loads along r (rows need 4-byte alignment only)
    LD_RC_SCALAR = 1,  // contiguous along r: 16 lanes read 16 consecutive r, one float each
    LD_XC_SCALAR = 2,  // contiguous along the free index: lanes read consecutive rows/columns
    // 3 is used inside the kernel (block-wise x-contiguous loads of a 192-row first operand)
    LD_XC_GATHER = 4,  // second operand only: element (r, x) at rowtab[r] + coltab[x]; lanes run along x
};

// Launch one tile configuration of the fast kernel (gemm_fast.h).  la/lb are
// Loader values; returns 0 or a recorded error.
int gemm_fast_128x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_192x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_128x256(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_256x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_64x64(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_64x256(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_64x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_96x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);  // first operand along r only
// Short-row variants: 48 of the tile's 64 rows multiplied (scattered products of a gathered B only).
int gemm_fast_48x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
int gemm_fast_48x256(const GemmArgs &g, int la, int lb, bool red, hipStream_t s);
// The bounds-checked kernel for shapes smaller than a tile (gemm_generic.hip).
int gemm_generic_64x64(const GemmArgs &g, bool a_rc, bool b_rc, bool red, hipStream_t s);

}  // namespace thgpu

// fp32 GEMM on CDNA4 matrix cores (v_mfma_f32_32x32x2_f32), shared by
// THGPUBlas_gemm and the three GEMMs of nn.SpatialConvolutionMM.
//
// The kernel computes, in row-major terms with the output contiguous along j,
//     C(i, j) = alpha * sum_r A(i, r) * B(r, j)  [+ beta * C(i, j)]  [+ bias(i)]
// with each operand contiguous either along the reduction index r or along
// its free index.  Two batching schemes cover the convolution:
//   * column batching: j enumerates (image, n) pairs, j = image*N + n; B and C
//     take a per-image stride, A is shared (forward and gradInput);
//   * reduction batching: r enumerates (image, n) pairs and both operands
//     take a per-image stride (gradWeight); the image range can be split over
//     several workgroups that write partial sums to a workspace which a
//     second kernel adds in a fixed order, so results are reproducible.
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
    const char *tag = "gemm";     // name used by per-kernel timing
};

// Enqueues the GEMM on the library stream.  Returns 0 or a recorded error.
int gemm_launch(const GemmProblem &p);

}  // namespace thgpu

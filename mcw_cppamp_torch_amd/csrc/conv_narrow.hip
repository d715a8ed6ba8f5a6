// Convolution forward for layers with a handful of taps (K = C*kH*kW <= 32: a 3x3 kernel on the three planes of an
// image) and 64 output planes.  As a GEMM such a layer is two reduction steps long, and a tiled kernel spends its
// time on the fixed cost of each tile (operands through LDS, barriers, prologue, epilogue) while the layer's real
// work is writing its output: 64 planes of H*W floats per image from 3 (VGG-A's first layer at batch 64: 822 MB
// written, 39 MB read, 11 GFLOP).  This kernel is built for that shape:
//   * the weights stay in registers for the whole launch as MFMA operands (v_mfma_f32_32x32x2_f32: lane (i, h) holds
//     W[i][2s + h] for step s and row block), so nothing is staged through LDS and there is no barrier in the loop;
//   * a wavefront walks groups of 128 consecutive output positions of a plane as four interleaved column blocks:
//     lane (j, h) owns positions 4j .. 4j+3 of the group, one in each block, and fetches their operands
//     P[tap(2s + h) + pixel(4j ..)] of the zero-padded image with ONE 16-byte load per step (unit column stride: the
//     four positions are neighbours in the image row; the image is small and stays in the caches);
//   * every output plane then leaves as 16 bytes per lane, 512 contiguous bytes per plane and store: full cache lines
//     in few requests, which is what a kernel whose work is its stores needs.
// The sums run over the same products as the GEMM's (the order of the additions differs: tolerance parity, exact on
// integers).  Reference: the forward pass of gpunn-impl/SpatialConvolutionMM.cpp:130-228.
#include "common.h"
#include "kernels.h"

namespace thgpu {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));
struct __attribute__((packed, aligned(4))) float4u {  // four floats at a 4-byte aligned address
    float x, y, z, w;
};

constexpr int kNarrowSteps = 16;  // at most 16 reduction steps of two taps: K <= 32
constexpr int kNarrowGroup = 128;  // output positions a wavefront takes at a time

struct NarrowGeom {
    const float *P;      // zero-padded images, image_stride floats apart
    const float *Wt;     // [64][K]
    const float *bias;   // [64] or null
    float *out;          // [B][64][N]
    const int *rowtab;   // [K]: offset of a tap in the padded image
    int K, N;            // taps; output positions per plane (Ho * Wo)
    int row_step;        // output position (y, x) reads the padded image from y * row_step + x on
    FastDiv divWo;
    long image_stride;
    unsigned groups;     // B * N / 128
    FastDiv divGroupsPerImage;
    bool act;
    float act_threshold, act_value;
};

// KS: reduction steps, the smallest even number with 2*KS >= K (so that only the last two steps can hold a tap
// beyond K, and no step is skipped at run time: a branch between the MFMAs costs a copy of every accumulator).
template <int KS>
__global__ __launch_bounds__(256, 2) void conv_narrow_forward_kernel(const NarrowGeom g) {
    const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
    const unsigned wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    const unsigned waves = gridDim.x * 4u;

    // ---- per launch: the weights as MFMA operands, the lane's tap offsets -------------------------------------------
    float a[2][KS];
    unsigned tap[KS];  // byte offsets
    bool live[KS];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        const int k = 2 * s + half;
        live[s] = k < g.K;
        const int kk = live[s] ? k : 0;
        tap[s] = (unsigned)g.rowtab[kk] * 4u;
#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
            const float w = g.Wt[(long)(rb * 32 + col) * g.K + kk];
            a[rb][s] = live[s] ? w : 0.0f;
        }
    }
    // Accumulator register v of lane (j, h) holds output plane 8*(v/4) + 4*h + v%4 (+32 for the second row block).
    // Registers are scarce here (128 accumulators), so neither the 32 bias values nor the store offsets of a lane are
    // kept in them: the bias sits in LDS (one read per store, the LDS has nothing else to do), and a store's address
    // is a scalar base per plane pair plus ONE per-lane offset.
    __shared__ float sbias[64];
    if (threadIdx.x < 64) sbias[threadIdx.x] = g.bias ? g.bias[threadIdx.x] : 0.0f;
    __syncthreads();
    const float *lane_bias = sbias + 4 * half;
    const unsigned lane_off = ((unsigned)(4 * half) * (unsigned)g.N + 4u * (unsigned)col) * 4u;

    float4u bv[KS];
    auto request = [&](unsigned grp) {
        unsigned img, gi;
        g.divGroupsPerImage.divmod(grp, img, gi);
        // a wavefront-uniform base and a 32-bit byte offset per lane: no 64-bit address arithmetic per load
        const char *image = reinterpret_cast<const char *>(g.P + (long)img * g.image_stride);
        unsigned y, x;
        g.divWo.divmod(gi * (unsigned)kNarrowGroup + 4u * (unsigned)col, y, x);  // (Wo is a multiple of 4: one row)
        const unsigned pixel = (y * (unsigned)g.row_step + x) * 4u;
#pragma unroll
        for (int s = 0; s < KS; ++s) bv[s] = *reinterpret_cast<const float4u *>(image + (pixel + tap[s]));
    };
    unsigned grp = wave;
    if (grp < g.groups) request(grp);
    while (grp < g.groups) {
        unsigned img, gi;
        g.divGroupsPerImage.divmod(grp, img, gi);
        float16v acc[4][2];
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int rb = 0; rb < 2; ++rb)
#pragma unroll
                for (int v = 0; v < 16; ++v) acc[q][rb][v] = 0.0f;
#pragma unroll
        for (int s = 0; s < KS; ++s) {
            // a tap beyond K multiplies nothing (weight 0), and the operand fetched for it (a repeat of tap 0) is
            // zeroed too, so that an infinity there stays out of the sum; only the last two steps can hold one
            float4u b = bv[s];
            if (s >= KS - 2 && !live[s]) b.x = b.y = b.z = b.w = 0.0f;
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                acc[0][rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][s], b.x, acc[0][rb], 0, 0, 0);
                acc[1][rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][s], b.y, acc[1][rb], 0, 0, 0);
                acc[2][rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][s], b.z, acc[2][rb], 0, 0, 0);
                acc[3][rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][s], b.w, acc[3][rb], 0, 0, 0);
            }
        }
        // The next group's operands are requested BEFORE this group's stores go out (into the registers the
        // multiplications above have just finished with): memory operations complete in order as far as the wait
        // counter knows, so a request issued behind the stores could not be used before every store had landed.
        const unsigned next = grp + waves;
        if (next < g.groups) request(next);

#pragma unroll
        for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                // plane 32*rb + 8*(v/4) + v%4 (lanes of the upper half: 4 planes further) of image img, the group's
                // first position: a wavefront-uniform base
                const int plane = rb * 32 + 8 * (v / 4) + (v % 4);
                char *base = reinterpret_cast<char *>(g.out + ((long)img * 64 + plane) * g.N + (long)gi * kNarrowGroup);
                const float bz = lane_bias[plane];
                float4u val;
                val.x = acc[0][rb][v] + bz;
                val.y = acc[1][rb][v] + bz;
                val.z = acc[2][rb][v] + bz;
                val.w = acc[3][rb][v] + bz;
                if (g.act) {
                    val.x = val.x > g.act_threshold ? val.x : g.act_value;
                    val.y = val.y > g.act_threshold ? val.y : g.act_value;
                    val.z = val.z > g.act_threshold ? val.z : g.act_value;
                    val.w = val.w > g.act_threshold ? val.w : g.act_value;
                }
                *reinterpret_cast<float4u *>(base + lane_off) = val;
            }
        }
        grp = next;
    }
}

// ---- gradWeight of the same layers ----------------------------------------------------------------------------------
// gradWeight[m][k] += scale * sum over images and positions n of gradOutput[m][n] * P[tap(k) + pixel(n)]: 64 x K results
// from a reduction over every output position of the batch.  As a tiled GEMM it runs 64 columns wide for K taps, split
// a thousand ways.  Here the work is what it is -- reading gradOutput once -- and the results never leave the
// registers until the end: a wavefront owns a 64 x 32 block of accumulators (rows m, columns k) for the whole launch
// and walks blocks of 32 positions; lane (i, h) fetches four consecutive positions of row i of gradOutput with one
// 16-byte load (positions 4h .. 4h+3 of every eight: the first operand of four MFMA steps), lane (j, h) the same four
// positions of the padded image at tap j (the second operand), so both operands pair the same positions.  The lanes
// also add up what they fetch of gradOutput: the row sums are the bias gradient.  Every wavefront leaves its 64 x 32
// partial sums and 64 x 2 partial row sums in the workspace, and a second small launch adds them in wavefront order
// (a fixed order: results do not depend on timing) into gradWeight and gradBias.
struct NarrowGradGeom {
    const float *P;      // zero-padded images, image_stride floats apart
    const float *go;     // gradOutput [B][64][N]
    float *partial;      // [waves][64 * 32 + 64 * 2]
    const int *rowtab;   // [K]
    int K, N;
    int row_step;
    FastDiv divWo;
    long image_stride;
    unsigned blocks;     // B * N / 32
    FastDiv divBlocksPerImage;
};

constexpr int kNarrowPartial = 64 * 32 + 64 * 2;

__global__ __launch_bounds__(256) void conv_narrow_gradweight_kernel(const NarrowGradGeom g) {
    const int lane = threadIdx.x & 63, col = lane & 31, half = lane >> 5;
    const unsigned wave = __builtin_amdgcn_readfirstlane(blockIdx.x * 4u + (threadIdx.x >> 6));
    const unsigned waves = gridDim.x * 4u;
    const unsigned tap = (unsigned)g.rowtab[col < g.K ? col : 0] * 4u;  // (columns beyond K: any valid tap; never stored)
    // row `col` (+32) of gradOutput, positions 4*half on: byte offset within an image's gradOutput
    const unsigned go_lane = ((unsigned)col * (unsigned)g.N + 4u * (unsigned)half) * 4u;

    float4u av[2][4], bv[4];
    auto request = [&](unsigned blk) {
        unsigned img, bi;
        g.divBlocksPerImage.divmod(blk, img, bi);
        const char *rows = reinterpret_cast<const char *>(g.go + (long)img * 64 * g.N + (long)bi * 32);
        const char *image = reinterpret_cast<const char *>(g.P + (long)img * g.image_stride);
#pragma unroll
        for (int c = 0; c < 4; ++c) {  // eight positions at a time: this half's four
            av[0][c] = *reinterpret_cast<const float4u *>(rows + (go_lane + (unsigned)c * 32u));
            av[1][c] = *reinterpret_cast<const float4u *>(rows + (go_lane + (unsigned)c * 32u + 32u * (unsigned)g.N * 4u));
            unsigned y, x;
            g.divWo.divmod(bi * 32u + (unsigned)c * 8u + 4u * (unsigned)half, y, x);  // (Wo is a multiple of 4: one row)
            bv[c] = *reinterpret_cast<const float4u *>(image + ((y * (unsigned)g.row_step + x) * 4u + tap));
        }
    };

    float16v acc[2];
    float rowsum[2] = {0.0f, 0.0f};
#pragma unroll
    for (int rb = 0; rb < 2; ++rb)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[rb][v] = 0.0f;
    unsigned blk = wave;
    if (blk < g.blocks) request(blk);
    while (blk < g.blocks) {
        float4u a[2][4], b[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            a[0][c] = av[0][c];
            a[1][c] = av[1][c];
            b[c] = bv[c];
        }
        const unsigned next = blk + waves;
        if (next < g.blocks) request(next);  // the next block's operands are on their way during this block's MFMAs
#pragma unroll
        for (int c = 0; c < 4; ++c) {
#pragma unroll
            for (int rb = 0; rb < 2; ++rb) {
                acc[rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][c].x, b[c].x, acc[rb], 0, 0, 0);
                acc[rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][c].y, b[c].y, acc[rb], 0, 0, 0);
                acc[rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][c].z, b[c].z, acc[rb], 0, 0, 0);
                acc[rb] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[rb][c].w, b[c].w, acc[rb], 0, 0, 0);
                rowsum[rb] += (a[rb][c].x + a[rb][c].y) + (a[rb][c].z + a[rb][c].w);
            }
        }
        blk = next;
    }
    // accumulator register v of lane (j, h): row 8*(v/4) + 4*h + v%4 (+32), column j
    float *out = g.partial + (long)wave * kNarrowPartial;
#pragma unroll
    for (int rb = 0; rb < 2; ++rb) {
#pragma unroll
        for (int v = 0; v < 16; ++v) out[(rb * 32 + 8 * (v / 4) + 4 * half + (v % 4)) * 32 + col] = acc[rb][v];
        out[64 * 32 + (rb * 32 + col) * 2 + half] = rowsum[rb];
    }
}

// gradWeight[m][k] += scale * (sum over wavefronts of partial[w][m][k]), gradBias[m] += scale * (sum of the row sums):
// one wavefront per result, lanes striding the wavefronts' partial sums, then a butterfly over the lanes -- a fixed
// order of additions.
__global__ __launch_bounds__(256) void conv_narrow_gradweight_finish_kernel(const float *__restrict__ partial,
                                                                            unsigned waves, int K, float scale,
                                                                            float *__restrict__ gradWeight,
                                                                            float *__restrict__ gradBias) {
    const unsigned lane = threadIdx.x & 63u;
    const unsigned result = blockIdx.x * 4u + (threadIdx.x >> 6);  // 64*K weight results, then 64 bias results
    const unsigned nweights = 64u * (unsigned)K;
    if (result >= nweights + (gradBias ? 64u : 0u)) return;
    float sum = 0.0f;
    if (result < nweights) {
        const unsigned m = result / (unsigned)K, k = result % (unsigned)K;
        for (unsigned w = lane; w < waves; w += 64u) sum += partial[(long)w * kNarrowPartial + m * 32u + k];
    } else {
        const unsigned m = result - nweights;
        for (unsigned w = lane; w < waves; w += 64u) {
            const float *p = partial + (long)w * kNarrowPartial + 64 * 32 + m * 2u;
            sum += p[0] + p[1];
        }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) sum += __shfl_xor(sum, off);
    if (lane == 0) {
        if (result < nweights) gradWeight[result] += scale * sum;
        else gradBias[result - nweights] += scale * sum;
    }
}

}  // namespace

bool conv_narrow_forward_fits(long B, int M, long K, int Wo, long N, int col_step, OutputLayout out) {
    // (the conv_narrow_off switch, or a forced GEMM tile, asks for the tiled kernels)
    if (tuning().conv_narrow_off || tuning().gemm_tile[0] || tuning().gemm_split > 0) return false;
    // 64 planes, at most 32 taps, unit column stride, rows of a multiple of 4 positions, planes of a multiple of 128,
    // a dense output, 32-bit byte offsets within an image's output
    return M == 64 && K >= 1 && K <= 2 * kNarrowSteps && col_step == 1 && Wo % 4 == 0 && N >= kNarrowGroup &&
           N % kNarrowGroup == 0 && (out.plane == 0 || out.plane == N) && out.pitch == 0 && 64L * N * 4 < (1L << 31) &&
           B * (N / kNarrowGroup) < (1L << 31) && B >= 1;
}

int conv_narrow_forward(const float *padded, long image_stride, const float *weight, const float *bias, float *output,
                        long B, int M, int K, int Ho, int Wo, int row_step, const int *rowtab, OutputThreshold act) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (!padded || !weight || !output || !rowtab) return fail("conv_narrow_forward: null operand");
    const int N = Ho * Wo;
    NarrowGeom g;
    g.P = padded;
    g.Wt = weight;
    g.bias = bias;
    g.out = output;
    g.rowtab = rowtab;
    g.K = K;
    g.N = N;
    g.row_step = row_step;
    g.divWo = FastDiv((uint32_t)Wo);
    g.image_stride = image_stride;
    g.groups = (unsigned)(B * (N / kNarrowGroup));
    g.divGroupsPerImage = FastDiv((uint32_t)(N / kNarrowGroup));
    g.act = act.on;
    g.act_threshold = act.threshold;
    g.act_value = act.value;
    const int steps = ((K + 3) / 4) * 2;  // ceil(K / 2) rounded up to an even number
    void (*kernel)(NarrowGeom) = nullptr;
    switch (steps) {
        case 2: kernel = conv_narrow_forward_kernel<2>; break;
        case 4: kernel = conv_narrow_forward_kernel<4>; break;
        case 6: kernel = conv_narrow_forward_kernel<6>; break;
        case 8: kernel = conv_narrow_forward_kernel<8>; break;
        case 10: kernel = conv_narrow_forward_kernel<10>; break;
        case 12: kernel = conv_narrow_forward_kernel<12>; break;
        case 14: kernel = conv_narrow_forward_kernel<14>; break;
        case 16: kernel = conv_narrow_forward_kernel<16>; break;
        default: return fail("conv_narrow_forward: %d taps", K);
    }
    // ONE workgroup per CU (measured on 64 x 3 x 224 x 224: 0.184 ms; two per CU, which the registers allow, 0.193;
    // every wavefront writes 64 planes at once, and more of them in flight spread the requests to one DRAM page
    // further apart in time).
    unsigned grid = (unsigned)num_cus();
    const unsigned need = (g.groups + 3u) / 4u;
    if (grid > need) grid = need;
    {
        const double bytes = 4.0 * ((double)B * M * N + (double)B * image_stride + (double)M * K);
        const char *label = prof_enabled() ? prof_label("conv_narrow_fwd M=%d J=%ld R=%d", M, B * (long)N, K) : "conv_narrow_fwd";
        LaunchScope scope(label, 2.0 * M * (double)K * (double)B * N, bytes);  // (the layer's flops; bound by its stores)
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), 0, s, g);
    }
    return check_launch("conv_narrow_forward");
}

bool conv_narrow_gradweight_fits(long B, int M, long K, int Wo, long N, int col_step) {
    if (tuning().conv_narrow_off || tuning().gemm_tile[0] || tuning().gemm_split > 0) return false;
    // 64 planes, at most 32 taps, unit column stride, rows of a multiple of 4 positions, planes of a multiple of 32
    // positions, 32-bit byte offsets within an image's gradOutput
    return M == 64 && K >= 1 && K <= 32 && col_step == 1 && Wo % 4 == 0 && N >= 32 && N % 32 == 0 &&
           64L * N * 4 < (1L << 31) && B * (N / 32) < (1L << 31) && B >= 1;
}

int conv_narrow_gradweight(const float *padded, long image_stride, const float *gradOutput, float *gradWeight,
                           float *gradBias, long B, int M, int K, int Ho, int Wo, int row_step, const int *rowtab,
                           float scale) {
    hipStream_t s = stream();
    if (!s) return 1;
    if (!padded || !gradOutput || !gradWeight || !rowtab) return fail("conv_narrow_gradweight: null operand");
    const int N = Ho * Wo;
    NarrowGradGeom g;
    g.P = padded;
    g.go = gradOutput;
    g.rowtab = rowtab;
    g.K = K;
    g.N = N;
    g.row_step = row_step;
    g.divWo = FastDiv((uint32_t)Wo);
    g.image_stride = image_stride;
    g.blocks = (unsigned)(B * (N / 32));
    g.divBlocksPerImage = FastDiv((uint32_t)(N / 32));
    // ONE workgroup per CU (a wavefront per SIMD, the next block's operands always in flight).  More resident
    // wavefronts are slower here, measured: 0.186 ms with one workgroup per CU, 0.236 with two, 0.245 with three on
    // 64 x 3 x 224 x 224 -- every wavefront reads 64 rows of gradOutput at once, 200 KB apart, and the more of them are
    // in flight the further apart in time the requests to one DRAM page arrive.
    unsigned grid = (unsigned)num_cus();
    const unsigned need = (g.blocks + 3u) / 4u;
    if (grid > need) grid = need;
    const unsigned waves = grid * 4u;
    g.partial = workspace((size_t)waves * kNarrowPartial * sizeof(float));
    if (!g.partial) return 1;
    {
        const double bytes = 4.0 * ((double)B * M * N + (double)B * image_stride + (double)waves * kNarrowPartial);
        const char *label = prof_enabled() ? prof_label("conv_narrow_gradweight M=%d J=%d R=%ld", M, K, B * (long)N)
                                           : "conv_narrow_gradweight";
        LaunchScope scope(label, 2.0 * M * (double)K * (double)B * N, bytes);  // (the layer's flops; bound by its loads)
        hipLaunchKernelGGL(conv_narrow_gradweight_kernel, dim3(grid), dim3(256), 0, s, g);
    }
    if (check_launch("conv_narrow_gradweight")) return 1;
    {
        const unsigned results = 64u * (unsigned)K + (gradBias ? 64u : 0u);
        LaunchScope scope("conv_narrow_gradweight_finish", 0.0, 4.0 * ((double)waves * kNarrowPartial + 2.0 * results));
        hipLaunchKernelGGL(conv_narrow_gradweight_finish_kernel, dim3((results + 3u) / 4u), dim3(256), 0, s, g.partial, waves,
                           K, scale, gradWeight, gradBias);
    }
    return check_launch("conv_narrow_gradweight_finish");
}

}  // namespace thgpu

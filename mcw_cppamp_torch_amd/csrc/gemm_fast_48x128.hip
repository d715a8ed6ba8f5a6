// Fast fp32 MFMA GEMM, short-row variant: 48 of a 64 x 128 tile's rows multiplied (1 x 4 wavefronts, 16x16 blocks).
#include "gemm_fast.h"

namespace thgpu {

int gemm_fast_48x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
    if (la != LD_RC_VEC || lb != LD_XC_GATHER || red) return fail("gemm: the short-row kernel takes a gathered B and an r-contiguous A");
    return gemm_fast_short_rows_go<128, 4, 3>(g, s);
}

}  // namespace thgpu

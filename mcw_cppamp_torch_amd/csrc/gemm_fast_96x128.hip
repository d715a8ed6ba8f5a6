// Fast fp32 MFMA GEMM, 96 x 128 workgroup tile (1 x 4 wavefronts, each 96 x 32): for products of 96 to 127 rows,
// which two 64-row tiles would cover with a third of their work repeated.  First operand along r only (its 384
// 128-bit loads per step are made by 256 threads in two rounds, the second by the first two wavefronts).
#include "gemm_fast.h"

namespace thgpu {

int gemm_fast_96x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
    if (la != LD_RC_VEC) return fail("gemm: the 96-row tile takes a first operand contiguous along r");
    if (lb == LD_RC_VEC)
        return red ? gemm_fast_go<96, 128, 1, 4, LD_RC_VEC, LD_RC_VEC, true>(g, s)
                   : gemm_fast_go<96, 128, 1, 4, LD_RC_VEC, LD_RC_VEC, false>(g, s);
    if (lb == LD_XC_GATHER)
        return red ? gemm_fast_go<96, 128, 1, 4, LD_RC_VEC, LD_XC_GATHER, true>(g, s)
                   : gemm_fast_go<96, 128, 1, 4, LD_RC_VEC, LD_XC_GATHER, false>(g, s);
    if (lb == LD_XC_SCALAR && !red) return gemm_fast_go<96, 128, 1, 4, LD_RC_VEC, LD_XC_SCALAR, false>(g, s);
    return fail("gemm: unknown loader combination (%d, %d)", la, lb);
}

}  // namespace thgpu

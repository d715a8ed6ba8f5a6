// Fast fp32 MFMA GEMM, 192 x 128 workgroup tile (2 x 2 wavefronts of 96 x 64): for row counts that are
// multiples of 192 rather than 128.
#include "gemm_fast.h"

#include <type_traits>

namespace thgpu {

int gemm_fast_192x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
    return gemm_fast_dispatch<192, 128, 2, 2>(g, la, lb, red, s);
}

}  // namespace thgpu

// Fast fp32 MFMA GEMM, 128 x 128 workgroup tile (2 x 2 wavefronts).
#include "gemm_fast.h"

#include <type_traits>

namespace thgpu {

int gemm_fast_128x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
    return gemm_fast_dispatch<128, 128, 2, 2>(g, la, lb, red, s);
}

}  // namespace thgpu

// Fast fp32 MFMA GEMM, 64 x 256 workgroup tile (1 x 4 wavefronts).
#include "gemm_fast.h"

#include <type_traits>

namespace thgpu {

int gemm_fast_64x256(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
    return gemm_fast_dispatch<64, 256, 1, 4>(g, la, lb, red, s);
}

}  // namespace thgpu

// The fast GEMM kernel for 64 x 128 tiles: four wavefronts side by side, each 64 x 32 outputs.  For products
// with 64 rows (a first layer's 64 output planes, a gathered gradInput with 64 input planes).
#include "gemm_fast.h"

#include <type_traits>

namespace thgpu {

int gemm_fast_64x128(const GemmArgs &g, int la, int lb, bool red, hipStream_t s) {
    return gemm_fast_dispatch<64, 128, 1, 4>(g, la, lb, red, s);
}

}  // namespace thgpu

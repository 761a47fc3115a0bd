// Instances of the tiled GEMM kernel for one tile family (see gemm_tiled.hpp).
#include "gemm_tiled.hpp"

namespace miw {

const void *tiled_kernel_256x256_w2x2(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    return pick_types<256, 256, 2, 2, 2>(xk, yk, c_type, d_type, f16acc);
}

}  // namespace miw

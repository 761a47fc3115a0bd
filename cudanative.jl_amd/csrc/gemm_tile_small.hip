// Instances of the tiled GEMM kernel for one tile family (see gemm_tiled.hpp).
#include "gemm_tiled.hpp"

namespace miw {

const void *tiled_kernel_128x128_w2x4_s4(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    return pick_types<128, 128, 2, 4, 4>(xk, yk, c_type, d_type, f16acc);
}

const void *tiled_kernel_128x128_w2x2_s4(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    return pick_types<128, 128, 2, 2, 4>(xk, yk, c_type, d_type, f16acc);
}

const void *tiled_kernel_128x128_w2x2(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    return pick_types<128, 128, 2, 2, 2>(xk, yk, c_type, d_type, f16acc);
}

const void *tiled_kernel_64x64_w2x2(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    return pick_types<64, 64, 2, 2, 4>(xk, yk, c_type, d_type, f16acc);
}

}  // namespace miw

// Instances of the ping-pong GEMM kernel with 64-k clusters (see gemm_pingpong.hpp).
#include "gemm_pingpong.hpp"

namespace miw {

template <int BI, int BJ, int WI, int WJ, int NS, class CT, class DT, bool F16ACC>
static const void *pp64_layout(bool xk, bool yk)
{
    if (xk && yk) return (const void *)k_gemm_pp64<BI, BJ, WI, WJ, NS, true, true, CT, DT, F16ACC>;
    if (xk && !yk) return (const void *)k_gemm_pp64<BI, BJ, WI, WJ, NS, true, false, CT, DT, F16ACC>;
    if (!xk && yk) return (const void *)k_gemm_pp64<BI, BJ, WI, WJ, NS, false, true, CT, DT, F16ACC>;
    return (const void *)k_gemm_pp64<BI, BJ, WI, WJ, NS, false, false, CT, DT, F16ACC>;
}

template <int BI, int BJ, int WI, int WJ, int NS>
static const void *pp64_types(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    if (f16acc) return pp64_layout<BI, BJ, WI, WJ, NS, half_t, half_t, true>(xk, yk);
    if (c_type == 0 && d_type == 0) return pp64_layout<BI, BJ, WI, WJ, NS, half_t, half_t, false>(xk, yk);
    if (c_type == 0 && d_type == 1) return pp64_layout<BI, BJ, WI, WJ, NS, half_t, float, false>(xk, yk);
    if (c_type == 1 && d_type == 0) return pp64_layout<BI, BJ, WI, WJ, NS, float, half_t, false>(xk, yk);
    return pp64_layout<BI, BJ, WI, WJ, NS, float, float, false>(xk, yk);
}

// Kernel for a bm x bn tile, or null when the tile is not instantiated.
const void *pp64_kernel(int bm, int bn, bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    if (bm == 256 && bn == 128) return pp64_types<256, 128, 4, 2, 3>(xk, yk, c_type, d_type, f16acc);
    if (bm == 128 && bn == 256) return pp64_types<128, 256, 2, 4, 3>(xk, yk, c_type, d_type, f16acc);
    if (bm == 128 && bn == 128) return pp64_types<128, 128, 4, 2, 4>(xk, yk, c_type, d_type, f16acc);
    return nullptr;
}

}  // namespace miw

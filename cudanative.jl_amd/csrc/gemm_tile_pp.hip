// Instances of the ping-pong GEMM kernel (see gemm_pingpong.hpp).
#include "gemm_pingpong.hpp"

namespace miw {

template <int BI, int BJ, int WI, int WJ, bool XK, bool YK>
static const void *pp_types(int c_type, int d_type)
{
    if constexpr (!pp_fits(BI, BJ, XK, YK)) {
        return nullptr;
    } else {
        if (c_type == 0 && d_type == 0) return (const void *)k_gemm_pp<BI, BJ, WI, WJ, XK, YK, half_t, half_t>;
        if (c_type == 0 && d_type == 1) return (const void *)k_gemm_pp<BI, BJ, WI, WJ, XK, YK, half_t, float>;
        if (c_type == 1 && d_type == 0) return (const void *)k_gemm_pp<BI, BJ, WI, WJ, XK, YK, float, half_t>;
        return (const void *)k_gemm_pp<BI, BJ, WI, WJ, XK, YK, float, float>;
    }
}

template <int BI, int BJ, int WI, int WJ>
static const void *pp_layout(bool xk, bool yk, int c_type, int d_type)
{
    if (xk && yk) return pp_types<BI, BJ, WI, WJ, true, true>(c_type, d_type);
    if (xk && !yk) return pp_types<BI, BJ, WI, WJ, true, false>(c_type, d_type);
    if (!xk && yk) return pp_types<BI, BJ, WI, WJ, false, true>(c_type, d_type);
    return pp_types<BI, BJ, WI, WJ, false, false>(c_type, d_type);
}

// Kernel for a bm x bn tile, or null when there is none (tile not instantiated, or its ring does not fit in LDS).
const void *pp_kernel(int bm, int bn, bool xk, bool yk, int c_type, int d_type)
{
    if (bm == 256 && bn == 256) return pp_layout<256, 256, 2, 4>(xk, yk, c_type, d_type);
    return nullptr;
}
int pp_lds(int bm, int bn, bool xk, bool yk) { return pp_lds_bytes(bm, bn, xk, yk); }

}  // namespace miw

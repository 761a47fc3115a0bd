// Instances of the one-wavefront-per-SIMD GEMM kernel (see gemm_wave128.hpp).
#include "gemm_wave128.hpp"

namespace miw {

template <bool XK, bool YK>
static const void *w128_types(int c_type, int d_type)
{
    if (c_type == 0 && d_type == 0) return (const void *)k_gemm_w128<XK, YK, half_t, half_t>;
    if (c_type == 0 && d_type == 1) return (const void *)k_gemm_w128<XK, YK, half_t, float>;
    if (c_type == 1 && d_type == 0) return (const void *)k_gemm_w128<XK, YK, float, half_t>;
    return (const void *)k_gemm_w128<XK, YK, float, float>;
}

const void *w128_kernel(bool xk, bool yk, int c_type, int d_type)
{
    if (xk && yk) return w128_types<true, true>(c_type, d_type);
    if (xk && !yk) return w128_types<true, false>(c_type, d_type);
    if (!xk && yk) return w128_types<false, true>(c_type, d_type);
    return w128_types<false, false>(c_type, d_type);
}

}  // namespace miw

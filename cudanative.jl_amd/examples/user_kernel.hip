// A user's own kernels written with the device-side fragment API (miwmma_fragment.hpp), built
// into a code object and run through miw_module_load / miw_module_get_kernel / miw_launch.
//
// user_mac is the kernel of CUDAnative.jl's examples/wmma/high-level.jl:30-44 in HIP C++:
// one wavefront computes D = A * B + beta .* C on a 16x16x16 tile, column-major.
// user_gemm_chain is the chain the reference's documentation describes (docs/src/device/wmma.md:51-52):
// "the D of one mma is the C of the next", here over K in steps of 16 for one 16x16 tile of D per
// wavefront, with A and B staged through LDS (the shared-memory overloads of load_a / load_b).
#include "miwmma_fragment.hpp"

using namespace miw;
using conf = config<16, 16, 16, float>;

extern "C" __global__ void user_mac(const _Float16 *a, const _Float16 *b, const float *c, float *d, float beta)
{
    auto a_frag = load_a<conf, layout::col_major>(a, 16);
    auto b_frag = load_b<conf, layout::col_major>(b, 16);
    auto c_frag = load_c<conf, float>(c, 16, layout::col_major);
    c_frag = scale(beta, c_frag);
    auto d_frag = mma<conf>(a_frag, b_frag, c_frag);
    store_d<conf>(d, d_frag, 16, layout::col_major);
}

// D (M x N, column-major) = A (M x K, column-major) * B (K x N, column-major) + C; grid (M/16, N/16), 64 threads;
// dynamic LDS: 2 * 16 * 16 halves.
extern "C" __global__ void user_gemm_chain(const _Float16 *A, const _Float16 *B, const float *C, float *D, long M, long N, long K)
{
    extern __shared__ __attribute__((aligned(32))) _Float16 tiles[];
    MIW_LDS _Float16 *sa = (MIW_LDS _Float16 *)tiles, *sb = sa + 256;
    const long i0 = blockIdx.x * 16, j0 = blockIdx.y * 16;
    auto acc = load_c<conf, float>(C + (long)j0 * M + i0, M, layout::col_major);
    for (long k0 = 0; k0 < K; k0 += 16) {
        for (int e = threadIdx.x; e < 256; e += 64) {
            sa[e] = A[(long)(k0 + e / 16) * M + i0 + e % 16];      // tile of A, column-major, ld 16
            sb[e] = B[(long)(j0 + e / 16) * K + k0 + e % 16];      // tile of B, column-major, ld 16
        }
        __syncthreads();
        auto a_frag = load_a<conf, layout::col_major>((const MIW_LDS _Float16 *)sa, 16);
        auto b_frag = load_b<conf, layout::col_major>((const MIW_LDS _Float16 *)sb, 16);
        acc = mma<conf>(a_frag, b_frag, acc);
        __syncthreads();
    }
    store_d<conf>(D + (long)j0 * M + i0, acc, M, layout::col_major);
}

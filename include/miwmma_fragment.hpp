// Device-side WMMA fragment API for gfx950 (wave64, MFMA): include it from a HIP kernel of your
// own (hipcc --offload-arch=gfx950 -I<this directory>), build the kernel into a code object
// (--genco) and run it through miw_module_load / miw_module_get_kernel / miw_launch, or link it
// into a HIP program directly.  The kernels inside libmiwmma.so are written with the same header.
//
// Counterpart of CUDAnative.jl's WMMA module (src/device/cuda/wmma.jl):
//   Config{M,N,K,d_type}            :394      -> miw::config<M,N,K,D>
//   Fragment{M,N,K,FS,T,L,U}        :358-360  -> miw::fragment<Use,M,N,K,T,L>
//   load_a / load_b / load_c        :507-530  -> miw::load_a/_b/_c (global and LDS overloads)
//   mma                             :558-583  -> miw::mma
//   store_d                         :613-632  -> miw::store_d
//   fill_c                          :654-667  -> miw::fill_c
//   f.(frag, scalar)                :678-716  -> miw::scale / miw::shift / miw::map
//
// One wavefront (64 lanes) holds a 16x16x16 tile as the operands of
// v_mfma_f32_16x16x16_f16.  With l = lane, q = l / 16, r = l % 16:
//   A fragment : x[i] = A[r][4q + i]           (4 halves, K-contiguous)
//   B fragment : x[i] = B[4q + i][r]
//   C/D        : x[i] = C[4q + i][r]
// The memory layout (row/column major) is resolved when loading, so the
// register layout does not depend on it; the layout tag stays in the type only
// because the reference keeps it there (wmma.jl:527).
#pragma once
#include <hip/hip_runtime.h>

namespace miw {

typedef _Float16 half_t;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

#define MIW_LDS __attribute__((address_space(3)))

enum class layout { row_major, col_major, unspecified };
struct matrix_a {};
struct matrix_b {};
struct accumulator {};

template <int M, int N, int K, class D>
struct config {
    static_assert(M == 16 && N == 16 && K == 16, "Invalid shape for WMMA");
    using d_type = D;
};

template <class Use, int M, int N, int K, class T, layout L>
struct fragment {
    static_assert(M == 16 && N == 16 && K == 16, "Invalid shape for WMMA");
    static constexpr int num_elements = 4;
    T x[4];
    __device__ T &operator[](int i) { return x[i]; }
    __device__ const T &operator[](int i) const { return x[i]; }
};

__device__ inline int lane_id() { return (int)(threadIdx.x & 63u); }

// Offset in elements of tile element (i, j) for a leading dimension ld.
__device__ inline long tile_offset(layout l, int i, int j, long ld)
{
    return l == layout::col_major ? (long)i + (long)j * ld : (long)i * ld + (long)j;
}

// ---------------------------------------------------------------- loads ----
// PtrT is `const T*` (global / generic) or `const MIW_LDS T*` (LDS); the
// compiler emits global_load / flat_load / ds_read accordingly.

template <class Cfg, layout L, class PtrT>
__device__ inline fragment<matrix_a, 16, 16, 16, half_t, L> load_a(PtrT addr, long stride)
{
    fragment<matrix_a, 16, 16, 16, half_t, L> f;
    const int l = lane_id(), r = l & 15, q = l >> 4;
#pragma unroll
    for (int i = 0; i < 4; i++) f.x[i] = addr[tile_offset(L, r, 4 * q + i, stride)];
    return f;
}

template <class Cfg, layout L, class PtrT>
__device__ inline fragment<matrix_b, 16, 16, 16, half_t, L> load_b(PtrT addr, long stride)
{
    fragment<matrix_b, 16, 16, 16, half_t, L> f;
    const int l = lane_id(), r = l & 15, q = l >> 4;
#pragma unroll
    for (int i = 0; i < 4; i++) f.x[i] = addr[tile_offset(L, 4 * q + i, r, stride)];
    return f;
}

// load_c returns layout `unspecified` (wmma.jl:520).
template <class Cfg, class T, class PtrT>
__device__ inline fragment<accumulator, 16, 16, 16, T, layout::unspecified> load_c(PtrT addr, long stride, layout l)
{
    fragment<accumulator, 16, 16, 16, T, layout::unspecified> f;
    const int ln = lane_id(), r = ln & 15, q = ln >> 4;
#pragma unroll
    for (int i = 0; i < 4; i++) f.x[i] = addr[tile_offset(l, 4 * q + i, r, stride)];
    return f;
}

template <class Cfg, class T>
__device__ inline fragment<accumulator, 16, 16, 16, T, layout::unspecified> fill_c(T value)
{
    fragment<accumulator, 16, 16, 16, T, layout::unspecified> f;
#pragma unroll
    for (int i = 0; i < 4; i++) f.x[i] = value;
    return f;
}

// ---------------------------------------------------------------- store ----
// store_d requires eltype(addr) == eltype(d) == d_type (wmma.jl:613-617).
template <class Cfg, class T, class PtrT>
__device__ inline void store_d(PtrT addr, const fragment<accumulator, 16, 16, 16, T, layout::unspecified> &d,
                               long stride, layout l)
{
    static_assert(__is_same(T, typename Cfg::d_type), "store_d: fragment type must equal Config d_type");
    const int ln = lane_id(), r = ln & 15, q = ln >> 4;
#pragma unroll
    for (int i = 0; i < 4; i++) addr[tile_offset(l, 4 * q + i, r, stride)] = d.x[i];
}

// ------------------------------------------------------------ broadcast ----
template <class Frag, class F>
__device__ inline Frag map(const Frag &f, F fn)
{
    Frag out;
#pragma unroll
    for (int i = 0; i < Frag::num_elements; i++) out.x[i] = fn(f.x[i]);
    return out;
}

template <class Use, class T, layout L>
__device__ inline fragment<Use, 16, 16, 16, T, L> scale(T s, const fragment<Use, 16, 16, 16, T, L> &f)
{
    return map(f, [s](T v) { return (T)(s * v); });
}

template <class Use, class T, layout L>
__device__ inline fragment<Use, 16, 16, 16, T, L> shift(T s, const fragment<Use, 16, 16, 16, T, L> &f)
{
    return map(f, [s](T v) { return (T)(s + v); });
}

// ------------------------------------------------------------------ mma ----
// D = A*B + C.  Products and the sum run in fp32 inside the matrix core; an
// fp16 C is widened exactly before, an fp16 D is rounded (nearest even) after.
template <class Cfg, layout LA, layout LB, class CT>
__device__ inline fragment<accumulator, 16, 16, 16, typename Cfg::d_type, layout::unspecified>
mma(const fragment<matrix_a, 16, 16, 16, half_t, LA> &a, const fragment<matrix_b, 16, 16, 16, half_t, LB> &b,
    const fragment<accumulator, 16, 16, 16, CT, layout::unspecified> &c)
{
    using DT = typename Cfg::d_type;
    half4_t av = {a.x[0], a.x[1], a.x[2], a.x[3]};
    half4_t bv = {b.x[0], b.x[1], b.x[2], b.x[3]};
    float4_t cv = {(float)c.x[0], (float)c.x[1], (float)c.x[2], (float)c.x[3]};
    float4_t dv = __builtin_amdgcn_mfma_f32_16x16x16f16(av, bv, cv, 0, 0, 0);
    fragment<accumulator, 16, 16, 16, DT, layout::unspecified> d;
#pragma unroll
    for (int i = 0; i < 4; i++) d.x[i] = (DT)dv[i];
    return d;
}

}  // namespace miw

// Declarations shared by the kernel translation units and the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace miw {

// Arguments of every GEMM kernel: D = alpha * A*B + beta * C, A (M x K) and
// B (K x N) Float16, leading dimensions and batch strides in elements.
struct gemm_params {
    const _Float16 *A;
    const _Float16 *B;
    const void *C;
    void *D;
    long M, N, K;
    long lda, ldb, ldc, ldd;
    long sa, sb, sc, sd;
    long batch;
    int a_row, b_row, c_row, d_row;  // 1: row major, 0: column major
    int use_c;
    float alpha, beta;
};

// --- frag_kernels.hip
hipError_t launch_frag_load(int use, int dtype, int row_major, int as_mode, const void *addr, long stride, void *img,
                            hipStream_t s);
hipError_t launch_frag_store(int dtype, int row_major, int as_mode, void *addr, const void *img, long stride,
                             hipStream_t s);
hipError_t launch_frag_fill(int dtype, float value, void *img, hipStream_t s);
hipError_t launch_frag_map(int dtype, int op, float scalar, const void *in, void *out, size_t n, hipStream_t s);
hipError_t launch_frag_mma(int c_type, int d_type, const void *a, const void *b, const void *c, void *d, hipStream_t s);
hipError_t launch_wmma_mac(int c_type, int d_type, const void *A, const void *B, const void *C, void *D, long lda,
                           long ldb, long ldc, long ldd, int a_row, int b_row, int c_row, int d_row, int use_c,
                           int shared, float alpha, float beta, hipStream_t s);
hipError_t launch_gemm_fragops(const gemm_params &p, int c_type, int d_type, bool f16acc, hipStream_t s);
// Wavefronts that share one 16x16 tile's K loop in the fragment-op kernel launch_gemm_fragops picks (1: none).
int fragops_ksplit(const gemm_params &p, bool f16acc);
hipError_t launch_dummy_store(float *ptr, int threads, hipStream_t s);
const void *frag_kernel_symbol(const char *name);
int frag_kernel_count();
const char *frag_kernel_name(int i);

// --- gemm_kernels.hip
// Kernel families of the LDS-tiled GEMM.
enum {
    KIND_PIPELINED = 0,   // gemm_tiled.hpp: every wavefront overlaps its own loads, LDS reads and MFMAs
    KIND_PINGPONG32 = 1,  // gemm_pingpong.hpp: the two wavefronts of a SIMD alternate between MFMA and memory clusters of 32 k-values
    KIND_PINGPONG64 = 2,  // the same with clusters of 64 k-values
    KIND_WAVE128 = 3      // gemm_wave128.hpp: one wavefront per SIMD with a 128x128 sub-tile, memory instructions between its MFMAs
};
struct tiled_variant {
    const char *name;
    int bm, bn, bk, wm, wn, stages, lds_bytes;
    int kind;  // KIND_*
    // What the variant picker prices a launch with (measured on MI355X, U[-1,1] operands, all CUs
    // busy, i.e. under the power cap): workgroups that fit on one CU together, microseconds per
    // 64 k-values for a workgroup that has its CU to itself, and microseconds per 64 k-values and
    // workgroup when a CU works through a queue of them.
    int occupancy;
    float us_pair_alone, us_pair_queued;
};
int tiled_variant_count();
const tiled_variant &tiled_variant_at(int i);
// acc_chunk the tiled fp16-accumulate kernels round at.
int tiled_f16acc_chunk();
// Variants whose accumulators do not fit in ordinary VGPRs have no fp16-accumulate form.
bool tiled_supports_f16acc(int i);
// Launches tiled variant i.  The caller has checked what the kernels assume: M and N of at least
// one tile (whole tiles when C and D share memory), K of at least 64, 16-byte alignment of
// pointers and leading dimensions, and for fp16 accumulation c_type == d_type == Float16 and,
// outside the 64-k ping-pong kernels, alpha == 1.
hipError_t launch_gemm_tiled(int i, const gemm_params &p, int c_type, int d_type, bool f16acc, hipStream_t s);
// Does variant i have a kernel for this combination of operand layouts?
bool tiled_supports_layout(int i, const gemm_params &p);
// Does the problem's tile count fit the launch grid of variant i?
bool tiled_grid_fits(int i, const gemm_params &p);
const void *tiled_kernel_symbol(int i);
// Second pass of the split-K GEMM: D = alpha * (sum over `splits` Float32 partial products in ws,
// each M x N laid out as D without padding) + beta * C.
hipError_t launch_splitk_reduce(const gemm_params &p, int c_type, int d_type, int splits, const float *ws, hipStream_t s);

hipError_t launch_mfma_peak(int blocks, int iters, float *sink, hipStream_t s);
// One 8-wavefront workgroup per block: 64 MFMAs per wavefront and iteration; ticks[2b], ticks[2b+1]:
// shader-clock and wall-clock ticks workgroup b spent in the chain.
hipError_t launch_mfma_power(int blocks, int iters, float scale, float *sink, long long *ticks, hipStream_t s);
hipError_t launch_copy(void *dst, const void *src, size_t bytes, hipStream_t s);

}  // namespace miw

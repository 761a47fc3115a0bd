// Variant table, dispatch and launch of the LDS-tiled GEMM, and the probe kernels.
// The kernel template lives in gemm_tiled.hpp; its instances are compiled in the
// gemm_tile_*.hip translation units (one per tile family, so that they build in parallel).
#include "gemm_tiled.hpp"

#include <cstdlib>
#include <mutex>
#include <unordered_map>

namespace miw {

// --------------------------------------------------------------- variants --

static const tiled_variant g_variants[] = {
    // name                    bm   bn  bk     wm wn slots lds, kind (32-k ping-pong: ring depth of a K-major operand, largest ring),
    //                                                          workgroups per CU, us per 64 k alone, us per 64 k in a queue
    {"tile256x256_w2x2", 256, 256, KGRAN, 2, 2, 2, 2 * (256 + 256) * KGRAN * 2, 0, 1, 1.55f, 1.55f},
    {"tile256x128_w4x2", 256, 128, KGRAN, 4, 2, 3, 3 * (256 + 128) * KGRAN * 2, 0, 1, 0.80f, 0.80f},
    {"tile128x256_w2x4", 128, 256, KGRAN, 2, 4, 3, 3 * (128 + 256) * KGRAN * 2, 0, 1, 0.80f, 0.80f},
    {"tile128x128_w2x4_s4", 128, 128, KGRAN, 2, 4, 4, 4 * (128 + 128) * KGRAN * 2, 0, 1, 0.50f, 0.50f},
    {"tile128x128_w2x2_s4", 128, 128, KGRAN, 2, 2, 4, 4 * (128 + 128) * KGRAN * 2, 0, 1, 0.50f, 0.50f},
    {"tile128x128_w2x2", 128, 128, KGRAN, 2, 2, 2, 2 * (128 + 128) * KGRAN * 2, 0, 2, 0.63f, 0.455f},
    {"tile64x64_w2x2", 64, 64, KGRAN, 2, 2, 4, 4 * (64 + 64) * KGRAN * 2, 0, 2, 0.22f, 0.19f},
    {"tile256x256_pingpong", 256, 256, KGRAN, 2, 4, 3, 160 * 1024, 1, 1, 1.30f, 1.30f},
    {"tile256x128_pingpong", 256, 128, KGRAN, 4, 2, 3, 3 * (256 + 128) * KGRAN * 2, 2, 1, 0.785f, 0.785f},
    {"tile128x256_pingpong", 128, 256, KGRAN, 2, 4, 3, 3 * (128 + 256) * KGRAN * 2, 2, 1, 0.785f, 0.785f},
    {"tile128x128_pingpong", 128, 128, KGRAN, 4, 2, 4, 4 * (128 + 128) * KGRAN * 2, 2, 1, 0.50f, 0.50f},
    {"tile256x256_wave128", 256, 256, KGRAN, 2, 2, 3, 160 * 1024, KIND_WAVE128, 1, 1.27f, 1.27f},
};

int tiled_variant_count() { return (int)(sizeof(g_variants) / sizeof(g_variants[0])); }
const tiled_variant &tiled_variant_at(int i) { return g_variants[i]; }
int tiled_f16acc_chunk() { return KGRAN; }
bool tiled_supports_f16acc(int i)
{
    const tiled_variant &v = g_variants[i];
    if (v.kind == KIND_PINGPONG32 || v.kind == KIND_WAVE128) return false;  // 32-k clusters, accumulators in AGPRs: fp32 accumulation only
    if (v.kind == KIND_PINGPONG64) return true;   // 64-k clusters round in the compute cluster
    return waves_per_simd(v.bm, v.bn, v.wm * v.wn * 64) >= 2;
}

// One lookup per tile family, each defined in its own translation unit.
const void *tiled_kernel_256x256_w2x2(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *tiled_kernel_256x128_w4x2(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *tiled_kernel_128x256_w2x4(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *tiled_kernel_128x128_w2x4_s4(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *tiled_kernel_128x128_w2x2_s4(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *tiled_kernel_128x128_w2x2(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *tiled_kernel_64x64_w2x2(bool xk, bool yk, int c_type, int d_type, bool f16acc);
const void *pp_kernel(int bm, int bn, bool xk, bool yk, int c_type, int d_type);
int pp_lds(int bm, int bn, bool xk, bool yk);
const void *w128_kernel(bool xk, bool yk, int c_type, int d_type);
const void *pp64_kernel(int bm, int bn, bool xk, bool yk, int c_type, int d_type, bool f16acc);


// Tile shape in canonical (I, J) terms: bm applies to I, bn to J.
static const void *pick_kernel(int i, bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    const tiled_variant &v = g_variants[i];
    if (v.kind == KIND_PINGPONG32) return f16acc ? nullptr : pp_kernel(v.bm, v.bn, xk, yk, c_type, d_type);
    if (v.kind == KIND_PINGPONG64) return pp64_kernel(v.bm, v.bn, xk, yk, c_type, d_type, f16acc);
    if (v.kind == KIND_WAVE128) return f16acc ? nullptr : w128_kernel(xk, yk, c_type, d_type);
    const int waves = v.wm * v.wn;
    if (v.bm == 256 && v.bn == 256 && waves == 4) return tiled_kernel_256x256_w2x2(xk, yk, c_type, d_type, f16acc);
    if (v.bm == 256 && v.bn == 128) return tiled_kernel_256x128_w4x2(xk, yk, c_type, d_type, f16acc);
    if (v.bm == 128 && v.bn == 256) return tiled_kernel_128x256_w2x4(xk, yk, c_type, d_type, f16acc);
    if (v.bm == 128 && v.bn == 128 && waves == 8) return tiled_kernel_128x128_w2x4_s4(xk, yk, c_type, d_type, f16acc);
    if (v.bm == 128 && v.bn == 128 && v.stages == 4) return tiled_kernel_128x128_w2x2_s4(xk, yk, c_type, d_type, f16acc);
    if (v.bm == 128 && v.bn == 128) return tiled_kernel_128x128_w2x2(xk, yk, c_type, d_type, f16acc);
    if (v.bm == 64 && v.bn == 64) return tiled_kernel_64x64_w2x2(xk, yk, c_type, d_type, f16acc);
    return nullptr;
}

const void *tiled_kernel_symbol(int i) { return pick_kernel(i, false, true, 1, 1, false); }

// The workgroup index is a 32-bit grid coordinate and the kernels keep tile counts in int.
bool tiled_grid_fits(int i, const gemm_params &g)
{
    const tiled_variant &v = g_variants[i];
    const long I = g.d_row ? g.N : g.M, J = g.d_row ? g.M : g.N;
    if (I < v.bm || J < v.bn) return false;
    const long tiles = ((I + v.bm - 1) / v.bm) * ((J + v.bn - 1) / v.bn);
    return tiles * (long)(v.wm * v.wn * 64) < (1l << 32) && tiles <= 0x7fffffffl;
}

// Which operands have k contiguous once the problem is in canonical form (see gemm_tiled.hpp).
static void canonical_layout(const gemm_params &g, bool *xk, bool *yk)
{
    if (!g.d_row) { *xk = g.a_row != 0; *yk = g.b_row == 0; }
    else { *xk = g.b_row == 0; *yk = g.a_row != 0; }
}

bool tiled_supports_layout(int i, const gemm_params &g)
{
    if (g_variants[i].kind == KIND_WAVE128) return true;  // (the ping-pong kernel's rings: one fits for every layout)
    if (g_variants[i].kind != KIND_PINGPONG32) return true;
    bool xk, yk;
    canonical_layout(g, &xk, &yk);
    return pp_kernel(g_variants[i].bm, g_variants[i].bn, xk, yk, 1, 1) != nullptr;  // (every layout has a ring that fits in LDS at 256 x 256)
}

// hipFuncAttributeMaxDynamicSharedMemorySize is a property of the kernel, not of the launch: set once.
static hipError_t allow_dynamic_lds(const void *fn, int bytes)
{
    static std::mutex mu;
    static std::unordered_map<const void *, int> done;
    std::lock_guard<std::mutex> lock(mu);
    auto it = done.find(fn);
    if (it != done.end() && it->second >= bytes) return hipSuccess;
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
    if (e == hipSuccess) done[fn] = bytes;
    return e;
}

hipError_t launch_gemm_tiled(int i, const gemm_params &g, int c_type, int d_type, bool f16acc, hipStream_t s)
{
    const tiled_variant &v = g_variants[i];
    tiled_params p;
    bool xk, yk;
    if (!g.d_row) {
        // P = D (M x N, M contiguous): X = A, Y = B
        p.X = g.A; p.Y = g.B;
        p.I = (int)g.M; p.J = (int)g.N;
        p.ldx = g.lda; p.ldy = g.ldb; p.sx = g.sa; p.sy = g.sb;
        xk = g.a_row != 0;   // A row-major: k contiguous
        yk = g.b_row == 0;   // B column-major: k contiguous
        p.c_trans = g.c_row != 0;
    } else {
        // P = D^T (N x M, N contiguous): X = B^T, Y = A^T
        p.X = g.B; p.Y = g.A;
        p.I = (int)g.N; p.J = (int)g.M;
        p.ldx = g.ldb; p.ldy = g.lda; p.sx = g.sb; p.sy = g.sa;
        xk = g.b_row == 0;
        yk = g.a_row != 0;
        p.c_trans = g.c_row == 0;
    }
    p.C = g.C; p.D = g.D;
    p.K = (int)g.K;
    p.ldc = g.ldc; p.ldd = g.ldd; p.sc = g.sc; p.sd = g.sd;
    p.use_c = g.use_c;
    p.alpha = g.alpha; p.beta = g.beta;
    p.tiles_i = (p.I + v.bm - 1) / v.bm;
    p.tiles_j = (p.J + v.bn - 1) / v.bn;
    // Rows of tiles per raster group: about the square root of one XCD's share.
    int per_xcd = (p.tiles_i * p.tiles_j + 7) / 8, gi = 1;
    while ((gi * 2) * (gi * 2) <= per_xcd) gi *= 2;
    p.group_i = gi < p.tiles_i ? gi : p.tiles_i;

#ifdef MIW_PP_TS
    // measurement builds: device address of the timestamp buffer, in hexadecimal
    p.ts = nullptr;
    if (const char *e = getenv("MIW_TS")) p.ts = (long long *)strtoull(e, nullptr, 16);
#endif
    const void *fn = pick_kernel(i, xk, yk, c_type, d_type, f16acc);
    if (!fn) return hipErrorInvalidValue;
    // (the 64-k ping-pong kernels stage a Float16 C tile beside the ring where both fit)
    const int c_stage = v.kind == KIND_PINGPONG64 && f16acc && v.lds_bytes + v.bm * v.bn * 2 <= 160 * 1024 ? v.bm * v.bn * 2 : 0;
    const int lds_bytes = v.kind == KIND_PINGPONG32 || v.kind == KIND_WAVE128 ? pp_lds(v.bm, v.bn, xk, yk)
                          : v.kind != KIND_PIPELINED ? v.lds_bytes + c_stage
                                                     : v.lds_bytes + fold_stage_bytes(v.bm, v.bn, v.wm * v.wn * 64, v.stages);
    hipError_t e = allow_dynamic_lds(fn, lds_bytes);
    if (e != hipSuccess) return e;
    void *args[] = {&p};
    // the tile count fits: tiled_grid_fits() is part of the caller's check
    dim3 grid((unsigned)(p.tiles_i * p.tiles_j), (unsigned)g.batch);
    return hipLaunchKernel(fn, grid, dim3((unsigned)(v.wm * v.wn * 64)), args, (size_t)lds_bytes, s);
}

// ---------------------------------------------------------- split-K ---------

// Second pass of the split-K GEMM.  The first pass left `splits` Float32 partial products in
// `ws`, each I x J with I contiguous (canonical form: I runs along D's contiguous dimension);
// this adds them in slice order and applies the scalars: D = alpha * sum_s P_s + beta * C.
// One lane owns four consecutive i of one j.
template <class CT, class DT>
__global__ __launch_bounds__(256) void k_splitk_reduce(const float *ws, int splits, long I, long J, const CT *C, DT *D,
                                                       long ldc, long ldd, int use_c, int c_trans, float alpha, float beta)
{
    const long quads = I / 4;
    const long idx = (long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= quads * J) return;
    const long j = idx / quads, i = (idx - j * quads) * 4;
    const float *src = ws + j * I + i;
    float4_t sum = *(const float4_t *)src;
    for (int s = 1; s < splits; s++) {
        const float4_t v = *(const float4_t *)(src + (long)s * I * J);
#pragma unroll
        for (int e = 0; e < 4; e++) sum[e] += v[e];
    }
#pragma unroll
    for (int e = 0; e < 4; e++) {
        float v = alpha * sum[e];
        if (use_c) {
            const float c = (float)(c_trans ? C[(i + e) * ldc + j] : C[j * ldc + i + e]);
            v = __builtin_fmaf(beta, c, v);
        }
        D[j * ldd + i + e] = (DT)v;
    }
}

hipError_t launch_splitk_reduce(const gemm_params &g, int c_type, int d_type, int splits, const float *ws, hipStream_t s)
{
    const long I = g.d_row ? g.N : g.M, J = g.d_row ? g.M : g.N;
    const int c_trans = g.d_row ? g.c_row == 0 : g.c_row != 0;
    const long lanes = I / 4 * J;
    const dim3 grid((unsigned)((lanes + 255) / 256)), block(256);
#define MIW_REDUCE(CT, DT)                                                                                          \
    hipLaunchKernelGGL((k_splitk_reduce<CT, DT>), grid, block, 0, s, ws, splits, I, J, (const CT *)g.C, (DT *)g.D, \
                       g.ldc, g.ldd, g.use_c, c_trans, g.alpha, g.beta)
    if (c_type == 0 && d_type == 0) MIW_REDUCE(half_t, half_t);
    else if (c_type == 0) MIW_REDUCE(half_t, float);
    else if (d_type == 0) MIW_REDUCE(float, half_t);
    else MIW_REDUCE(float, float);
#undef MIW_REDUCE
    return hipGetLastError();
}

// ------------------------------------------------------------ probes -------

// Register-resident MFMA chain: 8 independent accumulators per wavefront.
__global__ __launch_bounds__(256) void k_mfma_peak(int iters, float *sink)
{
    half8_t a, b;
    for (int i = 0; i < 8; i++) {
        a[i] = (half_t)(0.001f * (float)(threadIdx.x + i));
        b[i] = (half_t)(0.002f * (float)(threadIdx.x ^ i));
    }
    float4_t acc[8];
    for (int i = 0; i < 8; i++) acc[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; it++) {
#pragma unroll
        for (int u = 0; u < 4; u++)
#pragma unroll
            for (int i = 0; i < 8; i++) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, acc[i], 0, 0, 0);
    }
    float s = 0.f;
    for (int i = 0; i < 8; i++) s += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (s == 12345.678f) sink[0] = s;  // keeps the chain alive
}

hipError_t launch_mfma_peak(int blocks, int iters, float *sink, hipStream_t s)
{
    hipLaunchKernelGGL(k_mfma_peak, dim3((unsigned)blocks), dim3(256), 0, s, iters, sink);
    return hipGetLastError();
}

// The same chain on operands that change every k-step (four register-resident sets of four A
// and four B fragments, pseudo-random or all zero), as a GEMM's do: what the matrix cores
// sustain under the power cap.  Each workgroup reports its shader-clock and wall-clock ticks.
__device__ inline unsigned probe_hash(unsigned x)
{
    x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(512) void k_mfma_power(int iters, float scale, float *sink, long long *ticks)
{
    constexpr int NSET = 4;
    half8_t a[NSET][4], b[NSET][4];
    for (int s = 0; s < NSET; s++)
        for (int i = 0; i < 4; i++)
            for (int e = 0; e < 8; e++) {
                const unsigned seed = ((blockIdx.x * 512u + threadIdx.x) * 32u + s * 8u + i) * 16u + e;
                a[s][i][e] = (half_t)(scale * ((float)(probe_hash(2 * seed + 1) & 0xffff) / 32768.f - 1.f));
                b[s][i][e] = (half_t)(scale * ((float)(probe_hash(2 * seed + 2) & 0xffff) / 32768.f - 1.f));
            }
    float4_t acc[4][4];
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    const long long c0 = clock64(), w0 = wall_clock64();
    for (int it = 0; it < iters; it++)
#pragma unroll
        for (int s = 0; s < NSET; s++)
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
    const long long c1 = clock64(), w1 = wall_clock64();
    float r = 0.f;
    for (int i = 0; i < 4; i++)
        for (int j = 0; j < 4; j++) r += acc[i][j][0] + acc[i][j][3];
    if (r == 12345.678f) sink[0] = r;  // keeps the chain alive
    if (threadIdx.x == 0) {
        ticks[2 * blockIdx.x] = c1 - c0;
        ticks[2 * blockIdx.x + 1] = w1 - w0;
    }
}

hipError_t launch_mfma_power(int blocks, int iters, float scale, float *sink, long long *ticks, hipStream_t s)
{
    hipLaunchKernelGGL(k_mfma_power, dim3((unsigned)blocks), dim3(512), 0, s, iters, scale, sink, ticks);
    return hipGetLastError();
}

__global__ __launch_bounds__(256) void k_copy16(uint4_t *dst, const uint4_t *src, size_t n16)
{
    size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * 256;
    for (; i < n16; i += stride) dst[i] = src[i];
}

hipError_t launch_copy(void *dst, const void *src, size_t bytes, hipStream_t s)
{
    size_t n16 = bytes / 16;
    unsigned blocks = (unsigned)((n16 + 255) / 256);
    if (blocks > 256u * 16u) blocks = 256u * 16u;
    if (blocks == 0) return hipSuccess;
    hipLaunchKernelGGL(k_copy16, dim3(blocks), dim3(256), 0, s, (uint4_t *)dst, (const uint4_t *)src, n16);
    return hipGetLastError();
}

}  // namespace miw

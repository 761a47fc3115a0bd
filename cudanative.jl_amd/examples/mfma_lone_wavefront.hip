// Probe: what does a wavefront that is alone on its SIMD pay for the instructions it issues between its
// MFMAs?  (The one-wavefront-per-SIMD GEMM kernel of csrc/gemm_wave128.hpp is scheduled on these figures.)
//
//   part 1: 32 independent v_mfma_f32_16x16x32_f16 per iteration with one kind of extra instruction behind
//           every MFMA (or every n-th): cycles per MFMA (16 is the matrix core's own pace);
//   part 2: a k-step of a 128x128 tile (64 MFMAs, accumulators in AGPRs) with the fragment reads of the
//           next step (16 ds_read_b128, or 32 ds_read_b64_tr_b16), 8 direct-to-LDS loads and a barrier
//           in the slots behind the MFMAs, the way the kernel places them: cycles per step (ideal 1024).
//
// Operands are all zero (no power cap in the way): the figures are issue cycles.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++20 cudanative.jl_amd/examples/mfma_lone_wavefront.hip -o /tmp/mfma_lone_wavefront
//   /tmp/mfma_lone_wavefront
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
#define LDS __attribute__((address_space(3)))

// ---------------------------------------------------------------- part 1 ----
template <int AG>
__device__ inline void mfma(float4_t &c, half8_t a, half8_t b)
{
    if constexpr (AG == 1) asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b));
}
// KIND: 0 nothing, 1 s_nop 0, 2 s_add_u32, 3 v_mov_b32, 4 ds_read_b128, 5 two ds_read_b128, 6 ds_read_b64, 7 s_nop 3, 8 v_mov x2
// (the LDS reads stop six MFMAs before the end of an iteration, so that the wait there does not measure their latency)
// EVERY: after every EVERY-th MFMA
template <int AG, int KIND, int EVERY, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void k_slot(int iters, float *sink, long long *ticks)
{
    __shared__ __attribute__((aligned(128))) char smem[32768];
    const unsigned lds0 = (unsigned)(uintptr_t)(LDS char *)smem;
    const int lane = threadIdx.x & 63;
    float4_t acc[8][4];
    for (int i = 0; i < 8; i++) for (int j = 0; j < 4; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t f[12], g[8];
    for (int i = 0; i < 12; i++) for (int e = 0; e < 8; e++) f[i][e] = (_Float16)0.f;
    for (int i = 0; i < 8; i++) for (int e = 0; e < 8; e++) g[i][e] = (_Float16)0.f;
    const unsigned raddr = lds0 + lane * 16;
    unsigned sv = 0, vv = lane, vw = lane;
    for (int i = threadIdx.x; i < 8192; i += WAVES * 64) ((LDS float *)smem)[i] = 0.f;
    __syncthreads();
    const long long c0 = clock64();
    for (int it = 0; it < iters; it++) {
        [&]<int... M>(std::integer_sequence<int, M...>) {
            (([&] {
                 constexpr int a = M / 4, bb = M % 4, b = (a & 1) ? 3 - bb : bb;
                 mfma<AG>(acc[a][b], f[a], f[8 + b]);
                 if constexpr (M % EVERY == EVERY - 1) {
                     if constexpr (KIND == 1) asm volatile("s_nop 0");
                     if constexpr (KIND == 7) asm volatile("s_nop 3");
                     if constexpr (KIND == 2) asm volatile("s_add_u32 %0, %0, 4" : "+s"(sv) : : "scc");
                     if constexpr (KIND == 3) asm volatile("v_mov_b32 %0, %1" : "=v"(vv) : "v"(vw));
                     if constexpr (KIND == 8) { asm volatile("v_mov_b32 %0, %1" : "=v"(vv) : "v"(vw)); asm volatile("v_mov_b32 %0, %1" : "=v"(vw) : "v"(vv)); }
                     if constexpr (KIND == 4 && M < 26) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(g[(M / EVERY) % 8]) : "v"(raddr), "n"((M % 16) * 1024));
                     if constexpr (KIND == 5 && M < 26) { asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(g[(M / EVERY) % 4]) : "v"(raddr), "n"((M % 16) * 1024));
                                                asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(g[4 + (M / EVERY) % 4]) : "v"(raddr), "n"((M % 16) * 1024 + 16384)); }
                     if constexpr (KIND == 6 && M < 26) asm volatile("ds_read_b64 %0, %1 offset:%2" : "=v"(*(double *)&g[(M / EVERY) % 8]) : "v"(raddr), "n"((M % 16) * 1024));
                 }
                 __builtin_amdgcn_sched_barrier(0);
             }()),
             ...);
        }(std::make_integer_sequence<int, 32>{});
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }
    const long long c1 = clock64();
    float r = (float)sv + (float)vv;
    for (int i = 0; i < 8; i++) for (int j = 0; j < 4; j++) r += acc[i][j][0] + acc[i][j][3];
    for (int i = 0; i < 8; i++) r += (float)g[i][0];
    if (r == 12345.678f) sink[0] = r;
    if (threadIdx.x == 0) ticks[blockIdx.x] = c1 - c0;
}
template <int AG, int KIND, int EVERY, int WAVES = 4>
void run_slot(const char *name, float *sink, long long *ticks)
{
    const int iters = 4000;
    for (int rep = 0; rep < 2; rep++) { hipLaunchKernelGGL((k_slot<AG, KIND, EVERY, WAVES>), dim3(256), dim3(WAVES * 64), 0, 0, iters, sink, ticks); (void)hipDeviceSynchronize(); }
    std::vector<long long> t(256);
    (void)hipMemcpy(t.data(), ticks, 256 * 8, hipMemcpyDeviceToHost);
    double sum = 0; for (auto v : t) sum += v;
    printf("%-64s %6.2f cycles per MFMA\n", name, sum / 256 / iters / 32);
    fflush(stdout);
}

// ---------------------------------------------------------------- part 2 ----
template <int OFF>
__device__ inline half8_t ds128o(unsigned addr) { half8_t v; asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF)); return v; }
template <int OFF>
__device__ inline half4_t dstr(unsigned addr) { half4_t v; asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFF)); return v; }
template <int DST_IMM>
__device__ inline void dma16(const void *base, unsigned voff, unsigned lds_base)
{
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" : : "s"(lds_base), "v"(voff), "s"(base), "n"(DST_IMM) : "memory", "m0", "scc");
}

// NREAD b128 reads (TR: issued as pairs of transposing 8-byte reads), NLOAD loads per step of 64 MFMAs; BAR: barrier per step
template <int NREAD, bool TR, int NLOAD, int BAR, int WAITV, bool SPLIT>
__global__ __launch_bounds__(256) void k_step(int iters, const char *src, float *sink, long long *ticks)
{
    extern __shared__ __attribute__((aligned(128))) char smem[];
    const unsigned lds0 = (unsigned)(uintptr_t)(LDS char *)smem;
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    float4_t acc[8][8];
    for (int i = 0; i < 8; i++) for (int j = 0; j < 8; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    half8_t f[2][16];
    for (int s = 0; s < 2; s++) for (int i = 0; i < 16; i++) for (int e = 0; e < 8; e++) f[s][i][e] = (_Float16)0.f;
    const unsigned raddr = lds0 + wave * 16384 + lane * 16;
    const unsigned voff = (blockIdx.x * 4 + wave) * 32768u + lane * 16u;
    const unsigned wdst = lds0 + 65536 + wave * 8192;
    const char *g = src;
    __syncthreads();
    const long long c0 = clock64();
    half4_t lo[2];
    auto step = [&]<int S>(std::integral_constant<int, S>) {
        [&]<int... M>(std::integer_sequence<int, M...>) {
            (([&] {
                 constexpr int a = M / 8, bb = M % 8, b = (a & 1) ? 7 - bb : bb;
                 mfma<1>(acc[a][b], f[S][a], f[S][8 + b]);
                 // reads: fragment R at slot 3 R (transposing reads: halves at 3 R and 3 R + 1); loads: m0 at slot 6 L + 2, load at 6 L + 5
                 if constexpr (NREAD > 0) {
                     constexpr int R = M / 3;
                     if constexpr (TR) {
                         if constexpr (M % 3 == 0 && R < NREAD) lo[R % 2] = dstr<R * 1024>(raddr);
                         if constexpr (M % 3 == 1 && R < NREAD) { half4_t hi = dstr<R * 1024 + 512>(raddr); f[S ^ 1][R] = __builtin_shufflevector(lo[R % 2], hi, 0, 1, 2, 3, 4, 5, 6, 7); }
                     } else if constexpr (M % 3 == 0 && R < NREAD) f[S ^ 1][R] = ds128o<R * 1024>(raddr);
                 }
                 if constexpr (NLOAD > 0) {
                     constexpr int L = M / 6;
                     if constexpr (SPLIT) {
                         if constexpr (M % 6 == 2 && L < NLOAD) asm volatile("s_add_u32 m0, %0, %1" : : "s"(wdst), "n"(L * 1024) : "m0", "scc");
                         if constexpr (M % 6 == 5 && L < NLOAD) asm volatile("global_load_lds_dwordx4 %0, %1" : : "v"(voff), "s"(g) : "memory", "m0");
                     } else if constexpr (M % 6 == 5 && L < NLOAD) dma16<L * 1024>(g, voff, wdst);
                 }
                 __builtin_amdgcn_sched_barrier(0);
             }()),
             ...);
        }(std::make_integer_sequence<int, 64>{});
        if constexpr (NLOAD > 0) g += 8192 * NLOAD / 8;
        if (g >= src + 24576) g = src;
        if constexpr (NREAD > 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        if constexpr (NLOAD > 0) { if constexpr (WAITV >= 0) __builtin_amdgcn_s_waitcnt((WAITV & 15) | (7 << 4) | (15 << 8) | ((WAITV >> 4) << 14)); }
        if constexpr (BAR) __builtin_amdgcn_s_barrier();
        __builtin_amdgcn_sched_barrier(0);
        // make the fragments just read the next step's operands
#pragma unroll
        for (int u = 0; u < 16; u++) asm volatile("" : "+v"(f[S ^ 1][u]));
    };
    for (int it = 0; it < iters; it++) {
        step(std::integral_constant<int, 0>{});
        step(std::integral_constant<int, 1>{});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    const long long c1 = clock64();
    __syncthreads();
    float r = 0.f;
    for (int i = 0; i < 8; i++) for (int j = 0; j < 8; j++) r += acc[i][j][0] + acc[i][j][3];
    if (r == 12345.678f) sink[0] = r;
    if (lane == 0) ticks[blockIdx.x * 4 + wave] = c1 - c0;
}

template <int NREAD, bool TR, int NLOAD, int BAR, int WAITV, bool SPLIT = true>
void run_step(const char *name, const char *src, float *sink, long long *ticks)
{
    const int iters = 2000;
    auto kern = k_step<NREAD, TR, NLOAD, BAR, WAITV, SPLIT>;
    (void)hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    for (int rep = 0; rep < 2; rep++) {
        hipLaunchKernelGGL(kern, dim3(256), dim3(256), 128 * 1024, 0, iters, src, sink, ticks);
        (void)hipDeviceSynchronize();
    }
    std::vector<long long> t(1024);
    (void)hipMemcpy(t.data(), ticks, 1024 * 8, hipMemcpyDeviceToHost);
    double sum = 0; long long mx = 0;
    for (auto v : t) { sum += v; if (v > mx) mx = v; }
    printf("%-58s %7.1f cycles per step of 64 MFMAs (ideal 1024), slowest wave %7.1f\n", name, sum / 1024 / iters / 2, (double)mx / iters / 2);
    fflush(stdout);
}

int main()
{
    char *src; float *sink; long long *ticks;
    (void)hipMalloc(&src, 64u << 20); (void)hipMemset(src, 0, 64u << 20);
    (void)hipMalloc(&sink, 64); (void)hipMalloc(&ticks, 1024 * 8);
    printf("part 1: one kind of instruction between the MFMAs (4 wavefronts per workgroup, one per SIMD)\n");
    run_slot<1, 0, 1>("MFMAs only (accumulators in AGPRs)", sink, ticks);
    run_slot<0, 0, 1>("MFMAs only (accumulators in VGPRs)", sink, ticks);
    run_slot<1, 1, 1>("s_nop 0 behind every MFMA", sink, ticks);
    run_slot<1, 7, 1>("s_nop 3 behind every MFMA", sink, ticks);
    run_slot<1, 2, 1>("s_add_u32 behind every MFMA", sink, ticks);
    run_slot<1, 3, 1>("v_mov_b32 behind every MFMA", sink, ticks);
    run_slot<1, 8, 1>("two v_mov_b32 behind every MFMA", sink, ticks);
    run_slot<1, 4, 1>("ds_read_b128 behind every MFMA", sink, ticks);
    run_slot<1, 4, 4>("ds_read_b128 behind every 4th MFMA", sink, ticks);
    run_slot<1, 5, 4>("two ds_read_b128 behind every 4th MFMA", sink, ticks);
    run_slot<1, 4, 1, 8>("ds_read_b128 behind every MFMA, two wavefronts per SIMD", sink, ticks);
    printf("part 2: a k-step of a 128x128 tile per wavefront\n");
    run_step<0, false, 0, 0, -1>("MFMAs only", src, sink, ticks);
    run_step<0, false, 0, 1, -1>("MFMAs, barrier", src, sink, ticks);
    run_step<16, false, 0, 1, -1>("16 ds_read_b128, barrier", src, sink, ticks);
    run_step<16, true, 0, 1, -1>("32 ds_read_b64_tr_b16, barrier", src, sink, ticks);
    run_step<0, false, 8, 0, 16>("8 direct-to-LDS loads (M0 written one MFMA ahead), vmcnt(16)", src, sink, ticks);
    run_step<0, false, 8, 0, 16, false>("8 direct-to-LDS loads (M0 written right in front), vmcnt(16)", src, sink, ticks);
    run_step<16, false, 8, 1, 16>("16 ds_read_b128, 8 loads, vmcnt(16), barrier", src, sink, ticks);
    run_step<16, true, 8, 1, 16>("32 ds_read_b64_tr_b16, 8 loads, vmcnt(16), barrier", src, sink, ticks);
    return 0;
}

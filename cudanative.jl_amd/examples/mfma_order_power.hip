// Probe: matrix cores alone under the power cap, by the order in which a wavefront walks its grid of
// accumulator tiles (which operand fragment two consecutive MFMAs share), by the grid's shape (8 x 4
// tiles with two wavefronts per SIMD, 8 x 8 with one) and by the register file of the accumulators.
// Register-resident pseudo-random operands (scale 1) or zeros (scale 0: no power cap in the way).
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++20 cudanative.jl_amd/examples/mfma_order_power.hip -o /tmp/mfma_order_power
//   /tmp/mfma_order_power
#include <hip/hip_runtime.h>
#include <cstdio>
#include <vector>
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
__device__ inline unsigned probe_hash(unsigned x) { x ^= x >> 16; x *= 0x7feb352dU; x ^= x >> 15; x *= 0x846ca68bU; x ^= x >> 16; return x; }

// NA x NB accumulator tiles per wave, NSET operand sets, ORDER: 0 = a outer / b inner, 1 = b outer / a inner, 2 = diagonal (both change), 3 = snake over b
template <int FORM>
__device__ inline float4_t mfma_f(half8_t a, half8_t b, float4_t c)
{
    if constexpr (FORM == 1) { asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b)); return c; }
    else if constexpr (FORM == 2) { asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b)); return c; }
    else return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
}
#define MFMA(A,B,C) mfma_f<FORM>(A,B,C)
template <int NA, int NB, int NSET, int ORDER, int THREADS, int FORM>
__global__ __launch_bounds__(THREADS) void k(int iters, float scale, float *sink)
{
    half8_t a[NSET][NA], b[NSET][NB];
    for (int s = 0; s < NSET; s++) {
        for (int i = 0; i < NA; i++) for (int e = 0; e < 8; e++) { unsigned seed = ((blockIdx.x * 512u + threadIdx.x) * 64u + s * 16u + i) * 16u + e; a[s][i][e] = (_Float16)(scale * ((float)(probe_hash(2 * seed + 1) & 0xffff) / 32768.f - 1.f)); }
        for (int i = 0; i < NB; i++) for (int e = 0; e < 8; e++) { unsigned seed = ((blockIdx.x * 512u + threadIdx.x) * 64u + s * 16u + i) * 16u + e; b[s][i][e] = (_Float16)(scale * ((float)(probe_hash(2 * seed + 2) & 0xffff) / 32768.f - 1.f)); }
    }
    float4_t acc[NA][NB];
    for (int i = 0; i < NA; i++) for (int j = 0; j < NB; j++) acc[i][j] = float4_t{0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; it++)
#pragma unroll
        for (int s = 0; s < NSET; s++) {
            if constexpr (ORDER == 0) {
#pragma unroll
                for (int i = 0; i < NA; i++)
#pragma unroll
                    for (int j = 0; j < NB; j++) acc[i][j] = MFMA(a[s][i], b[s][j], acc[i][j]);
            } else if constexpr (ORDER == 1) {
#pragma unroll
                for (int j = 0; j < NB; j++)
#pragma unroll
                    for (int i = 0; i < NA; i++) acc[i][j] = MFMA(a[s][i], b[s][j], acc[i][j]);
            } else if constexpr (ORDER == 2) {
#pragma unroll
                for (int d = 0; d < NB; d++)
#pragma unroll
                    for (int i = 0; i < NA; i++) { const int j = (i + d) % NB; acc[i][j] = MFMA(a[s][i], b[s][j], acc[i][j]); }
            } else {
#pragma unroll
                for (int i = 0; i < NA; i++)
#pragma unroll
                    for (int jj = 0; jj < NB; jj++) { const int j = (i & 1) ? NB - 1 - jj : jj; acc[i][j] = MFMA(a[s][i], b[s][j], acc[i][j]); }
            }
            __builtin_amdgcn_sched_barrier(0);
        }
    float r = 0.f;
    for (int i = 0; i < NA; i++) for (int j = 0; j < NB; j++) r += acc[i][j][0] + acc[i][j][3];
    if (r == 12345.678f) sink[0] = r;
}

template <int NA, int NB, int NSET, int ORDER, int THREADS, int FORM = 0>
void run(const char *name, float scale, float *sink)
{
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    const int iters = 20000 * 16 / (NA * NB) ;
    // spin-up
    for (int r = 0; r < 3; r++) hipLaunchKernelGGL((k<NA, NB, NSET, ORDER, THREADS, FORM>), dim3(256), dim3(THREADS), 0, 0, iters, scale, sink);
    hipDeviceSynchronize();
    for (int rep = 0; rep < 2; rep++) {
        hipEventRecord(e0);
        hipLaunchKernelGGL((k<NA, NB, NSET, ORDER, THREADS, FORM>), dim3(256), dim3(THREADS), 0, 0, iters, scale, sink);
        hipEventRecord(e1); hipEventSynchronize(e1);
        float ms; hipEventElapsedTime(&ms, e0, e1);
        double flop = 256.0 * (THREADS / 64) * (double)iters * NSET * NA * NB * 16 * 16 * 32 * 2;
        printf("%-44s scale %.0f: %8.1f TFLOP/s (%.1f ms)\n", name, scale, flop / ms / 1e9, ms);
    }
    fflush(stdout);
}

int main()
{
    float *sink; hipMalloc(&sink, 64);
    for (float scale : {1.f, 0.f}) {
        run<8, 4, 2, 0, 512, 0>("8 waves 8x4 a-outer builtin", scale, sink);
        run<8, 4, 2, 0, 512, 2>("8 waves 8x4 a-outer asm vgpr acc", scale, sink);
        run<8, 4, 2, 0, 512, 1>("8 waves 8x4 a-outer asm agpr acc", scale, sink);
        run<8, 4, 2, 3, 512, 0>("8 waves 8x4 snake builtin", scale, sink);
        run<8, 4, 2, 3, 512, 1>("8 waves 8x4 snake asm agpr acc", scale, sink);
        run<8, 8, 1, 0, 256, 1>("4 waves 8x8 a-outer asm agpr acc", scale, sink);
        run<8, 8, 1, 3, 256, 1>("4 waves 8x8 snake asm agpr acc", scale, sink);
        run<8, 8, 1, 2, 256, 1>("4 waves 8x8 diagonal asm agpr acc", scale, sink);
        run<8, 4, 2, 0, 256, 0>("4 waves 8x4 a-outer builtin", scale, sink);
        run<8, 4, 2, 0, 512, 0>("8 waves 8x4 a-outer builtin (again)", scale, sink);
    }
    return 0;
}

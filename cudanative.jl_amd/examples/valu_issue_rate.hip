// Issue rate of single vector-ALU instructions on gfx950, from one wavefront per SIMD and from two:
// the conversions that round Float32 sums to Float16 and widen them again (v_cvt_pk_f16_f32,
// v_cvt_f32_f16), the mixed-precision fused multiply-add that would do both in one instruction per
// element (v_fma_mixlo_f16 / v_fma_mixhi_f16, which write one half of a register and keep the other),
// and v_fma_f32 / v_fma_mix_f32 for comparison.  Each wavefront runs 16384 instructions of one kind,
// four independent registers in turn, between two reads of the shader clock.
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++20 valu_issue_rate.hip -o valu_issue_rate && ./valu_issue_rate
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>

#define CHECK(x) do { hipError_t e_ = (x); if (e_ != hipSuccess) { fprintf(stderr, "%s: %s\n", #x, hipGetErrorString(e_)); exit(1); } } while (0)
#define REP8(x) x x x x x x x x
#define REP64(x) REP8(REP8(x))

template <int WHICH>
__global__ void k_rate(long long *out, float a)
{
    float x0 = threadIdx.x, x1 = x0 + 1, x2 = x0 + 2, x3 = x0 + 3;
    unsigned r0 = threadIdx.x, r1 = r0 * 3, r2 = r0 * 5, r3 = r0 * 7;
    const long long t0 = clock64();
    for (int i = 0; i < 64; i++) {
        if constexpr (WHICH == 0) {
            REP64(asm volatile("v_fma_mixlo_f16 %0, %4, %5, %0 op_sel_hi:[0,0,1]\n\tv_fma_mixlo_f16 %1, %4, %6, %1 op_sel_hi:[0,0,1]\n\t"
                               "v_fma_mixhi_f16 %2, %4, %5, %2 op_sel:[0,0,1] op_sel_hi:[0,0,1]\n\tv_fma_mixhi_f16 %3, %4, %6, %3 op_sel:[0,0,1] op_sel_hi:[0,0,1]"
                               : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3) : "s"(a), "v"(x0), "v"(x1));)
        } else if constexpr (WHICH == 1) {
            REP64(asm volatile("v_cvt_pk_f16_f32 %0, %4, %5\n\tv_cvt_pk_f16_f32 %1, %5, %4\n\tv_cvt_f32_f16 %2, %0\n\t"
                               "v_cvt_f32_f16_sdwa %3, %1 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:WORD_1"
                               : "+v"(r0), "+v"(r1), "+v"(r2), "+v"(r3) : "v"(x0), "v"(x1));)
        } else if constexpr (WHICH == 2) {
            REP64(asm volatile("v_fma_f32 %0, %4, %5, %0\n\tv_fma_f32 %1, %4, %5, %1\n\tv_fma_f32 %2, %4, %5, %2\n\tv_fma_f32 %3, %4, %5, %3"
                               : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "s"(a), "v"(r0));)
        } else {
            REP64(asm volatile("v_fma_mix_f32 %0, %4, %5, %0\n\tv_fma_mix_f32 %1, %4, %5, %1\n\tv_fma_mix_f32 %2, %4, %5, %2\n\tv_fma_mix_f32 %3, %4, %5, %3"
                               : "+v"(x0), "+v"(x1), "+v"(x2), "+v"(x3) : "s"(a), "v"(r0));)
        }
    }
    const long long t1 = clock64();
    if (threadIdx.x % 64 == 0) out[threadIdx.x / 64] = t1 - t0;
    if (x0 + x1 + x2 + x3 == 12345.f && r0 + r1 + r2 + r3 == 77) out[0] = 0;  // keeps the chains alive
}

template <int WHICH>
static void run(const char *name, int threads)
{
    long long *d, h[8];
    CHECK(hipMalloc(&d, sizeof h));
    for (int rep = 0; rep < 2; rep++) hipLaunchKernelGGL(k_rate<WHICH>, dim3(1), dim3(threads), 0, 0, d, 1.0f);
    CHECK(hipDeviceSynchronize());
    CHECK(hipMemcpy(h, d, sizeof h, hipMemcpyDeviceToHost));
    printf("%-36s %d wavefront%s per SIMD: %5.2f cycles per instruction and wavefront\n", name, threads / 256, threads > 256 ? "s" : " ",
           (double)h[0] / (64.0 * 64 * 4));
    CHECK(hipFree(d));
}

int main()
{
    for (int threads = 256; threads <= 512; threads += 256) {
        run<1>("v_cvt_pk_f16_f32 / v_cvt_f32_f16", threads);
        run<0>("v_fma_mixlo_f16 / v_fma_mixhi_f16", threads);
        run<2>("v_fma_f32", threads);
        run<3>("v_fma_mix_f32", threads);
    }
    return 0;
}

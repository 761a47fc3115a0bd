// Probe: how fast does the memory system take the D tile stores of a GEMM epilogue, by store pattern?
//
//   hipcc --offload-arch=gfx950 -O3 -std=c++20 cudanative.jl_amd/examples/store_patterns.hip -o /tmp/store_patterns
//   /tmp/store_patterns
//
// 256 workgroups of 512 lanes each write one 256 x 256 Float32 tile of a 4096 x 4096 column-major
// matrix (64 MiB per launch, nothing is read), the tiles dealt to the XCDs as the GEMM kernels deal
// them.  Patterns, 16 bytes per lane and instruction in all of them:
//   accumulator layout: a wavefront's instruction writes 16 columns x 64 contiguous bytes (what an MFMA
//       accumulator tile gives when every lane stores its own registers);
//   128 B / 512 B / 1 KiB pieces: 8 columns x 128 bytes, 2 columns x 512 bytes, 1 column x 1 KiB;
//   the 128-byte pattern again with the sc1, sc0 sc1 and nt cache-policy bits on the store.
// Prints microseconds per launch over 200 back-to-back launches (HIP events), three repetitions.
#include <hip/hip_runtime.h>

#include <cstdio>
#include <cstdlib>
#include <vector>

typedef float float4_t __attribute__((ext_vector_type(4)));
#define CHECK(x)                                                                       \
    do {                                                                               \
        hipError_t e = (x);                                                            \
        if (e != hipSuccess) {                                                         \
            printf("%s failed: %s (line %d)\n", #x, hipGetErrorString(e), __LINE__);   \
            exit(1);                                                                   \
        }                                                                              \
    } while (0)

// workgroup -> tile: consecutive workgroup ids go round-robin over the 8 XCDs; each XCD owns a 4 x 8 block of tiles
__device__ inline void tile_of(int pid, int &ti, int &tj)
{
    const int tiles_j = 16, group_i = 4, per_xcd = 32;
    const int tile_id = (pid & 7) * per_xcd + (pid >> 3);
    const int gsz = group_i * tiles_j, gid = tile_id / gsz, in = tile_id - gid * gsz;
    ti = gid * group_i + in % group_i;
    tj = in / group_i;
}

enum { ACC_LAYOUT, PIECES_128, PIECES_512, PIECES_1K, PIECES_128_SC1, PIECES_128_SC0_SC1, PIECES_128_NT };

template <int MODE>
__global__ __launch_bounds__(512) void k_store(float *D, long ldd, float val)
{
    int ti, tj;
    tile_of(blockIdx.x, ti, tj);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wi = wave % 2, wj = wave / 2;  // a wavefront owns 128 rows x 64 columns of the tile
    const float4_t v = {val, val + 1, val + 2, val + lane};
    float *T = D + (long)(tj * 256) * ldd + ti * 256;
    if constexpr (MODE == ACC_LAYOUT) {
        const int row = wi * 128 + 4 * (lane >> 4), col = wj * 64 + (lane & 15);
#pragma unroll
        for (int b = 0; b < 4; b++)
#pragma unroll
            for (int a = 0; a < 8; a++) *(float4_t *)(T + (long)(col + 16 * b) * ldd + row + 16 * a) = v;
    } else if constexpr (MODE == PIECES_512) {
        const int row = wi * 128 + 4 * (lane & 31), col = wj * 64 + (lane >> 5);
#pragma unroll
        for (int b = 0; b < 32; b++) *(float4_t *)(T + (long)(col + 2 * b) * ldd + row) = v;
    } else if constexpr (MODE == PIECES_1K) {
        const int row = 4 * lane, col = wave * 32;  // (here a wavefront owns 256 rows x 32 columns)
#pragma unroll
        for (int b = 0; b < 32; b++) *(float4_t *)(T + (long)(col + b) * ldd + row) = v;
    } else {
        const int row = wi * 128 + 4 * (lane & 7), col = wj * 64 + (lane >> 3);
#pragma unroll
        for (int b = 0; b < 8; b++)
#pragma unroll
            for (int a = 0; a < 4; a++) {
                float *dst = T + (long)(col + 8 * b) * ldd + row + 32 * a;
                if constexpr (MODE == PIECES_128) *(float4_t *)dst = v;
                if constexpr (MODE == PIECES_128_SC1) asm volatile("global_store_dwordx4 %0, %1, off sc1" ::"v"(dst), "v"(v) : "memory");
                if constexpr (MODE == PIECES_128_SC0_SC1) asm volatile("global_store_dwordx4 %0, %1, off sc0 sc1" ::"v"(dst), "v"(v) : "memory");
                if constexpr (MODE == PIECES_128_NT) asm volatile("global_store_dwordx4 %0, %1, off nt" ::"v"(dst), "v"(v) : "memory");
            }
    }
}

template <int MODE>
float microseconds_per_launch(float *D, int launches)
{
    hipEvent_t e0, e1;
    CHECK(hipEventCreate(&e0));
    CHECK(hipEventCreate(&e1));
    for (int i = 0; i < 20; i++) hipLaunchKernelGGL(k_store<MODE>, dim3(256), dim3(512), 0, 0, D, 4096l, 1.0f);
    CHECK(hipDeviceSynchronize());
    CHECK(hipEventRecord(e0, 0));
    for (int i = 0; i < launches; i++) hipLaunchKernelGGL(k_store<MODE>, dim3(256), dim3(512), 0, 0, D, 4096l, (float)i);
    CHECK(hipEventRecord(e1, 0));
    CHECK(hipEventSynchronize(e1));
    float ms;
    CHECK(hipEventElapsedTime(&ms, e0, e1));
    CHECK(hipEventDestroy(e0));
    CHECK(hipEventDestroy(e1));
    return ms / launches * 1e3f;
}

template <int MODE>
long untouched_after_one_launch(float *D)
{
    CHECK(hipMemset(D, 0xff, 4096l * 4096 * 4));
    hipLaunchKernelGGL(k_store<MODE>, dim3(256), dim3(512), 0, 0, D, 4096l, 1.0f);
    std::vector<unsigned> h(4096l * 4096);
    CHECK(hipMemcpy(h.data(), D, h.size() * 4, hipMemcpyDeviceToHost));
    long n = 0;
    for (unsigned x : h) n += x == 0xffffffffu;
    return n;
}

int main()
{
    float *D;
    CHECK(hipMalloc(&D, 4096l * 4096 * 4));
    // every pattern covers the whole matrix
    const long holes = untouched_after_one_launch<ACC_LAYOUT>(D) + untouched_after_one_launch<PIECES_128>(D) +
                       untouched_after_one_launch<PIECES_512>(D) + untouched_after_one_launch<PIECES_1K>(D) +
                       untouched_after_one_launch<PIECES_128_SC1>(D) + untouched_after_one_launch<PIECES_128_NT>(D);
    printf("elements left unwritten by any pattern: %ld\n", holes);
    if (holes) return 1;
    printf("us per launch, 64 MiB written: accumulator layout | 128 B pieces | 512 B | 1 KiB | 128 B sc1 | 128 B sc0 sc1 | 128 B nt\n");
    for (int rep = 0; rep < 3; rep++) {
        printf("%.2f | %.2f | %.2f | %.2f | %.2f | %.2f | %.2f\n", microseconds_per_launch<ACC_LAYOUT>(D, 200),
               microseconds_per_launch<PIECES_128>(D, 200), microseconds_per_launch<PIECES_512>(D, 200),
               microseconds_per_launch<PIECES_1K>(D, 200), microseconds_per_launch<PIECES_128_SC1>(D, 200),
               microseconds_per_launch<PIECES_128_SC0_SC1>(D, 200), microseconds_per_launch<PIECES_128_NT>(D, 200));
        fflush(stdout);
    }
    CHECK(hipFree(D));
    return 0;
}

/*
 * miwmma.h -- C ABI of libmiwmma.so: WMMA fragment operations and the tiled
 * mixed-precision GEMM built on them, for AMD MI355X (gfx950, wave64, MFMA).
 *
 * This is the boundary that replaces, for the WMMA/GEMM path only, what
 * CUDAnative.jl reaches through CUDAdrv and the NVPTX back end.  Each entry
 * names the reference interface it stands in for (paths relative to the
 * CUDAnative.jl v3.1.0 tree).
 *
 * Conventions
 *   - every function returns 0 on success, a positive hipError_t when the HIP
 *     runtime failed, or a negative MIW_ERR_* code when the library rejected the
 *     arguments; miw_last_error() returns a thread-local message for the last
 *     non-zero return on the calling thread.  Nothing throws or aborts.
 *   - pointers named A, B, C, D, addr, frag are DEVICE pointers unless stated.
 *   - `stream` is a hipStream_t passed as void*; NULL is the default stream.
 *     Launches are asynchronous; the caller keeps buffers alive until
 *     miw_sync() (the GC.@preserve of src/execution.jl:105).
 *   - the library retains no caller pointer past a call.
 *   - a wavefront is 64 lanes: a fragment of the 16x16x16 tile holds 4 elements
 *     per lane for every use (the reference's warp32 held 16/16/8,
 *     src/device/cuda/wmma.jl:413-420).  A fragment image is the wavefront's
 *     registers spilled to memory: element i of lane l at index l*4 + i.
 */
#ifndef MIWMMA_H
#define MIWMMA_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ enums -- */

/* FragmentLayout: RowMajor / ColMajor (src/device/cuda/wmma.jl:313-338). */
enum { MIW_ROW_MAJOR = 0, MIW_COL_MAJOR = 1 };
/* Element types WMMA accepts (src/device/cuda/wmma.jl:11-15). */
enum { MIW_F16 = 0, MIW_F32 = 1 };
/* FragmentUse: MatrixA / MatrixB / Accumulator (src/device/cuda/wmma.jl:343-346). */
enum { MIW_MATRIX_A = 0, MIW_MATRIX_B = 1, MIW_ACCUMULATOR = 2 };
/* Address spaces, numbered as AS.Generic/Global/Shared (src/device/pointer.jl:11-27).
   SHARED stages the tile through LDS inside the kernel and runs the LDS-pointer
   overload of the fragment op, as test/device/wmma.jl:42-46,83-89 do. */
enum { MIW_AS_GENERIC = 0, MIW_AS_GLOBAL = 1, MIW_AS_SHARED = 3 };
/* Broadcast operators over a fragment (src/device/cuda/wmma.jl:703-716). */
enum { MIW_OP_MUL = 0, MIW_OP_ADD = 1 };

enum {
    MIW_OK = 0,
    MIW_ERR_INVALID_VALUE = -1,
    MIW_ERR_INVALID_SHAPE = -2,   /* "Invalid shape for WMMA" (wmma.jl:450-453) */
    MIW_ERR_INVALID_LAYOUT = -3,  /* "Invalid layout for WMMA" (wmma.jl:442-448) */
    MIW_ERR_INVALID_TYPE = -4,    /* "Invalid element type for WMMA" (wmma.jl:460-477) */
    MIW_ERR_INVALID_AS = -5,      /* "Invalid address space for WMMA" (wmma.jl:434-440) */
    MIW_ERR_MISALIGNED = -6,
    MIW_ERR_NULL_POINTER = -7,
    MIW_ERR_NOT_INITIALIZED = -8,
    MIW_ERR_UNSUPPORTED = -9,
    MIW_ERR_NOT_FOUND = -10
};

/* -------------------------------------------------------------- lifecycle -- */

/* Select the device and check it is a gfx950 part.  Replaces the lazy context
   creation of src/init.jl:101-112 (context()) for one GPU. */
int miw_init(int device);

/* Message for the last failing call on this thread ("" if none). */
const char *miw_last_error(void);

/* Hash of the sources this library was compiled from (16 hex digits; the build recipe computes
   it), so that tests and benchmarks can tell a stale binary from a current one. */
const char *miw_build_id(void);

typedef struct miw_device_info {
    char name[128];
    char arch[64];
    int cu_count;
    int wave_size;
    int clock_mhz;          /* peak engine clock */
    int mem_clock_mhz;
    int mem_bus_bits;
    int l2_bytes;
    int max_threads_per_block;
    size_t lds_per_block;   /* bytes a workgroup may allocate */
    size_t hbm_bytes;
    double peak_f16_tflops; /* cu_count * 4 SIMD * 1024 flop/clk * clock */
} miw_device_info;

/* Device properties (CUDAdrv device attributes used by src/execution.jl:418-426
   warpsize helpers and by the occupancy callback). */
int miw_device_info_get(miw_device_info *out);

/* ----------------------------------------------------------------- memory -- */
/* CuHostArray: Mem.alloc / Mem.free / unsafe_copyto! (src/array.jl:20-60). */
int miw_malloc(void **out, size_t bytes);
int miw_free(void *p);
int miw_memcpy_h2d(void *dst, const void *src_host, size_t bytes);
int miw_memcpy_d2h(void *dst_host, const void *src, size_t bytes);
int miw_memcpy_d2d(void *dst, const void *src, size_t bytes);
int miw_memset(void *dst, int byte, size_t bytes);
/* Free and total device memory in bytes: what the OOM -> GC.gc() -> retry path of the allocator
   (src/array.jl:23-29) consults, and what a test of an allocation-free call compares. */
int miw_mem_info(size_t *free_bytes, size_t *total_bytes);

/* stream= keyword of @cuda (src/execution.jl:59-63); synchronize() */
int miw_stream_create(void **out);
int miw_stream_destroy(void *stream);
int miw_sync(void *stream);

/* CuEvent timing as used by test/perf/launch_overhead. */
int miw_event_create(void **out);
int miw_event_destroy(void *event);
int miw_event_record(void *event, void *stream);
int miw_event_synchronize(void *event);
int miw_event_elapsed_ms(float *ms, void *start, void *stop);

/* ------------------------------------------------------- fragment operations */
/* Each call launches one wavefront (1 block x 64 threads; the reference
   launches 1 x 32, examples/wmma/high-level.jl:46). */

/* Elements per lane of a fragment: 4 for every (use, dtype) of the 16x16x16 tile. */
int miw_frag_elems_per_lane(int use, int dtype);
/* Bytes of a fragment image (64 lanes). */
size_t miw_frag_image_bytes(int use, int dtype);

/* load_a / load_b / load_c (src/device/cuda/wmma.jl:507-530;
   llvm_wmma_load_* :104-137).  use selects a/b/c; A and B must be MIW_F16.
   stride is the leading dimension in elements. M,N,K must be 16. */
int miw_frag_load(int use, int dtype, int layout, int addr_space, int m, int n, int k,
                  const void *addr, int64_t stride, void *frag, void *stream);

/* store_d (src/device/cuda/wmma.jl:613-632; llvm_wmma_store_d_* :162-191). */
int miw_frag_store(int dtype, int layout, int addr_space, int m, int n, int k,
                   void *addr, const void *frag, int64_t stride, void *stream);

/* fill_c (src/device/cuda/wmma.jl:654-667). */
int miw_frag_fill(int dtype, float value, void *frag, void *stream);

/* f.(frag, scalar) broadcasting (src/device/cuda/wmma.jl:678-716): out[i] =
   scalar op in[i] in the fragment's element type, n_elems elements in total. */
int miw_frag_map(int dtype, int op, float scalar, const void *in, void *out, size_t n_elems, void *stream);

/* mma (src/device/cuda/wmma.jl:558-583; llvm_wmma_mma_* :222-257):
   D = A*B + C on one 16x16x16 tile, A and B Float16, C and D independently
   Float16 or Float32.  a_layout/b_layout are the layouts the fragments were
   loaded with (part of the reference's fragment type); they are validated only:
   the lane layout here does not depend on them. */
int miw_frag_mma(int a_layout, int b_layout, int c_type, int d_type,
                 const void *a_frag, const void *b_frag, const void *c_frag, void *d_frag, void *stream);

typedef struct miw_mac_desc {
    int m, n, k;                 /* must be 16,16,16 */
    int a_layout, b_layout, c_layout, d_layout;
    int c_type, d_type;
    int use_c;                   /* 1: load_c (MAC); 0: fill_c(0) (MUL) */
    int addr_space;              /* MIW_AS_* for every operand */
    float alpha, beta;           /* a_frag = alpha .* a_frag (rounded to Float16),
                                    c_frag = beta .* c_frag (in c_type) */
    int64_t lda, ldb, ldc, ldd;
} miw_mac_desc;

/* The whole kernel of examples/wmma/high-level.jl:30-44 and of
   test/device/wmma.jl:212-231 fused in one launch: load_a, load_b,
   load_c | fill_c(0), alpha .* a, beta .* c, mma, store_d. */
int miw_wmma_mac(const miw_mac_desc *desc, const void *A, const void *B, const void *C, void *D, void *stream);

/* ------------------------------------------------------------------- GEMM -- */

typedef struct miw_gemm_desc {
    int64_t m, n, k;
    int64_t lda, ldb, ldc, ldd;          /* leading dimensions in elements */
    int a_layout, b_layout, c_layout, d_layout;
    int c_type, d_type;                  /* A and B are Float16 */
    int acc_type;                        /* MIW_F32: fp32 accumulate.  MIW_F16: the
                                            running sum is rounded to Float16 after
                                            every acc_chunk k-values (needs c_type =
                                            d_type = MIW_F16) */
    int acc_chunk;                       /* 0 = variant's default */
    float alpha, beta;
    int use_c;                           /* 0: C is never read (fill_c(0)) */
    int64_t batch;                       /* >= 1 */
    int64_t stride_a, stride_b, stride_c, stride_d; /* elements between problems */
    int variant;                         /* 0 = pick; see miw_gemm_variant_* */
} miw_gemm_desc;

/* D = alpha*A*B + beta*C, the chain of mma calls the reference describes
   (docs/src/device/wmma.md:51-52) carried over the whole K extent.  M, N, K
   must be multiples of 16; the LDS-tiled variants need multiples of their tile
   (otherwise the fragment-op variant is used). */
int miw_gemm(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, void *stream);

/* Enumerate kernel variants (variant ids are 1..count). */
int miw_gemm_variant_count(void);
typedef struct miw_gemm_variant_info {
    char name[64];
    int block_m, block_n, block_k;
    int waves_m, waves_n;
    int stages;
    int lds_bytes;
    int fragment_ops;   /* 1: built from load_a/load_b/mma on global memory, no LDS */
    int f16_accumulate; /* 1: has a Float16-accumulate form (accumulators fit in ordinary VGPRs) */
    int pingpong;       /* 1: the two wavefronts of a SIMD alternate between matrix-core and memory phases;
                           2: one wavefront per SIMD with a 128x128 sub-tile issues its memory instructions
                           between its MFMAs (K of at least 128); either way lds_bytes is the largest ring
                           over the operand layouts */
} miw_gemm_variant_info;
int miw_gemm_variant_info_get(int variant, miw_gemm_variant_info *out);
/* *supported = 1 when `variant` (1..count) can run this descriptor (M and N of at least one tile,
   K of at least 64, leading dimensions, accumulate type; pointers are assumed
   16-byte aligned and C and D apart), else 0. */
int miw_gemm_variant_supports(const miw_gemm_desc *desc, int variant, int *supported);
/* Variant of a single launch of this descriptor (what miw_gemm runs unless miw_gemm_plan
   cuts the problem up): the one with the shortest estimated duration
   (rounds of workgroups over the CUs, C and D traffic, and the K loop at each kernel's measured
   pace per 64 k-values) among those that can run it. */
int miw_gemm_pick_variant(const miw_gemm_desc *desc, int *variant);
/* The launches miw_gemm makes for this descriptor (no counterpart in the reference, whose GEMM
   would be the caller's own kernel over docs/src/device/wmma.md:51-52).  The LDS-tiled kernels take any M and N of
   at least one tile and any K of at least 64 (multiples of 16, as everywhere).  Where the tile does
   not divide an extent the last tile is shifted back so that it ends at the edge and overlaps its
   neighbour; both workgroups compute the overlap from the same operands in the same order and
   store equal values.  When C and D share memory (in_place != 0 here; miw_gemm looks at the
   pointers) that is not allowed and only whole tiles are used.  Where 64 does not divide K the
   last slot of 64 k-values is shifted back so that it ends at K, and the k-values it repeats are
   zeroed in the fragments: K is never cut, and with Float16 accumulation the last rounding follows
   the last K mod 64 k-values.  Beyond that, with Float32 accumulation and desc.variant 0, a problem
   is cut into parts, each a GEMM on a block of D with offset pointers, launched in order on the
   caller's stream, where the estimate says that is faster:
     whole large tiles, then a bottom strip and a right strip, each planned again (4160 rows:
       sixteen rows of 256 x 256 tiles and a strip of 64 x 64 tiles rather than seventeen rows of
       large tiles, which would take two rounds over the CUs).
   Writes min(*count, capacity) parts; *count is the number of launches. */
typedef struct miw_gemm_part {
    int variant;          /* as in miw_gemm_desc.variant */
    int reserved;
    int64_t m0, n0, k0;   /* first row, column and k-value of the part in the caller's problem */
    int64_t m, n, k;      /* its sizes */
} miw_gemm_part;
int miw_gemm_plan(const miw_gemm_desc *desc, int in_place, miw_gemm_part *parts, int capacity, int *count);
/* acc_chunk miw_gemm would use for this descriptor (fp16 accumulate only).  Like
   miw_gemm_pick_variant it sees no pointers and assumes 16-byte aligned operands with C and D
   apart; operands that are not (or a C that is D, with M or N no whole number of tiles) can send
   miw_gemm to another kernel with another acc_chunk: miw_gemm_resolve answers for the real ones. */
int miw_gemm_acc_chunk(const miw_gemm_desc *desc, int *acc_chunk);
/* What miw_gemm(desc, A, B, C, D, ...) will run, from the same checks and plan but without a
   launch: *variant = the variant of its first launch, *acc_chunk = the k-values between two
   roundings of the Float16 running sum (0 with Float32 accumulation).  Either output may be null.
   No counterpart in the reference (its mma chain always rounds once per 16 x 16 x 16 tile). */
int miw_gemm_resolve(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, const void *D,
                     int *variant, int *acc_chunk);

/* Split-K form of miw_gemm for problems with few output tiles and a long K: the chain of mma
   calls over K (docs/src/device/wmma.md:51-52) is cut into `splits` equal slices (each a multiple
   of 64 k-values), the LDS-tiled kernels write every slice's product as Float32 into `workspace`
   (splits * m * n * 4 bytes, 16-byte aligned, contents on entry irrelevant), and a second kernel
   adds the slices in order: D = alpha * sum_s A_s*B_s + beta*C.  The result does not depend on
   timing; it differs from miw_gemm's by the rounding of one Float32 sum per slice.  Float32
   accumulation, batch 1, desc.variant 0, M and N of at least one LDS tile (64).  splits = 0 chooses
   the slice count with the shortest estimated duration (both kernels and the workspace traffic
   counted).  One slice, asked for or chosen, is the plain launch of miw_gemm: no workspace
   (0 bytes, `workspace` may be null) and no second kernel.  miw_gemm_splitk_workspace reports
   the slice count and the bytes miw_gemm_splitk will ask for. */
int miw_gemm_splitk_workspace(const miw_gemm_desc *desc, int splits, int *splits_out, size_t *bytes);
int miw_gemm_splitk(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, int splits,
                    void *workspace, size_t workspace_bytes, void *stream);

/* miw_gemm_splitk for callers that cannot allocate device memory (tight serving loops, harnesses
   that forbid hipMalloc).  It has no counterpart in the reference.
   Same kernels and results as miw_gemm_splitk, with the slices going through a workspace that is
   part of the library's device code: miw_gemm_splitk_static_capacity() bytes (32 MiB) that every
   GPU the library runs on holds until the process ends.  It calls no hipMalloc, hipFree or other
   allocating routine, and refuses (MIW_ERR_UNSUPPORTED) a problem whose splits * m * n * 4 bytes
   exceed the capacity.  All calls on one GPU share that GPU's workspace: calls that overlap on one
   GPU (two streams, two host threads) race; calls on one stream are ordered and safe.  Nothing in
   the workspace needs clearing: the first pass writes every element the second pass reads.
   splits = 0 chooses among the slice counts whose partial products fit the capacity (one slice, the
   plain launch, always does).  miw_gemm_splitk_static_plan reports the count and the bytes of the
   static workspace a call will use, without touching the device. */
int miw_gemm_splitk_static(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D, int splits,
                           void *stream);
size_t miw_gemm_splitk_static_capacity(void);
int miw_gemm_splitk_static_plan(const miw_gemm_desc *desc, int splits, int *splits_out, size_t *bytes);

/* warmup untimed launches, then iters launches each bracketed by HIP events on
   `stream`; ms_each[i] receives launch i's duration in milliseconds. */
int miw_gemm_bench(const miw_gemm_desc *desc, const void *A, const void *B, const void *C, void *D,
                   void *stream, int warmup, int iters, float *ms_each);

/* Register-resident back-to-back v_mfma_f32_16x16x32_f16 on every CU (the idea
   of examples/peakflops.jl): measured TFLOP/s of the matrix cores alone. */
int miw_mfma_peak_probe(int iters, double *tflops, void *stream);

/* The same chain on operands that change every k-step (register-resident sets, all zero or
   pseudo-random in [-1, 1)), one 8-wavefront workgroup per CU: what the matrix cores sustain
   under the power cap, and the shader clock (MHz, mean over the CUs) they run at meanwhile. */
int miw_mfma_power_probe(int iters, int random_operands, double *tflops, double *shader_mhz, void *stream);

/* The raw-driver leg of the launch-overhead benchmark (test/perf/launch_overhead/cuda.c:60-80):
   iters times { record event; launch the dummy kernel with `threads` lanes; record event;
   synchronize }, all inside the library with no foreign-function hop; cpu_us[i] receives the
   host wall time of iteration i and gpu_us[i] the time between the two events, both in
   microseconds.  The other leg launches "dummy_store" through miw_launch from the host language. */
int miw_launch_overhead_probe(int iters, int threads, float *cpu_us, float *gpu_us);

/* Plain device copy kernel (16 B per lane), used to calibrate HBM counters. */
int miw_copy_probe(void *dst, const void *src, size_t bytes, void *stream);

/* ----------------------------------------------------------- generic launch */
/* @cuda threads= blocks= shmem= stream= f(args...) (src/execution.jl:45-114)
   and cufunction / HostKernel (:205-219, :290-297) for the kernels compiled into
   this library: look a kernel up by name, query its attributes
   (registers/memory/maxthreads, :227-266), launch it with raw argument slots. */
int miw_kernel_count(void);
int miw_kernel_name(int index, char *buf, size_t buflen);
int miw_kernel_lookup(const char *name, void **kernel);

typedef struct miw_kernel_attributes {
    int num_regs;
    int max_threads_per_block;
    size_t static_shared_bytes;
    size_t local_bytes;
    size_t const_bytes;
} miw_kernel_attributes;
int miw_kernel_attributes_get(void *kernel, miw_kernel_attributes *out);
/* config= occupancy callback of @cuda (src/execution.jl:59-63):
   hipOccupancyMaxPotentialBlockSize for this kernel. */
int miw_kernel_occupancy(void *kernel, size_t dynamic_shmem, int *min_grid, int *block);
int miw_launch(void *kernel, const unsigned grid[3], const unsigned block[3], unsigned shmem,
               void *stream, void **args);

/* Kernels of the caller's own: what cufunction ends in, CuModule(image) and CuFunction(mod, name)
   (src/execution.jl:300-342), for code objects compiled ahead of time (hipcc --genco
   --offload-arch=gfx950; the device-side fragment API is include/miwmma_fragment.hpp).  `image` is
   a host buffer holding an ELF code object or a clang offload bundle; it may be released after the
   call.  Kernels obtained from a module work with miw_kernel_attributes_get,
   miw_kernel_occupancy and miw_launch (at most 64 KiB of dynamic LDS) until the module is
   unloaded; unloading while one of its kernels is still running is undefined. */
int miw_module_load(const void *image, size_t bytes, void **module);
int miw_module_get_kernel(void *module, const char *name, void **kernel);
int miw_module_unload(void *module);

#ifdef __cplusplus
}
#endif
#endif /* MIWMMA_H */

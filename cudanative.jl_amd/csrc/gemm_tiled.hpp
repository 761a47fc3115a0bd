// LDS-tiled mixed-precision GEMM for gfx950: D = alpha * A*B + beta * C with
// Float16 A and B, fp32 accumulation in v_mfma_f32_16x16x32_f16 (optionally
// rounded to Float16 every 64 k-values: the fp16-accumulate variant).
//
// It is the chain "D of one mma is C of the next" (CUDAnative.jl
// docs/src/device/wmma.md:51-52) carried over K, with the fragment loads of
// src/device/cuda/wmma.jl:507-530 split in two: global -> LDS by 16-byte
// direct-to-LDS loads, LDS -> registers in the matrix cores' operand layout.
//
// Canonical problem.  The kernel computes P = X * Y where P is I x J and is
// stored with I contiguous.  For a column-major D this is X = A, Y = B,
// I = M, J = N; for a row-major D the host passes X = B^T, Y = A^T, I = N,
// J = M (same memory, roles swapped), so both D layouts write 16 contiguous
// bytes per lane.  X is "K-major" when its k index is contiguous in memory
// (A row-major / B column-major) and "I-major" otherwise; likewise Y.
//
// Pipeline.  K is consumed in steps of 32 k-values (one MFMA k-step), fetched
// in pairs: LDS holds two to four slots of 64 k-values (as many as fit).  While the matrix cores work
// through the fragments of step s out of one register set, the fragments of
// step s+1 are read from LDS into a second set (reads first, so that they have
// landed long before the step ends), and the direct-to-LDS loads of the next
// pair are in flight.  One s_barrier per pair publishes the pair that landed
// and frees the slot of the pair that has been read.
//
// LDS slot layouts (16-byte chunks of 8 k-values or 8 i-values), chosen so that
// every 8 consecutive lanes of a direct-to-LDS load fetch one full 128-byte
// line and every fragment read is free of bank conflicts:
//   K-major operand, R rows of 128 bytes: chunk (r, c), c = 0..7, sits at chunk
//       index r*8 + (c ^ ((r >> 1) & 7)).  A lane reads its 8 k-values of a
//       32-k step with one ds_read_b128.
//   I-major operand (64 k-rows of R contiguous i): row pieces of 64 i (128 B)
//       at chunk index ((i/64)*64 + k)*8 + (c ^ 2g(k)), c = 0..7,
//       g(k) = ((k>>1)&1) | (((k>>3)&1)<<1).  A fragment is fetched with two
//       ds_read_b64_tr_b16 (the LDS transpose read): 16 lanes pick up 4 k-rows
//       x 16 i and each lane receives 4 consecutive k-values of its row; the
//       XOR spreads the 16 row pieces of one read over all banks.
//   Direct-to-LDS loads write lane-contiguous 1 KiB per wavefront instruction;
//   the layouts above are produced by choosing which global chunk each lane
//   fetches.
#pragma once
#include "kernels.hpp"

#include <utility>

namespace miw {

typedef _Float16 half_t;
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef __fp16 fp16x4_t __attribute__((ext_vector_type(4)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef unsigned int uint2_t __attribute__((ext_vector_type(2)));
typedef unsigned int uint4_t __attribute__((ext_vector_type(4)));

#define MIW_LDS __attribute__((address_space(3)))
#define MIW_GLOBAL __attribute__((address_space(1)))

// Measurement switch, 0 in every shipped build: bit 0 drops the direct-to-LDS loads of the K loop,
// bit 1 its fragment reads (the registers keep the prologue's fragments), bit 2 its MFMAs.  The
// results are wrong; the timings say what each unit costs in cycles and, under the power cap, in clock.
#ifndef MIW_PP_ABLATE
#define MIW_PP_ABLATE 0
#endif

constexpr int BKS = 32;    // k-values per pipeline step (one MFMA k-step)
constexpr int KGRAN = 64;  // k-values per LDS slot and K granularity of the kernel

struct tiled_params {
    const half_t *X;
    const half_t *Y;
    const void *C;
    void *D;
    // K: any multiple of 16 from 64 up.  The kernels walk K in slots of 64; when 64 does not divide K
    // the last slot is shifted back to end at K, and the k-values it repeats from the slot before
    // (the first 64 * ceil(K / 64) - K of it) are zeroed in the fragments of both operands.
    int I, J, K;
    long ldx, ldy, ldc, ldd;
    long sx, sy, sc, sd;
    int c_trans;  // C is stored with J contiguous (its layout differs from D's)
    int use_c;
    float alpha, beta;
    // tiles_i = ceil(I / BI), tiles_j = ceil(J / BJ).  Where the tile does not divide an extent the
    // last tile starts at I - BI (J - BJ) and overlaps its neighbour: both workgroups compute the
    // overlap from the same operands in the same order and store equal values.  The host allows
    // this only when C and D do not share memory.
    int tiles_i, tiles_j, group_i;
#ifdef MIW_PP_TS
    long long *ts;  // measurement builds: 10 counters per wavefront (see k_gemm_pp64), or null
#endif
};

// s_waitcnt vmcnt(N) lgkmcnt(0); s_barrier.  The direct-to-LDS loads are issued
// from inline assembly (the compiler's own wait-count pass would otherwise
// serialise them with every LDS read of the other slot), so their completion is
// tracked by hand: vmcnt(N) leaves the N youngest in flight.  The wait itself
// is the compiler builtin, so that the compiler knows the LDS reads issued so
// far have landed; the empty asm statements keep LDS reads and loads from
// moving across the barrier.
template <int N>
__device__ inline void wait_loads_and_barrier()
{
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt((N & 15) | (7 << 4) | (0 << 8) | ((N >> 4) << 14));
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

// One 16-byte-per-lane direct-to-LDS load: lane l fetches base + voff[l] and
// the wavefront's 1 KiB lands at LDS byte lds_addr + 16*l.
__device__ inline void lds_dma16(const void *base, unsigned voff, unsigned lds_addr)
{
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
                 :
                 : "s"(lds_addr), "v"(voff), "s"(base)
                 : "memory", "m0");
}

// The same with a compile-time byte offset added to the global address.  The
// instruction's offset field advances the LDS address as well as the global
// one, so M0 is set back by as much.
template <int IMM>
__device__ inline void lds_dma16_imm(const void *base, unsigned voff, unsigned lds_addr)
{
    static_assert(IMM >= 0 && IMM < 4096, "instruction offset field");
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%3"
                 :
                 : "s"(lds_addr - (unsigned)IMM), "v"(voff), "s"(base), "n"(IMM)
                 : "memory", "m0");
}

// The same with both addresses given as a uniform base plus a compile-time byte offset: lane l
// fetches base + G_IMM + voff[l] into LDS byte lds_base + DST_IMM + 16*l.  M0 is written by the
// addition itself (the instruction's offset field advances the LDS address as well as the global
// one, so M0 is set back by as much).
template <int DST_IMM, int G_IMM>
__device__ inline void lds_dma16_at(const void *base, unsigned voff, unsigned lds_base)
{
    static_assert(G_IMM >= 0 && G_IMM < 4096, "instruction offset field");
    asm volatile("s_add_u32 m0, %0, %3\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2 offset:%4"
                 :
                 : "s"(lds_base), "v"(voff), "s"(base), "n"(DST_IMM - G_IMM), "n"(G_IMM)
                 : "memory", "m0", "scc");
}

__device__ inline int i_major_swizzle(int k) { return ((k >> 1) & 1) | (((k >> 3) & 1) << 1); }

// ------------------------------------------------------------ slot loader --
// Fetches one slot (R rows/columns x 64 k-values) with NT threads.  Thread t
// owns LDS chunks t, t + NT, t + 2 NT, ...; their global sources differ by
// offsets that are the same for every thread, so one lane offset is kept and
// the rest is scalar address arithmetic.
template <int R, bool KMAJOR, int NT>
struct slot_loader {
    static constexpr int CHUNKS = R * KGRAN / 8;
    static constexpr int NLOAD = CHUNKS / NT;
    static_assert(CHUNKS % NT == 0 && (NT == 256 || NT == 512), "slot must divide over the workgroup");

    // Byte offset, relative to the slot origin in global memory, of the chunk
    // this thread fetches first.
    __device__ static inline unsigned lane_offset(int tid, int ld)
    {
        if constexpr (KMAJOR) {
            const int r = tid >> 3, cpos = tid & 7;
            const int c = cpos ^ ((r >> 1) & 7);
            return 2u * (unsigned)(r * ld + c * 8);
        } else {
            const int k = (tid >> 3) & 63, cpos = tid & 7;  // tid / 512 == 0
            const int c = cpos ^ (2 * i_major_swizzle(k));
            return 2u * (unsigned)(k * ld + c * 8);
        }
    }

    // Element offset of load i relative to load 0 (uniform).
    __device__ static inline long load_delta(int i, long ld)
    {
        if constexpr (KMAJOR) {
            return (long)i * (NT / 8) * ld;  // NT/8 rows further down
        } else {
            const int k = (i * (NT / 8)) & 63, iblk = (i * NT) / 512;
            return (long)k * ld + iblk * 64;
        }
    }

    // base: uniform global address of the slot origin; lds_wave: this
    // wavefront's first destination byte for load 0 (uniform).
    __device__ static inline void issue(const half_t *base, long ld, unsigned voff, unsigned lds_wave)
    {
#pragma unroll
        for (int i = 0; i < NLOAD; i++) lds_dma16(base + load_delta(i, ld), voff, lds_wave + (unsigned)(i * NT * 16));
    }
};

// --------------------------------------------------------- fragment reads --
// Lane byte offsets (within the operand's LDS slot) of the wavefront's
// fragments; MFMA tile t and step-in-slot h add compile-time constants.
template <int R, bool KMAJOR>
struct frag_reader {
    static constexpr int READS_PER_FRAG = KMAJOR ? 1 : 2;
    int base[4];  // K-major: [h] (the XOR involves h); I-major: [t % 4]

    __device__ inline void init(int wave_row0, int lane)
    {
        const int j = lane & 15, q = lane >> 4;
        if constexpr (KMAJOR) {
            const int r = wave_row0 + j;
            base[0] = (r * 8 + ((0 + q) ^ ((j >> 1) & 7))) * 16;
            base[1] = (r * 8 + ((4 + q) ^ ((j >> 1) & 7))) * 16;
            base[2] = base[3] = 0;
        } else {
            const int jq = j >> 2, jr = j & 3;
            const int g = ((jq >> 1) & 1) | ((q & 1) << 1);  // i_major_swizzle of this lane's k
            const int w16 = wave_row0 / 16;
#pragma unroll
            for (int m = 0; m < 4; m++)
                base[m] = (w16 / 4) * 8192 + (8 * q + jq) * 128 + jr * 8 + ((((w16 & 3) + m) & 3) ^ g) * 32;
        }
    }

    template <int T, int H>
    __device__ inline half8_t read(MIW_LDS const char *slot) const
    {
        if constexpr (KMAJOR) {
            return *(MIW_LDS const half8_t *)(slot + base[H] + T * 2048);
        } else {
            const int off = base[T & 3] + (T >> 2) * 8192 + H * 4096;
            fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16((MIW_LDS fp16x4_t *)(slot + off));
            fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16((MIW_LDS fp16x4_t *)(slot + off + 512));
            uint2_t l2 = __builtin_bit_cast(uint2_t, lo), h2 = __builtin_bit_cast(uint2_t, hi);
            uint4_t v = {l2[0], l2[1], h2[0], h2[1]};
            return __builtin_bit_cast(half8_t, v);
        }
    }
};

__device__ inline float round_through_half(float v) { return (float)(half_t)v; }

// K tail.  A lane's fragment of k-step H of a slot holds the 8 k-values 32 H + 8 q .. + 7 of the slot
// (q = lane / 16), whichever operand layout it was read from.  In a last slot whose first `skip`
// k-values (a multiple of 16) repeat the slot before, tail_keep is all ones for a lane whose values
// count and zero otherwise.  The lane number is taken anew here: the mask is needed once per launch and
// must not hold registers through the K loop.
template <int H>
__device__ inline unsigned tail_keep(int skip)
{
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    return 32 * H + 8 * (lane >> 4) >= skip ? 0xffffffffu : 0u;
}
// The masks are applied without a branch, in copies of the loop body that only the last pair runs
// (a fragment that is changed on one side of a branch costs a second register set and a copy on the
// other side, in every trip of the K loop).
__device__ inline void tail_apply(half8_t &f, unsigned keep)
{
    uint4_t v = __builtin_bit_cast(uint4_t, f);
#pragma unroll
    for (int e = 0; e < 4; e++) v[e] &= keep;
    f = __builtin_bit_cast(half8_t, v);
}

// Epilogue store of two MFMA tiles that are neighbours along the contiguous dimension of D: tile rows
// row .. row + 15 (values v0) and row + 16 .. row + 31 (values v1) of the 16 columns col0 .. col0 + 15.
// In the accumulator layout a lane holds 4 consecutive rows of one column (lane % 16), the four lanes
// of a column 16 rows: one store instruction would write 16 pieces of 64 bytes (32 for Float16).  Here
// neighbouring lanes swap one tile's values (a DPP move inside the quad), so that the even columns go
// out with the first instruction and the odd ones with the second, each column as one piece of 128
// bytes (64 for Float16): whole cache lines when the tile starts on one.
__device__ inline unsigned quad_swap(unsigned v)
{
    return (unsigned)__builtin_amdgcn_mov_dpp((int)v, 0xB1 /* quad_perm:[1,0,3,2] */, 0xf, 0xf, true);
}
template <class DT>
__device__ inline void store_tile_pair(DT *D, long ldd, int row, int col0, int lane, float4_t v0, float4_t v1)
{
    const int r = lane & 15, q = lane >> 4;
    const bool odd = r & 1;
    // both instructions: this lane writes rows row + 16 * odd + 4 q .. + 3; column col0 + r - odd, then the next
    DT *dst = D + (long)(col0 + r - (odd ? 1 : 0)) * ldd + (row + (odd ? 16 : 0) + 4 * q);
    if constexpr (__is_same(DT, float)) {
        const uint4_t p = __builtin_bit_cast(uint4_t, v0), t = __builtin_bit_cast(uint4_t, v1);
        uint4_t s0, s1;
#pragma unroll
        for (int e = 0; e < 4; e++) {
            const unsigned ps = quad_swap(p[e]), ts = quad_swap(t[e]);
            s0[e] = odd ? ts : p[e];   // even column: own upper tile | the even neighbour's lower tile
            s1[e] = odd ? t[e] : ps;   // odd column: the odd neighbour's upper tile | own lower tile
        }
        *(uint4_t *)dst = s0;
        *(uint4_t *)(dst + ldd) = s1;
    } else {
        const half4_t h0 = {(half_t)v0[0], (half_t)v0[1], (half_t)v0[2], (half_t)v0[3]};
        const half4_t h1 = {(half_t)v1[0], (half_t)v1[1], (half_t)v1[2], (half_t)v1[3]};
        const uint2_t p = __builtin_bit_cast(uint2_t, h0), t = __builtin_bit_cast(uint2_t, h1);
        uint2_t s0, s1;
#pragma unroll
        for (int e = 0; e < 2; e++) {
            const unsigned ps = quad_swap(p[e]), ts = quad_swap(t[e]);
            s0[e] = odd ? ts : p[e];
            s1[e] = odd ? t[e] : ps;
        }
        *(uint2_t *)dst = s0;
        *(uint2_t *)(dst + ldd) = s1;
    }
}

// Ordinal of the direct-to-LDS load issued after MFMA m of a step of nmfma
// matrix instructions that issues ndma loads, or -1.  The loads are spread
// evenly over the step: a wavefront's load occupies the texture-address path
// for some twenty cycles, and eight wavefronts that issue theirs back to back
// fill its queue and then stand still, MFMAs included, until it drains.
constexpr int dma_after_mfma(int m, int nmfma, int ndma)
{
    for (int k = 0; k < ndma && k < nmfma; k++)
        if (k * nmfma / (ndma < nmfma ? ndma : nmfma) == m) return k;
    return -1;
}

// MFMA number m of a step works on tile (m / tj, serpentine_column(m, tj)): rows of tiles are
// walked alternately left to right and right to left, so that every MFMA changes exactly one of
// its two operand fragments.  Under the power cap that is worth 7 % of matrix-core throughput on
// random data against the row-by-row order, in which both operands change at the end of a row.
constexpr int serpentine_column(int m, int tj) { return ((m / tj) & 1) ? tj - 1 - m % tj : m % tj; }

template <int TI, int TJ>
struct frag_set {
    half8_t x[TI];
    half8_t y[TJ];
};

// ----------------------------------------------------------------- kernel --
// Wavefronts per SIMD the register allocation aims at: two whenever the
// accumulators (BI*BJ/NT floats per lane) leave room for the fragments in 256
// registers, which also keeps them in ordinary VGPRs where the fp16-accumulate
// rounding can reach them without copies.
constexpr int waves_per_simd(int bi, int bj, int nt) { return bi * bj / nt <= 128 ? 2 : 1; }

// MFMA tiles of C that one trip of the loop's tail folds into the accumulators
// (0: the variant does not fold).  Folding needs the accumulators in ordinary
// VGPRs, at most one pair in flight across a barrier, and LDS room for two
// staging buffers of that many 1 KiB tiles per wavefront.  Only the 8-wavefront
// tiles fold: the 4-wavefront kernels issue half as many loads per thread again
// and the register allocator answers the unrolled tail with spills.
constexpr int fold_tiles(int bi, int bj, int nt, int nslot)
{
    if (waves_per_simd(bi, bj, nt) < 2 || nslot > 3 || nt != 512) return 0;
    for (int cpt = 2; cpt >= 1; cpt--)
        if (nslot * (bi + bj) * KGRAN * 2 + (nt / 64) * 2 * cpt * 1024 <= 160 * 1024) return cpt;
    return 0;
}
constexpr int fold_stage_bytes(int bi, int bj, int nt, int nslot) { return (nt / 64) * 2 * fold_tiles(bi, bj, nt, nslot) * 1024; }

template <int BI, int BJ, int WI, int WJ, int NSLOT, bool XK, bool YK, class CT, class DT, bool F16ACC>
__global__ __launch_bounds__(WI *WJ * 64) __attribute__((amdgpu_waves_per_eu(waves_per_simd(BI, BJ, WI *WJ * 64))))
void k_gemm_tiled(tiled_params p)
{
    constexpr int NT = WI * WJ * 64;
    constexpr int WTI = BI / WI, WTJ = BJ / WJ;
    constexpr int TI = WTI / 16, TJ = WTJ / 16;
    constexpr int XBYTES = BI * KGRAN * 2, YBYTES = BJ * KGRAN * 2, SLOT = XBYTES + YBYTES;
    using xload = slot_loader<BI, XK, NT>;
    using yload = slot_loader<BJ, YK, NT>;
    using xreader = frag_reader<BI, XK>;
    using yreader = frag_reader<BJ, YK>;
    constexpr int NREAD = TI * xreader::READS_PER_FRAG + TJ * yreader::READS_PER_FRAG;
    constexpr int NMFMA = TI * TJ;
    static_assert(WTI % 32 == 0 && WTJ % 32 == 0, "wave tile");

    extern __shared__ __attribute__((aligned(128))) char smem[];
    MIW_LDS char *lds = (MIW_LDS char *)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wi = wave % WI, wj = wave / WI;

    // Workgroup -> tile.  Consecutive workgroup ids go round-robin over the 8
    // XCDs; give each XCD a contiguous run of tile ids so that workgroups that
    // share X row-panels and Y column-panels share one L2, then walk the tile
    // grid in groups of group_i tile-rows.
    int tile_id;
    {
        const int total = p.tiles_i * p.tiles_j;
        const int pid = blockIdx.x;
        const int per = total >> 3, rem = total & 7;
        const int xcd = pid & 7, loc = pid >> 3;
        tile_id = xcd < rem ? xcd * (per + 1) + loc : rem * (per + 1) + (xcd - rem) * per + loc;
    }
    int ti0, tj0;
    {
        const int gsz = p.group_i * p.tiles_j;
        const int gid = tile_id / gsz;
        const int first = gid * p.group_i;
        const int gi = min(p.tiles_i - first, p.group_i);
        const int in = tile_id - gid * gsz;
        ti0 = first + in % gi;
        tj0 = in / gi;
    }
    const long bt = blockIdx.y;
    // the last tile of a row or column is shifted back so that it ends at the edge (see tiled_params)
    const int i0 = min(ti0 * BI, p.I - BI), j0 = min(tj0 * BJ, p.J - BJ);

    const half_t *X = p.X + bt * p.sx + (XK ? (long)i0 * p.ldx : (long)i0);
    const half_t *Y = p.Y + bt * p.sy + (YK ? (long)j0 * p.ldy : (long)j0);
    const unsigned xoff = xload::lane_offset(tid, (int)p.ldx);
    const unsigned yoff = yload::lane_offset(tid, (int)p.ldy);

    xreader xr;
    yreader yr;
    xr.init(wi * WTI, lane);
    yr.init(wj * WTJ, lane);

    const int q = lane >> 4, r = lane & 15;
    const int row = i0 + wi * WTI + 4 * q;  // + 16*ti
    const int col = j0 + wj * WTJ + r;      // + 16*tj
    const CT *C = (const CT *)p.C + bt * p.sc;
    DT *D = (DT *)p.D + bt * p.sd;

    float4_t acc[TI][TJ];
#pragma unroll
    for (int a = 0; a < TI; a++)
#pragma unroll
        for (int b = 0; b < TJ; b++) acc[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};

    // C in the accumulator layout: 4 consecutive i of one column j per lane.
    // `trans` (C stored with j contiguous) is uniform over the grid.
    auto read_c = [&](int a, int b, bool trans) -> float4_t {
        float4_t c;
        const int ii = row + 16 * a, jj = col + 16 * b;
        if (trans) {
#pragma unroll
            for (int v = 0; v < 4; v++) c[v] = (float)C[(long)(ii + v) * p.ldc + jj];
        } else if constexpr (__is_same(CT, float)) {
            c = *(const float4_t *)(C + (long)jj * p.ldc + ii);
        } else {
            half4_t h = *(const half4_t *)(C + (long)jj * p.ldc + ii);
            c = float4_t{(float)h[0], (float)h[1], (float)h[2], (float)h[3]};
        }
        return c;
    };

    if constexpr (F16ACC) {
        // acc = half(beta * C): the Float16 accumulator starts as the C operand.
        if (p.use_c) {
            auto init = [&](bool trans) {
#pragma unroll
                for (int a = 0; a < TI; a++)
#pragma unroll
                    for (int b = 0; b < TJ; b++) {
                        float4_t c = read_c(a, b, trans);
#pragma unroll
                        for (int v = 0; v < 4; v++) acc[a][b][v] = round_through_half(p.beta * c[v]);
                    }
            };
            if (p.c_trans) init(true);
            else init(false);
            // these were ordinary loads: drain them before the hand-counted ones start
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        }
    }

    const int NP = (p.K + KGRAN - 1) / KGRAN;  // slots' worth of K ("pairs" of steps)
    // K tail: the last pair starts at K - 64; tail_skip of its k-values repeat the pair before
    const int tail_skip = NP * KGRAN - p.K;
    const unsigned wave_dst = (unsigned)(uintptr_t)lds + (unsigned)wave * 1024u;
    constexpr int NLX = xload::NLOAD, NLY = yload::NLOAD, LPAIR = NLX + NLY;  // loads per thread and pair
    int next = 0;          // next pair to request
    int wslot = 0;         // the slot it goes to
    unsigned dma_dst = 0;  // this wavefront's first destination byte in that slot
    auto begin_request = [&]() { dma_dst = wave_dst + (unsigned)(wslot * SLOT); };
    // Load number I of the pair being requested.
    auto request_one = [&]<int I>(std::integral_constant<int, I>) {
        if constexpr (I < NLX)
            lds_dma16(X + xload::load_delta(I, p.ldx), xoff, dma_dst + (unsigned)(I * NT * 16));
        else
            lds_dma16(Y + yload::load_delta(I - NLX, p.ldy), yoff, dma_dst + XBYTES + (unsigned)((I - NLX) * NT * 16));
    };
    // Past the end of K the last pair is requested again, into a slot nobody
    // reads any more: the pipeline stays free of branches.
    auto end_request = [&]() {
        next++;
        wslot = wslot + 1 == NSLOT ? 0 : wslot + 1;
        const int kstep = next < NP - 1 ? KGRAN : next == NP - 1 ? KGRAN - tail_skip : 0;
        // (64 leading dimensions fit in 32 bits: the host checks that 256 do)
        X += XK ? kstep : kstep * (int)p.ldx;
        Y += YK ? kstep : kstep * (int)p.ldy;
    };
    auto request_pair = [&]() {
        begin_request();
        [&]<int... I>(std::integer_sequence<int, I...>) { (request_one(std::integral_constant<int, I>{}), ...); }
        (std::make_integer_sequence<int, LPAIR>{});
        end_request();
    };

    frag_set<TI, TJ> f0, f1;
    // Fragment unit U of a step: the TI x-fragments, then the TJ y-fragments.
    auto fetch_unit = [&]<int U, int H>(frag_set<TI, TJ> &f, MIW_LDS const char *xs, std::integral_constant<int, U>,
                                        std::integral_constant<int, H>) {
        if constexpr (U < TI) f.x[U] = xr.template read<U, H>(xs);
        else f.y[U - TI] = yr.template read<U - TI, H>(xs + XBYTES);
    };
    constexpr int NUNIT = TI + TJ;
    // Zeroes the repeated k-values in the fragments of half H of the shifted last pair.
    auto mask_tail = [&]<int H>(frag_set<TI, TJ> &f, std::integral_constant<int, H>) {
        const unsigned keep = tail_keep<H>(tail_skip);
#pragma unroll
        for (int a = 0; a < TI; a++) tail_apply(f.x[a], keep);
#pragma unroll
        for (int b = 0; b < TJ; b++) tail_apply(f.y[b], keep);
    };
    // One pipeline step, in source order and pinned there: before MFMA m the
    // fragment unit m of the next step is fetched from LDS (all of them early
    // in the step, so they have landed long before it ends); the
    // direct-to-LDS loads DMA_LO..DMA_HI-1 of the pair being requested are
    // issued at even distances over the step, in the shadow of the matrix cores.
    // fp16 accumulate: the tile an MFMA of the pair's second step has just
    // finished is rounded to Float16 two MFMAs later, in the shadow of the
    // matrix cores, instead of all tiles at once after the step.
    constexpr int ROUND_LAG = 2;
    auto round_tile = [&](int m) {
        const int a = m / TJ, b = m % TJ;
        half4_t h = __builtin_convertvector(acc[a][b], half4_t);
        acc[a][b] = __builtin_convertvector(h, float4_t);
    };
    auto step = [&]<int H, int DMA_LO, int DMA_HI>(const frag_set<TI, TJ> &cur, frag_set<TI, TJ> &nxt, int slot,
                                                   std::integral_constant<int, H> h, std::integral_constant<int, DMA_LO>,
                                                   std::integral_constant<int, DMA_HI>) {
        constexpr bool ROUND = F16ACC && H == 0;  // the step that fetches a first half is the pair's second step
        MIW_LDS const char *xs = lds + slot * SLOT;
        constexpr int NDMA = DMA_HI - DMA_LO;
        constexpr int DMA_INSIDE = NDMA < NMFMA ? NDMA : NMFMA;  // issued between MFMAs; the rest after the last
        [&]<int... Mi>(std::integer_sequence<int, Mi...>) {
            (([&] {
                 constexpr int m = Mi;
                 // The SIMD issues from its oldest ready wavefront first, which lets one of its two
                 // wavefronts run a whole step ahead and then stand at the barrier while the other
                 // works alone; raising the priority over the first half of every step makes the
                 // two take turns.
                 if constexpr (NMFMA >= 8 && m == 0) __builtin_amdgcn_s_setprio(1);
                 if constexpr (NMFMA >= 8 && m == NMFMA / 2) __builtin_amdgcn_s_setprio(0);
                 if constexpr (m < NUNIT && !(MIW_PP_ABLATE & 2)) fetch_unit(nxt, xs, std::integral_constant<int, m>{}, h);
                 constexpr int a = m / TJ, b = m % TJ;
                 if constexpr (!(MIW_PP_ABLATE & 4)) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(cur.x[a], cur.y[b], acc[a][b], 0, 0, 0);
                 constexpr int d = dma_after_mfma(m, NMFMA, NDMA);
                 if constexpr (d >= 0 && !(MIW_PP_ABLATE & 1)) {
                     __builtin_amdgcn_sched_barrier(0);
                     request_one(std::integral_constant<int, DMA_LO + d>{});
                 }
                 if constexpr (ROUND && m >= ROUND_LAG) round_tile(m - ROUND_LAG);
                 __builtin_amdgcn_sched_barrier(0);
             }()),
             ...);
        }(std::make_integer_sequence<int, NMFMA>{});
        if constexpr (ROUND)
#pragma unroll
            for (int m = NMFMA > ROUND_LAG ? NMFMA - ROUND_LAG : 0; m < NMFMA; m++) round_tile(m);
        // tiles with fewer MFMAs than fragment units or loads: the rest follows the last MFMA
        if constexpr (NUNIT > NMFMA)
            [&]<int... U>(std::integer_sequence<int, U...>) {
                (fetch_unit(nxt, xs, std::integral_constant<int, NMFMA + U>{}, h), ...);
            }(std::make_integer_sequence<int, NUNIT - NMFMA>{});
        if constexpr (NDMA > DMA_INSIDE)
            [&]<int... I>(std::integer_sequence<int, I...>) {
                (request_one(std::integral_constant<int, DMA_LO + DMA_INSIDE + I>{}), ...);
            }(std::make_integer_sequence<int, NDMA - DMA_INSIDE>{});
    };
    constexpr std::integral_constant<int, 0> first_half{};
    constexpr std::integral_constant<int, 1> second_half{};
    constexpr std::integral_constant<int, 0> dma_begin{};
    constexpr std::integral_constant<int, LPAIR> dma_end{};

    // Prologue: every slot requested, pair 0 published and its first fragments fetched.
#pragma unroll
    for (int s = 0; s < NSLOT; s++) request_pair();
    wait_loads_and_barrier<(NSLOT - 1) * LPAIR>();
    [&]<int... U>(std::integer_sequence<int, U...>) {
        (fetch_unit(f0, lds, std::integral_constant<int, U>{}, first_half), ...);
    }(std::make_integer_sequence<int, NUNIT>{});
    if constexpr (MIW_PP_ABLATE & 2) f1 = f0;

    // Folding C.  With alpha == 1 the C operand is added into the accumulators
    // during the last NCT trips of the loop, CPT MFMA tiles per trip, so that
    // the memory system delivers C while the matrix cores run and the epilogue
    // only stores.  Group g (tiles g*CPT..) is requested at the end of a trip
    // with direct-to-LDS loads: lane l fetches the 16 bytes it will own, so the
    // wavefront's staging buffer is read back lane-contiguously by the same
    // wavefront and needs no barrier of its own.  These loads are the youngest
    // when the next trip waits, which lets exactly them stay in flight; the
    // wait of the trip after that covers them (they are older than everything
    // it leaves in flight), and that trip adds the group in: C has two trips to
    // arrive from HBM.  Two staging buffers alternate.  Tiles are taken in the
    // order of their addresses: 16 rows (64 bytes, the instruction's offset
    // field) further down a column block, then the next 16 columns.  The
    // accumulators are registers, so the folding trips are unrolled.
    constexpr int CPT = fold_tiles(BI, BJ, NT, NSLOT);
    constexpr bool CAN_FOLD = !F16ACC && __is_same(CT, float) && CPT > 0;
    constexpr int NTILE = TI * TJ;
    constexpr int NCT = CAN_FOLD ? NTILE / CPT : 1;  // groups, and trips that fold
    static_assert(!CAN_FOLD || (TI % CPT == 0 && NCT >= 2), "fold groups");
    bool fold_c = false;
    // (the lane offset into the tile of C is kept in 32 bits)
    if constexpr (CAN_FOLD) fold_c = p.use_c && !p.c_trans && p.alpha == 1.0f && NP > NCT && p.ldc < (1l << 22);
    const unsigned cstage = (unsigned)(uintptr_t)lds + (unsigned)(NSLOT * SLOT) + (unsigned)wave * (2u * CPT * 1024u);
    const char *cnext = (const char *)(C + (long)j0 * p.ldc + i0);
    const unsigned coff = 4u * (unsigned)((wj * WTJ + r) * (int)p.ldc + wi * WTI + 4 * q);
    auto fold_request = [&]<int G>(std::integral_constant<int, G>) {
        [&]<int... U>(std::integer_sequence<int, U...>) {
            (([&] {
                 constexpr int a = (G * CPT + U) % TI;
                 lds_dma16_imm<64 * a>(cnext, coff, cstage + (unsigned)(((G & 1) * CPT + U) * 1024));
                 if constexpr (a == TI - 1) cnext += 64 * p.ldc;
             }()),
             ...);
        }(std::make_integer_sequence<int, CPT>{});
    };
    float4_t cfold[CPT > 0 ? CPT : 1];
    auto fold_fetch = [&]<int G>(std::integral_constant<int, G>) {
#pragma unroll
        for (int u = 0; u < CPT; u++)
            cfold[u] = *(MIW_LDS const float4_t *)(lds + NSLOT * SLOT + wave * (2 * CPT * 1024) +
                                                   ((G & 1) * CPT + u) * 1024 + lane * 16);
    };
    auto fold_add = [&]<int G>(std::integral_constant<int, G>) {
#pragma unroll
        for (int u = 0; u < CPT; u++) {
            const int a = (G * CPT + u) % TI, b = (G * CPT + u) / TI;
#pragma unroll
            for (int e = 0; e < 4; e++) acc[a][b][e] = __builtin_fmaf(p.beta, cfold[u][e], acc[a][b][e]);
        }
    };

    // Trip pr: step 2pr (second half of pair pr's slot is fetched; nothing to
    // request yet: the slot is still being read), barrier (pair pr+1 has
    // landed, pair pr's slot is free), step 2pr+1 (first half of pair pr+1 is
    // fetched while pair pr+NSLOT is requested into the freed slot; NSLOT-2
    // younger pairs stay in flight across the barrier).  On the last trip
    // nothing new lands; its odd step reads another slot's stale bytes into
    // registers nobody uses.
    int rslot = 0;
    // MASK 1: the trip before the last pair's (its second step fetches the first half of the last pair);
    // MASK 2: the last pair's own trip (its first step fetches the second half).
    // G >= 0: the trip folds group G of C.  RT: whether it does is decided at run time (fold_c): the two
    // trips that meet the last pair are one piece of code for launches that fold and launches that do
    // not (two alternative pieces that each update all accumulators cost spills where they join).
    auto trip = [&]<int MASK, int G, bool RT>(std::integral_constant<int, MASK>, std::integral_constant<int, G>, std::bool_constant<RT>) {
        step(f0, f1, rslot, second_half, dma_begin, dma_begin);
        if constexpr (MASK == 2) mask_tail(f1, second_half);
        if constexpr (G >= 0) {
            if (!RT || fold_c) wait_loads_and_barrier<(NSLOT - 2) * LPAIR + (G > 0 ? CPT : 0)>();
            else wait_loads_and_barrier<(NSLOT - 2) * LPAIR>();
        } else {
            wait_loads_and_barrier<(NSLOT - 2) * LPAIR>();
        }
        rslot = rslot + 1 == NSLOT ? 0 : rslot + 1;
        if constexpr (G > 1)
            if (!RT || fold_c) fold_fetch(std::integral_constant<int, G - 2>{});
        __builtin_amdgcn_sched_barrier(0);
        begin_request();
        step(f1, f0, rslot, first_half, dma_begin, dma_end);
        if constexpr (MASK == 1) mask_tail(f0, first_half);
        end_request();
        if constexpr (G > 1)
            if (!RT || fold_c) fold_add(std::integral_constant<int, G - 2>{});
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (G >= 0)
            if (!RT || fold_c) fold_request(std::integral_constant<int, G>{});
        __builtin_amdgcn_sched_barrier(0);
    };
    constexpr std::integral_constant<int, -1> no_group{};
    // the loop runs the trips that neither fold nor meet the last pair
    const int NPM = fold_c ? NP - NCT : NP >= 2 ? NP - 2 : 0;
    for (int pr = 0; pr < NPM; pr++) trip(std::integral_constant<int, 0>{}, no_group, std::false_type{});
    if constexpr (CAN_FOLD) {
        if (fold_c) {
            [&]<int... G>(std::integer_sequence<int, G...>) {
                (trip(std::integral_constant<int, 0>{}, std::integral_constant<int, G>{}, std::false_type{}), ...);
            }(std::make_integer_sequence<int, NCT - 2>{});
        }
        if (NP >= 2) trip(std::integral_constant<int, 1>{}, std::integral_constant<int, NCT - 2>{}, std::true_type{});
        trip(std::integral_constant<int, 2>{}, std::integral_constant<int, NCT - 1>{}, std::true_type{});
    } else {
        if (NP >= 2) trip(std::integral_constant<int, 1>{}, no_group, std::false_type{});
        trip(std::integral_constant<int, 2>{}, no_group, std::false_type{});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may outlive the workgroup's LDS
    if constexpr (CAN_FOLD) {
        if (fold_c) {
            fold_fetch(std::integral_constant<int, NCT - 2>{});
            fold_add(std::integral_constant<int, NCT - 2>{});
            fold_fetch(std::integral_constant<int, NCT - 1>{});
            fold_add(std::integral_constant<int, NCT - 1>{});
        }
    }

    // Epilogue: each lane owns 4 consecutive i of one column j per MFMA tile.
    static_assert(TI % 2 == 0, "the epilogue stores pairs of tiles");
    auto epilogue = [&](bool with_c, bool trans) {
        auto value = [&](int a, int b) {
            float4_t v = acc[a][b];
            if constexpr (!F16ACC) {
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] *= p.alpha;
                if (with_c) {
                    float4_t c = read_c(a, b, trans);
#pragma unroll
                    for (int e = 0; e < 4; e++) v[e] = __builtin_fmaf(p.beta, c[e], v[e]);
                }
            }
            return v;
        };
#pragma unroll
        for (int b = 0; b < TJ; b++)
#pragma unroll
            for (int a = 0; a < TI; a += 2)
                store_tile_pair<DT>(D, p.ldd, i0 + wi * WTI + 16 * a, j0 + wj * WTJ + 16 * b, lane, value(a, b), value(a + 1, b));
    };
    if (F16ACC || !p.use_c || fold_c) epilogue(false, false);
    else if (p.c_trans) epilogue(true, true);
    else epilogue(true, false);
}

// ------------------------------------------------- kernel instance lookup --

template <int BI, int BJ, int WI, int WJ, int NS, class CT, class DT, bool F16ACC>
inline const void *pick_layout(bool xk, bool yk)
{
    if (xk && yk) return (const void *)k_gemm_tiled<BI, BJ, WI, WJ, NS, true, true, CT, DT, F16ACC>;
    if (xk && !yk) return (const void *)k_gemm_tiled<BI, BJ, WI, WJ, NS, true, false, CT, DT, F16ACC>;
    if (!xk && yk) return (const void *)k_gemm_tiled<BI, BJ, WI, WJ, NS, false, true, CT, DT, F16ACC>;
    return (const void *)k_gemm_tiled<BI, BJ, WI, WJ, NS, false, false, CT, DT, F16ACC>;
}

template <int BI, int BJ, int WI, int WJ, int NS>
inline const void *pick_types(bool xk, bool yk, int c_type, int d_type, bool f16acc)
{
    if (f16acc) {
        // the rounding runs on the VALU: it needs the accumulators in ordinary VGPRs
        if constexpr (waves_per_simd(BI, BJ, WI * WJ * 64) < 2) return nullptr;
        else return pick_layout<BI, BJ, WI, WJ, NS, half_t, half_t, true>(xk, yk);
    }
    if (c_type == 0 && d_type == 0) return pick_layout<BI, BJ, WI, WJ, NS, half_t, half_t, false>(xk, yk);
    if (c_type == 0 && d_type == 1) return pick_layout<BI, BJ, WI, WJ, NS, half_t, float, false>(xk, yk);
    if (c_type == 1 && d_type == 0) return pick_layout<BI, BJ, WI, WJ, NS, float, half_t, false>(xk, yk);
    return pick_layout<BI, BJ, WI, WJ, NS, float, float, false>(xk, yk);
}

}  // namespace miw

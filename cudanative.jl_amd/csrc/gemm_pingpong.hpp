// Ping-pong form of the LDS-tiled GEMM for gfx950 (fp32 accumulation): the two
// wavefronts that share a SIMD take turns.  While one of them issues nothing
// but the 32 MFMAs of a k-step (a "compute cluster", 512 cycles of matrix-core
// time), the other one runs its "memory cluster": it reads its fragments of the
// next k-step from LDS into registers and issues its share of the direct-to-LDS
// loads that refill the ring.  A workgroup barrier ends every cluster and the
// two swap roles.  The matrix cores never wait for an LDS read or for the issue
// of a load (a wavefront alone on its SIMD loses 15-20 cycles of MFMA issue per
// 1 KiB load it issues), and the two wavefronts never compete for them.
//
// Wavefronts 0-3 of the workgroup sit on SIMDs 0-3 and wavefronts 4-7 join
// them in the same order; the second group enters the loop one barrier late, so
// that it runs one cluster behind the first for the whole K loop.
//
// Same canonical problem, tile mapping and LDS chunk layouts as gemm_tiled.hpp
// (P = X * Y, I contiguous in P).  What differs is how the ring is cut:
//   I-major operand: four entries of 32 k-values (one k-step).  The loads of
//       step t+3 are issued in the memory cluster of step t.
//   K-major operand: three slots of 64 k-values (rows of 128 bytes, so that
//       every direct-to-LDS load still fetches full 128-byte lines).  The loads
//       of pair p+2 are issued in the two memory clusters of pair p, half each.
// Either way a wavefront waits, at the end of memory cluster t, for the loads
// it issued in cluster t-2 and earlier (s_waitcnt vmcnt(2 * loads per cluster)):
// a load has two full clusters of both groups (about 2000 cycles) to land
// before anyone waits for it, and the barriers between that wait and the first
// read publish it to the other wavefronts.
//   Two K-major operands: three slots each would be 192 KiB.  X keeps three, Y
//       gets two (160 KiB).  A slot of Y is free once both groups have read its
//       second k-step, which is when group 0 starts the memory cluster after
//       that; so the first cluster of pair p+1 requests all of Y's pair p+2
//       into the slot of pair p, and the wait at the end of the second cluster
//       of pair p+1 must cover it: that cluster leaves only its own loads in
//       flight, and those are X's (all of X's pair p+3, into the slot of pair
//       p).  Y's loads have one compute and one memory cluster to land, X's two
//       of each as before.
#pragma once
#include "gemm_tiled.hpp"

namespace miw {

// (The measurement switch MIW_PP_ABLATE of gemm_tiled.hpp applies to the loops of these kernels too.)


// Second measurement switch (off in every shipped build; gemm_kernels.hip must be compiled with it
// too): with MIW_PP_TS the ping-pong kernels record, per wavefront, the shader clock at kernel
// entry [0], after the prologue's loads have landed [1], at the middle of the loop [2], one pair
// of k-steps later [3], at the end of the pairs that do not fold C [9], at the end of the loop [4],
// when the last store is issued [5] and when the stores have drained [6], plus the 100 MHz wall
// clock at exit [7] and entry [8], into the buffer whose device address the environment variable
// MIW_TS holds (cudanative.jl_amd/timestamps.py sets it and prints the phases).
#ifdef MIW_PP_TS
#define MIW_PP_STAMP(i) { __builtin_amdgcn_sched_barrier(0); ts[i] = clock64(); __builtin_amdgcn_sched_barrier(0); }
// (in the unrolled part of the loop: the ring of pairs that holds pair NPM / 2 stamps its first pair)
#define MIW_PP_MIDDLE(pr) { stamp_pair = (pr) <= NPM / 2 && NPM / 2 < (pr) + NSLOT; if (stamp_pair) MIW_PP_STAMP(2) }
#else
#define MIW_PP_STAMP(i)
#define MIW_PP_MIDDLE(pr)
#endif

constexpr int PP_KMAJOR_SLOTS = 3;
constexpr int PP_IMAJOR_ENTRIES = 4;

// Slots of a K-major Y: two when X is K-major as well (see above), else three.
constexpr int pp_y_slots(bool xk) { return xk ? 2 : PP_KMAJOR_SLOTS; }
constexpr int pp_operand_bytes(int rows, bool kmajor, int kslots)
{
    return kmajor ? kslots * rows * KGRAN * 2 : PP_IMAJOR_ENTRIES * rows * BKS * 2;
}
constexpr int pp_lds_bytes(int bi, int bj, bool xk, bool yk)
{
    return pp_operand_bytes(bi, xk, PP_KMAJOR_SLOTS) + pp_operand_bytes(bj, yk, pp_y_slots(xk));
}
constexpr bool pp_fits(int bi, int bj, bool xk, bool yk) { return pp_lds_bytes(bi, bj, xk, yk) <= 160 * 1024; }

// One operand of the ping-pong kernel: its ring in LDS, the loads that fill it
// and the fragment reads.  R rows (or columns) of the tile, NT threads.
template <int R, bool KMAJOR, int NT, int KSLOTS = PP_KMAJOR_SLOTS>
struct pp_operand {
    // loads per thread: per 64-k slot (K-major) or per 32-k entry (I-major)
    static constexpr int NL = KMAJOR ? R * KGRAN / 8 / NT : R * BKS / 8 / NT;
    // loads per thread and memory cluster (a K-major operand: half a slot, unless both operands are K-major)
    static constexpr int PER_CLUSTER = KMAJOR ? NL / 2 : NL;
    static constexpr int UNIT_BYTES = KMAJOR ? R * KGRAN * 2 : R * BKS * 2;
    static constexpr int UNITS = KMAJOR ? KSLOTS : PP_IMAJOR_ENTRIES;
    static constexpr int BYTES = UNITS * UNIT_BYTES;
    static_assert(NL >= 1 && (!KMAJOR || NL % 2 == 0), "operand must divide over the workgroup");
    static_assert(NT == 512 || NT == 256, "lane offsets below assume 256 or 512 threads");

    __device__ static inline unsigned lane_offset(int tid, int ld)
    {
        if constexpr (KMAJOR) {
            return slot_loader<R, true, NT>::lane_offset(tid, ld);
        } else {
            // chunk tid of the entry: i-block tid / 256, k-row (tid / 8) % 32, chunk position tid % 8
            const int k = (tid >> 3) & 31, cpos = tid & 7, iblk = tid >> 8;
            const int c = cpos ^ (2 * i_major_swizzle(k));
            return 2u * (unsigned)(k * ld + iblk * 64 + c * 8);
        }
    }
    // Element offset of load i of a unit relative to load 0 (uniform).
    __device__ static inline long load_delta(int i, long ld)
    {
        if constexpr (KMAJOR) return (long)i * (NT / 8) * ld;
        else return (long)i * (NT / 256) * 64;
    }

    // Fragment reads.  K-major: the reader of gemm_tiled.hpp on a 64-k slot.
    // I-major: the same transpose reads on an entry of 32 k-rows (i-blocks of
    // 64 i are 4 KiB apart instead of 8).
    frag_reader<R, true> kr;
    int ibase[4];
    __device__ inline void init(int wave_row0, int lane)
    {
        if constexpr (KMAJOR) {
            kr.init(wave_row0, lane);
        } else {
            const int j = lane & 15, q = lane >> 4;
            const int jq = j >> 2, jr = j & 3;
            const int g = ((jq >> 1) & 1) | ((q & 1) << 1);
            const int w16 = wave_row0 / 16;
#pragma unroll
            for (int m = 0; m < 4; m++)
                ibase[m] = (w16 / 4) * 4096 + (8 * q + jq) * 128 + jr * 8 + ((((w16 & 3) + m) & 3) ^ g) * 32;
        }
    }
    // Fragment T of k-step H (0/1: which half of the slot; ignored for I-major) out of the unit at `unit`.
    template <int T, int H>
    __device__ inline half8_t read(MIW_LDS const char *unit) const
    {
        if constexpr (KMAJOR) {
            return kr.template read<T, H>(unit);
        } else {
            const int off = ibase[T & 3] + (T >> 2) * 4096;
            fp16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4f16((MIW_LDS fp16x4_t *)(unit + off));
            fp16x4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4f16((MIW_LDS fp16x4_t *)(unit + off + 512));
            uint2_t l2 = __builtin_bit_cast(uint2_t, lo), h2 = __builtin_bit_cast(uint2_t, hi);
            uint4_t v = {l2[0], l2[1], h2[0], h2[1]};
            return __builtin_bit_cast(half8_t, v);
        }
    }
};

template <int BI, int BJ, int WI, int WJ, bool XK, bool YK, class CT, class DT>
__global__ __launch_bounds__(WI *WJ * 64) __attribute__((amdgpu_waves_per_eu(2)))
void k_gemm_pp(tiled_params p)
{
    constexpr int NT = WI * WJ * 64;
    static_assert(NT == 512, "two wavefronts per SIMD");
    constexpr int WTI = BI / WI, WTJ = BJ / WJ;
    constexpr int TI = WTI / 16, TJ = WTJ / 16;
    constexpr bool KK = XK && YK;  // two K-major operands: Y has two slots, clusters alternate between Y's loads and X's
    using xop = pp_operand<BI, XK, NT>;
    using yop = pp_operand<BJ, YK, NT, pp_y_slots(XK)>;
    constexpr int XB = xop::BYTES;
    constexpr int ND = xop::PER_CLUSTER + yop::PER_CLUSTER;  // loads per thread and memory cluster
    static_assert(!KK || (xop::NL == ND && yop::NL == ND), "alternating clusters carry equal loads");
    static_assert(pp_fits(BI, BJ, XK, YK), "ring does not fit in LDS");

#ifdef MIW_PP_TS
    long long ts[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    ts[0] = clock64();
    ts[8] = wall_clock64();
#endif
    extern __shared__ __attribute__((aligned(128))) char smem[];
    MIW_LDS char *lds = (MIW_LDS char *)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wi = wave % WI, wj = wave / WI;
    const bool late_group = wave >= 4;

    // Workgroup -> tile, as in k_gemm_tiled.
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
    const unsigned xoff = xop::lane_offset(tid, (int)p.ldx);
    const unsigned yoff = yop::lane_offset(tid, (int)p.ldy);

    xop xr;
    yop yr;
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

    const int NP = (p.K + KGRAN - 1) / KGRAN;  // pairs of k-steps
    const int NS = 2 * NP;                     // k-steps
    // K tail: the last pair starts at K - 64; tail_skip of its k-values repeat the pair before
    const int tail_skip = NP * KGRAN - p.K;
    const unsigned lds0 = (unsigned)(uintptr_t)lds;
    const unsigned wave_dst = lds0 + (unsigned)wave * 1024u;

    // ---- ring state (uniform).  I-major operand: the pair's two entries sit at `pair` and
    // pair + UNIT_BYTES, pair toggling between 0 and 2 UNIT_BYTES.  K-major operand: `pair` is the
    // slot of the current pair and `prev` the slot of the pair before it, which is the one being
    // refilled (with pair pr + 2).
    unsigned xpair = 0, xprev = 2 * xop::UNIT_BYTES, ypair = 0, yprev = (yop::UNITS - 1) * yop::UNIT_BYTES;
    int xnext = 0, ynext = 0;  // next unit to request (step index for I-major, pair index for K-major)
    // Lane offsets of the loads of one unit: K-major loads differ by whole rows (a per-load lane
    // offset keeps one uniform base address), I-major loads by 256 bytes (the instruction's offset field).
    unsigned xvo[XK ? xop::NL : 1], yvo[YK ? yop::NL : 1];
#pragma unroll
    for (int i = 0; i < (XK ? xop::NL : 1); i++) xvo[i] = xoff + 2u * (unsigned)xop::load_delta(i, p.ldx);
#pragma unroll
    for (int i = 0; i < (YK ? yop::NL : 1); i++) yvo[i] = yoff + 2u * (unsigned)yop::load_delta(i, p.ldy);
    // Load I of the unit at ring offset `unit` (bytes from the operand's region).
    auto x_load = [&]<int I>(unsigned unit, std::integral_constant<int, I>) {
        if constexpr (XK) lds_dma16_at<I * NT * 16, 0>(X, xvo[I], wave_dst + unit);
        else lds_dma16_at<I * NT * 16, I * 256>(X, xvo[0], wave_dst + unit);
    };
    auto y_load = [&]<int I>(unsigned unit, std::integral_constant<int, I>) {
        if constexpr (YK) lds_dma16_at<XB + I * NT * 16, 0>(Y, yvo[I], wave_dst + unit);
        else lds_dma16_at<XB + I * NT * 16, I * 256>(Y, yvo[0], wave_dst + unit);
    };
    // Past the end of K the last unit is requested again, into a unit nobody reads any more.
    // Elements from one unit to the next; the first unit of the last pair (pair NP - 1, or entry NS - 2)
    // lies tail_skip k-values short of where it would follow on (a step back for an entry of 32 when 48
    // repeat).  Both steps are kept as 64-bit values: computed per request, the multiplication by the
    // leading dimension is a chain of scalar instructions at the end of every memory cluster, which is
    // the longer of the two clusters.
    constexpr int XUK = XK ? KGRAN : BKS, YUK = YK ? KGRAN : BKS;
    const long xunit = XK ? (long)XUK : (long)XUK * p.ldx, xtail = XK ? (long)(XUK - tail_skip) : (long)(XUK - tail_skip) * p.ldx;
    const long yunit = YK ? (long)YUK : (long)YUK * p.ldy, ytail = YK ? (long)(YUK - tail_skip) : (long)(YUK - tail_skip) * p.ldy;
    auto x_advance = [&]() {
        xnext++;
        X += xnext == (XK ? NP - 1 : NS - 2) ? xtail : xnext < (XK ? NP : NS) ? xunit : 0;
    };
    auto y_advance = [&]() {
        ynext++;
        Y += ynext == (YK ? NP - 1 : NS - 2) ? ytail : ynext < (YK ? NP : NS) ? yunit : 0;
    };
    // Request number N (0 .. ND-1) of the memory cluster of k-step 2 pr + H: the X loads, then the Y loads.
    auto cluster_request = [&]<int H, int N>(std::integral_constant<int, H>, std::integral_constant<int, N>) {
        if constexpr (KK) {
            // first cluster of a pair: all of Y's pair after next, into the slot of the pair before
            // (read to the end one barrier ago); second cluster: all of X's, likewise
            if constexpr (H == 0) y_load(yprev, std::integral_constant<int, N>{});
            else x_load(xprev, std::integral_constant<int, N>{});
        } else if constexpr (N < xop::PER_CLUSTER) {
            if constexpr (XK) x_load(xprev, std::integral_constant<int, H * xop::NL / 2 + N>{});
            else x_load(H == 0 ? (xpair ^ (2u * xop::UNIT_BYTES)) + xop::UNIT_BYTES : xpair, std::integral_constant<int, N>{});
        } else {
            constexpr int M = N - xop::PER_CLUSTER;
            if constexpr (YK) y_load(yprev, std::integral_constant<int, H * yop::NL / 2 + M>{});
            else y_load(H == 0 ? (ypair ^ (2u * yop::UNIT_BYTES)) + yop::UNIT_BYTES : ypair, std::integral_constant<int, M>{});
        }
    };
    auto cluster_advance = [&]<int H>(std::integral_constant<int, H>) {
        if constexpr (!XK || H == 1) x_advance();
        if constexpr (!YK || H == (KK ? 0 : 1)) y_advance();
    };
    auto pair_advance = [&]() {
        if constexpr (XK) {
            xprev = xpair;
            xpair = xpair + xop::UNIT_BYTES == xop::BYTES ? 0 : xpair + xop::UNIT_BYTES;
        } else {
            xpair ^= 2u * xop::UNIT_BYTES;
        }
        if constexpr (YK) {
            yprev = ypair;
            ypair = ypair + yop::UNIT_BYTES == yop::BYTES ? 0 : ypair + yop::UNIT_BYTES;
        } else {
            ypair ^= 2u * yop::UNIT_BYTES;
        }
    };

    // Prologue: K-major operands request pairs 0 and 1, I-major operands steps 0, 1 and 2, in the order
    // in which the loop needs them: what step 0 reads (unit 0 of each operand), then step 1 (entry 1 of
    // an I-major operand), then step 2 (entry 2, pair 1).  The loop starts as soon as the units of step
    // 0 have landed; the rest arrives under the first clusters.  The loop's own wait covers it: at the
    // end of memory cluster t it leaves 2 ND loads in flight, and the units of step 2 are at least ND
    // loads, so after cluster 0 the units of step 1 have landed and after cluster 1 those of step 2.
    auto prologue_unit = [&]<int U>(std::integral_constant<int, U>, bool is_x) {
        if (is_x) {
            [&]<int... I>(std::integer_sequence<int, I...>) {
                (x_load((unsigned)(U * xop::UNIT_BYTES), std::integral_constant<int, I>{}), ...);
            }(std::make_integer_sequence<int, xop::NL>{});
            x_advance();
        } else {
            [&]<int... I>(std::integer_sequence<int, I...>) {
                (y_load((unsigned)(U * yop::UNIT_BYTES), std::integral_constant<int, I>{}), ...);
            }(std::make_integer_sequence<int, yop::NL>{});
            y_advance();
        }
    };
    constexpr std::integral_constant<int, 0> unit0{};
    constexpr std::integral_constant<int, 1> unit1{};
    constexpr std::integral_constant<int, 2> unit2{};
    prologue_unit(unit0, true);
    prologue_unit(unit0, false);
    if constexpr (!XK) prologue_unit(unit1, true);
    if constexpr (!YK) prologue_unit(unit1, false);
    if constexpr (XK) prologue_unit(unit1, true);
    else prologue_unit(unit2, true);
    if constexpr (!YK) prologue_unit(unit2, false);
    else if constexpr (!KK) prologue_unit(unit1, false);  // (two K-major operands: cluster 0 requests Y's pair 1)
    constexpr int PROLOGUE_LOADS = (XK ? 2 : 3) * xop::NL + (KK ? 1 : YK ? 2 : 3) * yop::NL;
    static_assert(xop::NL + yop::NL >= ND, "the units of step 2 must cover one cluster's requests");
    wait_loads_and_barrier<PROLOGUE_LOADS - xop::NL - yop::NL>();

    half8_t fx[TI], fy[TJ];
    if constexpr (MIW_PP_ABLATE & 2) {
        [&]<int... U>(std::integer_sequence<int, U...>) { ((fx[U] = xr.template read<U, 0>(lds)), ...); }(std::make_integer_sequence<int, TI>{});
        [&]<int... U>(std::integer_sequence<int, U...>) { ((fy[U] = yr.template read<U, 0>(lds + XB)), ...); }(std::make_integer_sequence<int, TJ>{});
    }
    // Memory cluster of step 2 pr + H: the fragments of the step, with the cluster's requests
    // issued at even distances between the reads (the reads are bound by the LDS, which the four
    // wavefronts that are in their memory cluster share: a load issued between two of them costs
    // no extra time).
    constexpr int NFRAG = TI + TJ;
    // Fragment unit U of a step (the TI x-fragments, then the TJ y-fragments), preceded by the
    // requests that go out before it: request N before unit N * NFRAG / ND.
    auto cluster_unit = [&]<int H, int U>(MIW_LDS const char *xu, MIW_LDS const char *yu, std::integral_constant<int, H> h,
                                          std::integral_constant<int, U>) {
        [&]<int... N>(std::integer_sequence<int, N...>) {
            (([&] {
                 // (Y's loads of a two-K-major kernel have the least time to land: they go out first)
                 if constexpr ((KK && H == 0 ? N : N * NFRAG / ND) == U && !(MIW_PP_ABLATE & 1)) {
                     cluster_request(h, std::integral_constant<int, N>{});
                     __builtin_amdgcn_sched_barrier(0);
                 }
             }()),
             ...);
        }(std::make_integer_sequence<int, ND>{});
        if constexpr (MIW_PP_ABLATE & 2) {
            asm volatile("" : "+v"(fx[U % TI]), "+v"(fy[U % TJ]));
        } else {
            if constexpr (U < TI) fx[U] = xr.template read<U, H>(xu);
            else fy[U - TI] = yr.template read<U - TI, H>(yu);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    auto memory_cluster = [&]<int H>(std::integral_constant<int, H> h) {
        MIW_LDS const char *xu = lds + xpair + (XK ? 0 : H * xop::UNIT_BYTES);
        MIW_LDS const char *yu = lds + XB + ypair + (YK ? 0 : H * yop::UNIT_BYTES);
        [&]<int... U>(std::integer_sequence<int, U...>) {
            (cluster_unit(xu, yu, h, std::integral_constant<int, U>{}), ...);
        }(std::make_integer_sequence<int, NFRAG>{});
        // The ring state and the operand pointers move on here, behind the last fragment read and under its
        // latency.  (Measured: the same scalar instructions between the first MFMAs of the compute cluster
        // hold the matrix core up for 65 cycles per cluster; between the fragment reads, for 19.)
        cluster_advance(h);
        if constexpr (H == 1) pair_advance();
        __builtin_amdgcn_sched_barrier(0);
    };
    auto compute_cluster = [&]() {
        __builtin_amdgcn_sched_barrier(0);
        // serpentine order: every MFMA changes exactly one of its two operand fragments
#pragma unroll
        for (int a = 0; a < TI; a++)
#pragma unroll
            for (int bb = 0; bb < TJ; bb++) {
                const int b = serpentine_column(a * TJ + bb, TJ);
                if constexpr (!(MIW_PP_ABLATE & 4)) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fx[a], fy[b], acc[a][b], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
    };

    // Folding C.  With alpha == 1 the C operand is added into the accumulators during the last
    // NFOLD k-steps, CPT MFMA tiles per memory cluster, so that the memory system delivers C
    // while the matrix cores run and the epilogue only stores.  The tiles of fold step S are
    // requested at the end of the memory cluster with ordinary loads into registers (the lane
    // fetches the 16 bytes it owns); they are the youngest loads of their cluster, so the wait at
    // the end of the cluster two steps later covers them, and that cluster adds them in: C has
    // two clusters of both wavefront groups to arrive.  Three register stages rotate.  Tiles go in
    // the order of their addresses: 16 rows (64 bytes, the instruction's offset field) further
    // down a column block, then the next 16 columns.  The accumulators are registers, so the
    // folding steps are unrolled.
    constexpr int CPT = 1;
    constexpr int NTILE = TI * TJ;
    constexpr int NFOLD = NTILE / CPT;
    constexpr bool CAN_FOLD = __is_same(CT, float) && TI % CPT == 0 && NFOLD % 2 == 0;
    bool fold_c = false;
    // (the lane offset into the tile of C is kept in 32 bits)
    if constexpr (CAN_FOLD) fold_c = p.use_c && !p.c_trans && p.alpha == 1.0f && NS >= NFOLD + 2 && p.ldc < (1l << 22);
    float4_t cst[3][CPT];
    const char *cnext = (const char *)(C + (long)j0 * p.ldc + i0);
    const unsigned coff = 4u * (unsigned)((wj * WTJ + r) * (int)p.ldc + wi * WTI + 4 * q);
    auto fold_request = [&]<int S>(std::integral_constant<int, S>) {
        [&]<int... U>(std::integer_sequence<int, U...>) {
            (([&] {
                 constexpr int a = (S * CPT + U) % TI;
                 asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(cst[S % 3][U]) : "v"(coff), "s"(cnext), "n"(64 * a) : "memory");
                 if constexpr (a == TI - 1) cnext += 64 * p.ldc;
             }()),
             ...);
        }(std::make_integer_sequence<int, CPT>{});
    };
    auto fold_add = [&]<int S>(std::integral_constant<int, S>) {
#pragma unroll
        for (int u = 0; u < CPT; u++) {
            const int a = (S * CPT + u) % TI, b = (S * CPT + u) / TI;
#pragma unroll
            for (int e = 0; e < 4; e++) acc[a][b][e] = __builtin_fmaf(p.beta, cst[S % 3][u][e], acc[a][b][e]);
        }
    };
    // One k-step: memory cluster, barrier, compute cluster, barrier.  FS >= 0: fold step FS.
    // Zeroes the repeated k-values in the fragments of step H of the shifted last pair.
    auto mask_tail = [&]<int H>(std::integral_constant<int, H>) {
        const unsigned keep = tail_keep<H>(tail_skip);
#pragma unroll
        for (int a = 0; a < TI; a++) tail_apply(fx[a], keep);
#pragma unroll
        for (int b = 0; b < TJ; b++) tail_apply(fy[b], keep);
    };
    // FS >= 0: fold step FS (always folds).  FS == -1: a step that does not fold.  FS == -2: a step of
    // the last pair: its fragments are masked, and it is fold step NFOLD - 2 + H when the launch folds C,
    // which is decided here at run time, so that the last pair is one piece of code for both cases (two
    // alternative pieces that each update all accumulators cost spills where they join).
    auto fold_wait = [&]<int H, int FS>(std::integral_constant<int, H>, std::integral_constant<int, FS>) {
        // fold step FS issues ND + CPT loads; steps before the first fold step issue ND
        constexpr int YOUNGER = (KK && H == 1 ? ND : 2 * ND) + (FS >= 1 ? 2 : 1) * CPT;
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt((YOUNGER & 15) | (7 << 4) | (0 << 8) | ((YOUNGER >> 4) << 14));
        asm volatile("" ::: "memory");
    };
    auto step = [&]<int H, int FS>(std::integral_constant<int, H> h, std::integral_constant<int, FS>) {
        memory_cluster(h);
        if constexpr (FS >= 0) {
            fold_request(std::integral_constant<int, FS>{});
            __builtin_amdgcn_sched_barrier(0);
            fold_wait(h, std::integral_constant<int, FS>{});
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (FS >= 2) fold_add(std::integral_constant<int, FS - 2>{});
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else if constexpr (FS == -2 && CAN_FOLD) {
            constexpr int LFS = NFOLD - 2 + H;
            if (fold_c) {
                fold_request(std::integral_constant<int, LFS>{});
                fold_wait(h, std::integral_constant<int, LFS>{});
                fold_add(std::integral_constant<int, LFS - 2>{});
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            } else {
                wait_loads_and_barrier<(KK && H == 1 ? ND : 2 * ND)>();
            }
        } else {
            wait_loads_and_barrier<(KK && H == 1 ? ND : 2 * ND)>();
        }
        if constexpr (FS == -2) mask_tail(h);
        compute_cluster();
        __builtin_amdgcn_s_barrier();
    };
    constexpr std::integral_constant<int, -1> no_fold{};
    constexpr std::integral_constant<int, -2> last_pair{};

    MIW_PP_STAMP(1)
    if (late_group) __builtin_amdgcn_s_barrier();
    // the loop runs the pairs that neither fold nor are the last one
    const int NPM = fold_c ? NP - NFOLD / 2 : NP - 1;
    for (int pr = 0; pr < NPM; pr++) {
#ifdef MIW_PP_TS
        if (pr == NPM / 2) MIW_PP_STAMP(2)
        if (pr == NPM / 2 + 1) MIW_PP_STAMP(3)
#endif
        step(std::integral_constant<int, 0>{}, no_fold);
        step(std::integral_constant<int, 1>{}, no_fold);
    }
    MIW_PP_STAMP(9)
    if constexpr (CAN_FOLD) {
        if (fold_c) {
            [&]<int... G>(std::integer_sequence<int, G...>) {
                ((step(std::integral_constant<int, 0>{}, std::integral_constant<int, 2 * G>{}),
                  step(std::integral_constant<int, 1>{}, std::integral_constant<int, 2 * G + 1>{})),
                 ...);
            }(std::make_integer_sequence<int, NFOLD / 2 - 1>{});
        }
    }
    step(std::integral_constant<int, 0>{}, last_pair);
    step(std::integral_constant<int, 1>{}, last_pair);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may outlive the workgroup's LDS
    if constexpr (CAN_FOLD) {
        if (fold_c) {
            fold_add(std::integral_constant<int, NFOLD - 2>{});
            fold_add(std::integral_constant<int, NFOLD - 1>{});
        }
    }
    if (!late_group) __builtin_amdgcn_s_barrier();
    MIW_PP_STAMP(4)

    // Epilogue: each lane owns 4 consecutive i of one column j per MFMA tile.
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
    static_assert(TI % 2 == 0, "the epilogue stores pairs of tiles");
    auto epilogue = [&](bool with_c, bool trans) {
        auto value = [&](int a, int b) {
            float4_t v = acc[a][b];
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] *= p.alpha;
            if (with_c) {
                float4_t c = read_c(a, b, trans);
#pragma unroll
                for (int e = 0; e < 4; e++) v[e] = __builtin_fmaf(p.beta, c[e], v[e]);
            }
            return v;
        };
#pragma unroll
        for (int b = 0; b < TJ; b++)
#pragma unroll
            for (int a = 0; a < TI; a += 2)
                store_tile_pair<DT>(D, p.ldd, i0 + wi * WTI + 16 * a, j0 + wj * WTJ + 16 * b, lane, value(a, b), value(a + 1, b));
    };
    if (!p.use_c || fold_c) epilogue(false, false);
    else if (p.c_trans) epilogue(true, true);
    else epilogue(true, false);
#ifdef MIW_PP_TS
    MIW_PP_STAMP(5)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    MIW_PP_STAMP(6)
    ts[7] = wall_clock64();
    if (p.ts && lane == 0)
        for (int i = 0; i < 10; i++) p.ts[((long)(blockIdx.y * gridDim.x + blockIdx.x) * 8 + wave) * 10 + i] = ts[i];
#endif
}

// ---------------------------------------------------------------------------
// Ping-pong kernel with clusters of 64 k-values (one LDS slot), for the tiles whose rings of whole
// slots fit in LDS: 256x128, 128x256 (three slots) and 128x128 (four).  A wavefront's memory
// cluster reads the fragments of both k-steps of pair p out of the pair's slot and requests pair
// p + NSLOT - 1 into the slot of pair p - 1 (which the other group finished reading one barrier
// ago); its compute cluster issues the pair's 2 * TI * TJ MFMAs.  At the end of the memory cluster
// the wavefront lets the NSLOT - 2 youngest pairs stay in flight: pair p + 1 has landed, and the
// two barriers that follow publish it before anyone reads it.  Both operand kinds use the slot
// layouts, loaders and fragment readers of gemm_tiled.hpp.
//
// A wavefront issues one instruction in four to five cycles, whatever the instruction, and only one
// instruction rides for nothing behind each MFMA.  So both clusters are as long as their instruction
// counts: the memory cluster is kept to the fragment reads, three instructions per load and a handful
// of scalar ones (the part of the loop that needs no look at the end of K is unrolled over the ring,
// so that slots are compile-time offsets, and advances the operand origins behind MFMAs of the compute
// cluster), and the compute cluster to the MFMAs and what must follow them.
//
// fp16 accumulation rounds once per slot (64 k-values), two MFMAs after a tile's last MFMA of the pair,
// inside the compute cluster, except the cluster's last two tiles, which the wavefront rounds at the
// end of its next memory cluster (more there, or the conversions between the fragment reads, lengthen
// the memory cluster beyond the compute cluster: measured, up to 25 % of the launch).  With alpha == 1
// the accumulators start as half(beta * C) and the MFMAs accumulate onto the rounded sum in place,
// otherwise the running sum is kept beside accumulators that restart from zero in every slot:
// run = half(run + alpha * slot sum).  C is requested before anything else and converted once the
// first pair's loads have landed.
template <int BI, int BJ, int WI, int WJ, int NSLOT, bool XK, bool YK, class CT, class DT, bool F16ACC>
__global__ __launch_bounds__(WI *WJ * 64) __attribute__((amdgpu_waves_per_eu(2)))
void k_gemm_pp64(tiled_params p)
{
    constexpr int NT = WI * WJ * 64;
    static_assert(NT == 512, "two wavefronts per SIMD");
    constexpr int WTI = BI / WI, WTJ = BJ / WJ;
    constexpr int TI = WTI / 16, TJ = WTJ / 16;
    constexpr int XBYTES = BI * KGRAN * 2, YBYTES = BJ * KGRAN * 2, SLOT = XBYTES + YBYTES;
    static_assert(NSLOT >= 3 && NSLOT * SLOT <= 160 * 1024, "ring does not fit in LDS");
    using xload = slot_loader<BI, XK, NT>;
    using yload = slot_loader<BJ, YK, NT>;
    constexpr int NLX = xload::NLOAD, NLY = yload::NLOAD, LPAIR = NLX + NLY;  // loads per thread and pair
    constexpr int NTILE = TI * TJ;
    constexpr int NFRAG = 2 * (TI + TJ);  // fragment units of a memory cluster

#ifdef MIW_PP_TS
    long long ts[10] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    ts[0] = clock64();
    ts[8] = wall_clock64();
#endif
    extern __shared__ __attribute__((aligned(128))) char smem[];
    MIW_LDS char *lds = (MIW_LDS char *)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wi = wave % WI, wj = wave / WI;
    const bool late_group = wave >= 4;

    // Workgroup -> tile, as in k_gemm_tiled.
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

    frag_reader<BI, XK> xr;
    frag_reader<BJ, YK> yr;
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

    const int NP = (p.K + KGRAN - 1) / KGRAN;
    // K tail: the last pair starts at K - 64; tail_skip of its k-values repeat the pair before
    const int tail_skip = NP * KGRAN - p.K;
    const unsigned wave_dst = (unsigned)(uintptr_t)lds + (unsigned)wave * 1024u;
    int next = 0;          // next pair to request
    unsigned woff = 0;     // byte offset in the ring of the slot it goes to
    unsigned dma_dst = 0;  // this wavefront's first destination byte in that slot
    // A wavefront issues little more than one instruction in four to five cycles, whatever the
    // instruction, and its memory cluster is a chain of some sixty of them: every scalar instruction
    // spent on addresses there lengthens the cluster as much as a fragment read does.  So a load is
    // three instructions (M0 written by the addition that forms the LDS address; the global address is
    // the slot's uniform origin plus a lane offset, the loads of a K-major operand, whose origins lie
    // a multiple of the leading dimension apart, each with a lane offset of their own, the others with
    // the instruction's offset field), the ring positions are kept as byte offsets, and the pairs whose
    // request needs no look at the end of K (FAST) advance the origins by a loop-invariant step.
    unsigned xvo[XK ? NLX : 1], yvo[YK ? NLY : 1];
#pragma unroll
    for (int i = 0; i < (XK ? NLX : 1); i++) xvo[i] = xoff + 2u * (unsigned)xload::load_delta(i, p.ldx);
#pragma unroll
    for (int i = 0; i < (YK ? NLY : 1); i++) yvo[i] = yoff + 2u * (unsigned)yload::load_delta(i, p.ldy);
    auto begin_request = [&]() { dma_dst = wave_dst + woff; };
    // the same for a pair that reads slot SL, known at compile time: its request goes to the slot before
    auto begin_request_at = [&]<int SL>(std::integral_constant<int, SL>) { dma_dst = wave_dst + (unsigned)((SL + NSLOT - 1) % NSLOT * SLOT); };
    auto request_one = [&]<int I>(std::integral_constant<int, I>) {
        if constexpr (I < NLX) {
            if constexpr (XK) lds_dma16_at<I * NT * 16, 0>(X, xvo[I], dma_dst);
            else lds_dma16_at<I * NT * 16, I * (NT / 512) * 128>(X, xvo[0], dma_dst);  // load_delta: 64 rows further along i
        } else {
            constexpr int J = I - NLX;
            if constexpr (YK) lds_dma16_at<XBYTES + J * NT * 16, 0>(Y, yvo[J], dma_dst);
            else lds_dma16_at<XBYTES + J * NT * 16, J * (NT / 512) * 128>(Y, yvo[0], dma_dst);
        }
    };
    // Past the end of K the last pair is requested again, into a slot nobody reads any more.
    auto end_request = [&]() {
        next++;
        woff = woff + SLOT == NSLOT * SLOT ? 0 : woff + SLOT;
        const int kstep = next < NP - 1 ? KGRAN : next == NP - 1 ? KGRAN - tail_skip : 0;
        // (64 leading dimensions fit in 32 bits: the host checks that 256 do)
        X += XK ? kstep : kstep * (int)p.ldx;
        Y += YK ? kstep : kstep * (int)p.ldy;
    };
    // FAST pairs: one origin per call, issued behind an MFMA of the compute cluster
    auto advance_fast = [&](int which) {
        if (which == 0) X += XK ? KGRAN : KGRAN * (int)p.ldx;
        else Y += YK ? KGRAN : KGRAN * (int)p.ldy;
    };

    // fp16 accumulation: the C operand is requested first, as raw bits that no instruction touches
    // before the prologue's wait (a conversion here would make the compiler wait for the loads
    // before the first direct-to-LDS load is issued).  C laid out as D: the lane's four halves in two
    // registers; C stored across D: one zero-extended half per register.
    //
    // Where LDS has room for the workgroup's whole tile of C beside the ring (128 x 128: 32 KiB), a C laid
    // out as D comes through LDS instead: the accumulator layout reads 32 contiguous bytes per column
    // and instruction, which costs the 128 x 128 kernel 6000 cycles of prologue, whereas direct-to-LDS
    // loads fetch whole 256-byte columns (16 lanes per column).  Chunk (column j, 16-byte piece c) sits at
    // chunk index j * 16 + (c ^ (j & 15)), so that the 16 lanes that later read 16 columns at one row
    // offset hit 16 different 16-byte slots.
    constexpr bool C_STAGE_FITS = F16ACC && NSLOT * SLOT + BI * BJ * 2 <= 160 * 1024 && (BI * 2) % 256 == 0;
    constexpr int C_STAGE = NSLOT * SLOT;                         // byte offset of the staged tile
    constexpr int C_CHUNKS_PER_COL = BI * 2 / 16, NLC = C_STAGE_FITS ? BI * BJ * 2 / 16 / NT : 0;
    const bool c_staged = C_STAGE_FITS && p.use_c && !p.c_trans && p.ldc < (1l << 22);  // (32-bit lane offsets)
    if constexpr (C_STAGE_FITS) {
        if (c_staged) {
            const char *ctile = (const char *)(C + (long)j0 * p.ldc + i0);
#pragma unroll
            for (int n = 0; n < NLC; n++) {
                const int g = n * NT + tid;
                const int j = g / C_CHUNKS_PER_COL, c = (g % C_CHUNKS_PER_COL) ^ (j & 15);
                lds_dma16(ctile, (unsigned)(j * (int)p.ldc * 2 + c * 16), wave_dst + (unsigned)(C_STAGE + n * NT * 16));
            }
        }
    }
    unsigned craw[F16ACC ? TI : 1][F16ACC ? TJ : 1][4];
    if constexpr (F16ACC) {
        if (p.use_c && !c_staged) {
            auto fetch = [&]<bool TRANS>(std::bool_constant<TRANS>) {
#pragma unroll
                for (int a = 0; a < TI; a++)
#pragma unroll
                    for (int b = 0; b < TJ; b++) {
                        const int ii = row + 16 * a, jj = col + 16 * b;
                        if constexpr (TRANS) {
#pragma unroll
                            for (int v = 0; v < 4; v++) craw[a][b][v] = *(const unsigned short *)(C + (long)(ii + v) * p.ldc + jj);
                        } else {
                            const uint2_t two = *(const uint2_t *)(C + (long)jj * p.ldc + ii);
                            craw[a][b][0] = two[0];
                            craw[a][b][1] = two[1];
                        }
                    }
            };
            if (p.c_trans) fetch(std::true_type{});
            else fetch(std::false_type{});
        }
    }
    // Prologue: the first NSLOT - 1 pairs are requested.
#pragma unroll
    for (int s = 0; s < NSLOT - 1; s++) {
        begin_request();
        [&]<int... I>(std::integer_sequence<int, I...>) { (request_one(std::integral_constant<int, I>{}), ...); }
        (std::make_integer_sequence<int, LPAIR>{});
        end_request();
    }
    // The loop starts when pair 0 (and the C operand, requested before it) has landed: the wait at the
    // end of memory cluster p leaves NSLOT - 2 pairs in flight, so pair p + 1 has landed by then, the
    // first time as every other.
    wait_loads_and_barrier<(NSLOT - 2) * LPAIR>();
    float4_t cinit[F16ACC ? TI : 1][F16ACC ? TJ : 1];
    if constexpr (F16ACC) {
        auto convert = [&]<bool TRANS>(std::bool_constant<TRANS>) {
#pragma unroll
            for (int a = 0; a < TI; a++)
#pragma unroll
                for (int b = 0; b < TJ; b++)
#pragma unroll
                    for (int v = 0; v < 4; v++) {
                        const unsigned bits = TRANS ? craw[a][b][v] : craw[a][b][v >> 1] >> (16 * (v & 1));
                        const float c = (float)__builtin_bit_cast(half_t, (unsigned short)bits);
                        cinit[a][b][v] = round_through_half(p.beta * c);
                    }
        };
        if (!p.use_c) {
#pragma unroll
            for (int a = 0; a < TI; a++)
#pragma unroll
                for (int b = 0; b < TJ; b++) cinit[a][b] = float4_t{0.f, 0.f, 0.f, 0.f};
        } else if (c_staged) {
            if constexpr (C_STAGE_FITS) {
#pragma unroll
                for (int a = 0; a < TI; a++)
#pragma unroll
                    for (int b = 0; b < TJ; b++) {
                        const int j = wj * WTJ + 16 * b + r, i = wi * WTI + 16 * a + 4 * q;
                        const int at = C_STAGE + (j * C_CHUNKS_PER_COL + ((i >> 3) ^ (j & 15))) * 16 + (i & 7) * 2;
                        const half4_t h = *(MIW_LDS const half4_t *)(lds + at);
#pragma unroll
                        for (int v = 0; v < 4; v++) cinit[a][b][v] = round_through_half(p.beta * (float)h[v]);
                    }
            }
        } else if (p.c_trans) {
            convert(std::true_type{});
        } else {
            convert(std::false_type{});
        }
    }

    half8_t fx[2][TI], fy[2][TJ];
    if constexpr (MIW_PP_ABLATE & 2) {
        [&]<int... U>(std::integer_sequence<int, U...>) { ((fx[0][U] = fx[1][U] = xr.template read<U, 0>(lds)), ...); }(std::make_integer_sequence<int, TI>{});
        [&]<int... U>(std::integer_sequence<int, U...>) { ((fy[0][U] = fy[1][U] = yr.template read<U, 0>(lds + XBYTES)), ...); }(std::make_integer_sequence<int, TJ>{});
    }
    // fp16 accumulation: rounding of tile t = a * TJ + b after its pair's MFMAs.
    // RMODE 1 (alpha == 1): the accumulators start as half(beta * C), the MFMAs accumulate onto the
    //     rounded running sum, and it is rounded in place once per slot.
    // RMODE 3 (any alpha): `cinit` is the running sum (a Float16 value held as Float32), the MFMA
    //     accumulators restart from zero in every slot and run = half(run + alpha * slot sum).
    auto round_tile = [&]<int RMODE>(int t, std::integral_constant<int, RMODE>) {
        const int a = t / TJ, b = t % TJ;
        float4_t v = acc[a][b];
        if constexpr (RMODE == 3) {
#pragma unroll
            for (int e = 0; e < 4; e++) v[e] = __builtin_fmaf(p.alpha, v[e], cinit[a][b][e]);
        }
        half4_t h = __builtin_convertvector(v, half4_t);
        if constexpr (RMODE == 3) cinit[a][b] = __builtin_convertvector(h, float4_t);
        else acc[a][b] = __builtin_convertvector(h, float4_t);
    };
    // Fragment unit U of a memory cluster (step 0: the TI x-fragments, then the TJ y-fragments; then
    // step 1), preceded by the direct-to-LDS loads that go out before it (load n before unit
    // n * NFRAG / LPAIR).
    auto cluster_unit = [&]<int U>(MIW_LDS const char *xs, std::integral_constant<int, U>) {
        [&]<int... N>(std::integer_sequence<int, N...>) {
            (([&] {
                 if constexpr (N * NFRAG / LPAIR == U && !(MIW_PP_ABLATE & 1)) {
                     request_one(std::integral_constant<int, N>{});
                     __builtin_amdgcn_sched_barrier(0);
                 }
             }()),
             ...);
        }(std::make_integer_sequence<int, LPAIR>{});
        constexpr int H = U / (TI + TJ), V = U % (TI + TJ);
        if constexpr (MIW_PP_ABLATE & 2) {
            asm volatile("" : "+v"(fx[H][V % TI]), "+v"(fy[H][V % TJ]));
        } else {
            if constexpr (V < TI) fx[H][V] = xr.template read<V, H>(xs);
            else fy[H][V - TI] = yr.template read<V - TI, H>(xs + XBYTES);
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    unsigned roff = 0;  // byte offset in the ring of the slot that is read next
    // SL: -2: any pair; -1: a FAST pair; >= 0: a FAST pair that reads slot SL, known at compile time (the
    // loop is unrolled over the ring there: no ring position to keep, and the slot's offset is part of
    // the instructions' offset fields).  FAST pairs advance the origins in their compute cluster.
    auto memory_cluster = [&]<int SL>(std::integral_constant<int, SL> sl) {
        MIW_LDS const char *xs = SL >= 0 ? lds + SL * SLOT : lds + roff;
        if constexpr (SL >= 0) begin_request_at(sl);
        else begin_request();
        [&]<int... U>(std::integer_sequence<int, U...>) {
            (cluster_unit(xs, std::integral_constant<int, U>{}), ...);
        }(std::make_integer_sequence<int, NFRAG>{});
        if constexpr (SL == -2) end_request();
        if constexpr (SL == -1) woff = woff + SLOT == NSLOT * SLOT ? 0 : woff + SLOT;
        if constexpr (SL < 0) roff = roff + SLOT == NSLOT * SLOT ? 0 : roff + SLOT;
        __builtin_amdgcn_sched_barrier(0);
    };
    // ZERO (fp16 accumulation with alpha != 1): the accumulators restart from zero in every slot.
    auto tile_of_mfma = [](int m) { return m / TJ * TJ + serpentine_column(m, TJ); };
    // (fp16 accumulation, measured: with both k-steps of a tile back to back, so that the tiles finish
    // one after the other and the conversions spread over the whole cluster, the second MFMA of a tile
    // waits for the first and the launch takes 6 to 15 % longer.)
    constexpr int ROUND_LAG = 2;
    // The tiles whose last MFMA closes the compute cluster would be rounded behind it, with no MFMA to hide
    // the conversions and the other group waiting at the barrier: the last ROUND_DEFER tiles are rounded
    // at the end of the wavefront's next memory cluster instead (round_deferred), behind its last
    // fragment read and before the next compute cluster touches them.  (Measured on 2048^3: 1 or 2 tiles
    // 3 % faster than none, 3 and more slower again: the memory cluster must stay the shorter one.)
    constexpr int ROUND_DEFER = F16ACC ? 2 : 0;
    static_assert(ROUND_DEFER <= NTILE && ROUND_DEFER <= ROUND_LAG, "deferred tiles are the cluster's last");
    auto compute_cluster = [&]<bool ZERO, bool ADVANCE>(std::bool_constant<ZERO>, std::bool_constant<ADVANCE>) {
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int h = 0; h < 2; h++)
#pragma unroll
            for (int m = 0; m < NTILE; m++) {
                // serpentine order: every MFMA changes exactly one of its two operand fragments
                const int a = m / TJ, b = serpentine_column(m, TJ);
                if constexpr (!(MIW_PP_ABLATE & 4)) {
                    if (ZERO && h == 0) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fx[h][a], fy[h][b], float4_t{0.f, 0.f, 0.f, 0.f}, 0, 0, 0);
                    else acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fx[h][a], fy[h][b], acc[a][b], 0, 0, 0);
                }
                // fp16 accumulation: a tile is rounded ROUND_LAG MFMAs after its last MFMA of the pair
                if constexpr (ADVANCE)
                    if (h == 0 && m < 2) advance_fast(m);
                if constexpr (F16ACC)
                    if (h == 1 && m >= ROUND_LAG && m - ROUND_LAG < NTILE - ROUND_DEFER) round_tile(tile_of_mfma(m - ROUND_LAG), std::integral_constant<int, ZERO ? 3 : 1>{});
                __builtin_amdgcn_sched_barrier(0);
            }
        if constexpr (F16ACC)
#pragma unroll
            for (int m = NTILE > ROUND_LAG ? NTILE - ROUND_LAG : 0; m < NTILE - ROUND_DEFER; m++) round_tile(tile_of_mfma(m), std::integral_constant<int, ZERO ? 3 : 1>{});
    };
    // The first memory cluster rounds sums that are Float16 values already, which changes nothing, and
    // the last compute cluster's tiles are rounded behind the loop.
    auto round_deferred = [&]<bool ZERO>(std::bool_constant<ZERO>) {
#pragma unroll
        for (int m = NTILE - ROUND_DEFER; m < NTILE; m++) round_tile(tile_of_mfma(m), std::integral_constant<int, ZERO ? 3 : 1>{});
    };

    // Folding C (Float32 C laid out as D, alpha == 1): CPT MFMA tiles per cluster over the last
    // NFOLD clusters, requested at the end of a memory cluster with ordinary loads into registers
    // (the lane fetches the 16 bytes it owns).  They are the youngest loads of their cluster; the
    // wait LAG clusters later covers them and that cluster adds them in, so C has LAG clusters of
    // both wavefront groups to arrive.  LAG + 1 register stages rotate.
    constexpr int CPT = 1;
    constexpr int NFOLD = NTILE / CPT;
    constexpr int LAG = NSLOT - 1;
    constexpr bool CAN_FOLD = !F16ACC && __is_same(CT, float) && TI % CPT == 0;
    bool fold_c = false;
    if constexpr (CAN_FOLD) fold_c = p.use_c && !p.c_trans && p.alpha == 1.0f && NP >= NFOLD + 1 && p.ldc < (1l << 22);
    float4_t cst[LAG + 1][CPT];
    const char *cnext = (const char *)(C + (long)j0 * p.ldc + i0);
    const unsigned coff = 4u * (unsigned)((wj * WTJ + r) * (int)p.ldc + wi * WTI + 4 * q);
    auto fold_request = [&]<int S>(std::integral_constant<int, S>) {
        [&]<int... U>(std::integer_sequence<int, U...>) {
            (([&] {
                 constexpr int a = (S * CPT + U) % TI;
                 asm volatile("global_load_dwordx4 %0, %1, %2 offset:%3" : "=v"(cst[S % (LAG + 1)][U]) : "v"(coff), "s"(cnext), "n"(64 * a) : "memory");
                 if constexpr (a == TI - 1) cnext += 64 * p.ldc;
             }()),
             ...);
        }(std::make_integer_sequence<int, CPT>{});
    };
    auto fold_add = [&]<int S>(std::integral_constant<int, S>) {
#pragma unroll
        for (int u = 0; u < CPT; u++) {
            const int a = (S * CPT + u) % TI, b = (S * CPT + u) / TI;
#pragma unroll
            for (int e = 0; e < 4; e++) acc[a][b][e] = __builtin_fmaf(p.beta, cst[S % (LAG + 1)][u][e], acc[a][b][e]);
        }
    };
    // One pair: memory cluster, barrier, compute cluster, barrier.  FS >= 0: fold cluster FS.
    // Zeroes the repeated k-values in the fragments of the shifted last pair.
    auto mask_tail = [&]() {
        const unsigned keep0 = tail_keep<0>(tail_skip), keep1 = tail_keep<1>(tail_skip);
#pragma unroll
        for (int a = 0; a < TI; a++) { tail_apply(fx[0][a], keep0); tail_apply(fx[1][a], keep1); }
#pragma unroll
        for (int b = 0; b < TJ; b++) { tail_apply(fy[0][b], keep0); tail_apply(fy[1][b], keep1); }
    };
    // FS >= 0: fold pair FS (always folds).  FS == -1: a pair that does not fold.  FS == -2: the last
    // pair: its fragments are masked, and it is fold pair NFOLD - 1 when the launch folds C, which is
    // decided here at run time, so that the last pair is one piece of code for both cases (two
    // alternative pieces that each update all accumulators cost spills where they join).
    auto fold_wait = [&]<int FS>(std::integral_constant<int, FS>) {
        // Allowed to stay in flight: the ring loads of the NSLOT - 2 youngest clusters with the fold
        // loads issued after them, and the fold loads of the cluster before those (younger than
        // that cluster's ring loads, which must have landed).
        constexpr int YOUNGER = (NSLOT - 2) * LPAIR + CPT * (FS + 1 < NSLOT - 1 ? FS + 1 : NSLOT - 1);
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_waitcnt((YOUNGER & 15) | (7 << 4) | (0 << 8) | ((YOUNGER >> 4) << 14));
        asm volatile("" ::: "memory");
    };
    // RMODE: how the compute cluster rounds its sums (0: fp32 accumulation; 1, 3: see round_tile).
    auto pair = [&]<int FS, int RMODE, int SL = -2>(std::integral_constant<int, FS>, std::integral_constant<int, RMODE>, std::integral_constant<int, SL> sl = {}) {
        memory_cluster(sl);
        if constexpr (RMODE != 0) {
            round_deferred(std::bool_constant<RMODE == 3>{});
            __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (FS >= 0) {
            fold_request(std::integral_constant<int, FS>{});
            __builtin_amdgcn_sched_barrier(0);
            fold_wait(std::integral_constant<int, FS>{});
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (FS >= LAG) fold_add(std::integral_constant<int, FS - LAG>{});
            __builtin_amdgcn_sched_barrier(0);
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else if constexpr (FS == -2 && CAN_FOLD) {
            constexpr int LFS = NFOLD - 1;
            if (fold_c) {
                fold_request(std::integral_constant<int, LFS>{});
                fold_wait(std::integral_constant<int, LFS>{});
                fold_add(std::integral_constant<int, LFS - LAG>{});
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
            } else {
                wait_loads_and_barrier<(NSLOT - 2) * LPAIR>();
            }
        } else {
            wait_loads_and_barrier<(NSLOT - 2) * LPAIR>();
        }
        if constexpr (FS == -2) mask_tail();
        compute_cluster(std::bool_constant<RMODE == 3>{}, std::bool_constant<SL != -2>{});
        __builtin_amdgcn_s_barrier();
    };
    constexpr std::integral_constant<int, -1> no_fold{};
    constexpr std::integral_constant<int, -1> fast_pair{};
    // NSLOT pairs that need no look at the end of K, the first of which reads slot 0
#ifdef MIW_PP_TS
    bool stamp_pair = false;
#endif
    auto ring_of_pairs = [&]<int RMODE>(std::integral_constant<int, RMODE> rmode) {
        [&]<int... S>(std::integer_sequence<int, S...>) {
            (([&] {
#ifdef MIW_PP_TS
                 if constexpr (S == 1)
                     if (stamp_pair) MIW_PP_STAMP(3)
#endif
                 pair(std::integral_constant<int, -1>{}, rmode, std::integral_constant<int, S>{});
             }()),
             ...);
        }(std::make_integer_sequence<int, NSLOT>{});
    };
    constexpr std::integral_constant<int, -2> last_pair{};
    constexpr std::integral_constant<int, 0> plain{};

    MIW_PP_STAMP(1)
    if (late_group) __builtin_amdgcn_s_barrier();
    // the loop runs the pairs that neither fold nor are the last one
    const int NPM = fold_c ? NP - NFOLD : NP - 1;
    // the request of pair pr is pair pr + NSLOT - 1; the pairs before NP - 1 lie a full step apart
    const int NFAST = min(NPM, max(0, NP - 1 - NSLOT));
    const bool separate_sum = F16ACC && p.alpha != 1.0f;
    if constexpr (F16ACC) {
        // The running sum starts as half(beta * C): with alpha == 1 in the accumulators, which the MFMAs
        // add onto; otherwise beside them.
        constexpr std::integral_constant<int, 1> rolling{};
        constexpr std::integral_constant<int, 3> separate{};
        if (separate_sum) {
            int pr = 0;
            for (; pr + NSLOT <= NFAST; pr += NSLOT) ring_of_pairs(separate);
            for (; pr < NFAST; pr++) pair(no_fold, separate, fast_pair);
            next = NSLOT - 1 + pr;
            for (; pr < NPM; pr++) pair(no_fold, separate);
            pair(last_pair, separate);
            round_deferred(std::true_type{});
        } else {
#pragma unroll
            for (int a = 0; a < TI; a++)
#pragma unroll
                for (int b = 0; b < TJ; b++) acc[a][b] = cinit[a][b];
            int pr = 0;
            for (; pr + NSLOT <= NFAST; pr += NSLOT) {
                MIW_PP_MIDDLE(pr)
                ring_of_pairs(rolling);
            }
            for (; pr < NFAST; pr++) pair(no_fold, rolling, fast_pair);
            next = NSLOT - 1 + pr;
            for (; pr < NPM; pr++) pair(no_fold, rolling);
            MIW_PP_STAMP(9)
            pair(last_pair, rolling);
            round_deferred(std::false_type{});
        }
    } else {
        int pr = 0;
        for (; pr + NSLOT <= NFAST; pr += NSLOT) {
            MIW_PP_MIDDLE(pr)
            ring_of_pairs(plain);
        }
        for (; pr < NFAST; pr++) pair(no_fold, plain, fast_pair);
        next = NSLOT - 1 + pr;
        for (; pr < NPM; pr++) pair(no_fold, plain);
        MIW_PP_STAMP(9)
        if constexpr (CAN_FOLD) {
            if (fold_c) {
                [&]<int... G>(std::integer_sequence<int, G...>) {
                    (pair(std::integral_constant<int, G>{}, plain), ...);
                }(std::make_integer_sequence<int, NFOLD - 1>{});
            }
        }
        pair(last_pair, plain);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may outlive the workgroup's LDS
    if constexpr (CAN_FOLD) {
        if (fold_c) {
            [&]<int... G>(std::integer_sequence<int, G...>) {
                (fold_add(std::integral_constant<int, NFOLD - LAG + G>{}), ...);
            }(std::make_integer_sequence<int, LAG>{});
        }
    }
    if (!late_group) __builtin_amdgcn_s_barrier();
    MIW_PP_STAMP(4)

    // Epilogue: each lane owns 4 consecutive i of one column j per MFMA tile.
    static_assert(TI % 2 == 0, "the epilogue stores pairs of tiles");
    auto epilogue = [&](bool with_c, bool trans) {
        auto value = [&](int a, int b) {
            float4_t v = separate_sum ? cinit[a][b] : acc[a][b];
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
#ifdef MIW_PP_TS
    MIW_PP_STAMP(5)
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    MIW_PP_STAMP(6)
    ts[7] = wall_clock64();
    if (p.ts && lane == 0)
        for (int i = 0; i < 10; i++) p.ts[((long)(blockIdx.y * gridDim.x + blockIdx.x) * 8 + wave) * 10 + i] = ts[i];
#endif
}

}  // namespace miw

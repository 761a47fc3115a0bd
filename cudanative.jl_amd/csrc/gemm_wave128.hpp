// One wavefront per SIMD, 128x128 of the 256x256 tile per wavefront (fp32 accumulation): the form of
// the LDS-tiled GEMM with the fewest LDS bytes per flop (a fragment feeds eight MFMAs instead of four
// or eight: two thirds of the ping-pong kernel's fragment reads) and half as many wavefronts to
// issue loads, waits and barriers for.
//
// The 64 accumulator tiles of a wavefront are 256 registers: they live in the accumulation registers
// (AGPRs), which is why the MFMAs are written as inline assembly with that register class (left to
// itself the compiler splits the tiles between both register files and copies them to and fro in
// every k-step).  The ordinary registers hold two sets of fragments (8 + 8 fragments each).
//
// A wavefront alone on its SIMD issues strictly in order, so there is no partner to run the memory
// phase: the fragment reads of k-step s and the direct-to-LDS loads that refill the ring are issued
// between the MFMAs of k-step s - 1, one LDS or load instruction behind an MFMA (measured: one such
// instruction is issued under the 16 cycles of an MFMA at no cost, a second one or a VALU instruction
// beside it costs 4 cycles each; with two transposing reads and an address addition behind one MFMA
// the loop ran 10 % longer).  The reads fill the first three quarters of the step, so that the last
// of them has landed when the step ends; the loads come at even distances (the texture-address path
// takes about twenty cycles per load and four wavefronts share it), M0 written before an MFMA and the
// load that uses it issued behind that MFMA, in one assembly statement; the scalar ring bookkeeping
// and the lane addresses of the next step's reads take the slots that are left.  One s_barrier per
// k-step.
//
// The ring in LDS, the request order and the waits are those of the ping-pong kernel with 32-k
// clusters (gemm_pingpong.hpp): the "memory cluster" of k-step s is what runs here between the MFMAs
// of step s - 1.  At the end of step s - 1 a wavefront waits for its reads (all of them) and for the
// loads it issued two steps ago and earlier, and the barrier publishes them: a load has two k-steps
// (about 2100 cycles) to land.
//
// C is added in the epilogue.  The ping-pong kernels fold C into the last k-steps (loads into registers,
// fused multiply-adds onto the accumulators, under the MFMAs of the other wavefront); here the VALU
// cannot reach the AGPRs, and an MFMA takes its C operand from the register file it writes its result
// to (one bit selects AGPRs for both), so a tile cannot pass through ordinary registers on its way
// from one MFMA to the next: folding would take twelve VALU instructions per tile (four reads, four
// multiply-adds, four writes) out of issue slots that a lone wavefront needs for its MFMAs.  A problem
// that reads C therefore pays for it behind the loop (measured on 4096^3: 116.9 us against 107.1 for
// the ping-pong kernel; without a C operand 104.2 against 105.5), and miw_gemm picks this kernel by
// itself only for problems without one.
//
// The MFMAs are opaque to the compiler, so the hazards between them and other instructions are kept
// by construction and checked on the built code (tests/test_reflection.py): two MFMAs on one
// accumulator tile are 64 MFMAs apart, fragments are masked (K tail) a barrier before their first
// use, the MFMAs outside the rolled loops carry idle cycles in front (see mfma_agpr), and the
// epilogue waits out the last MFMA before the accumulators are read.
#pragma once
#include "gemm_pingpong.hpp"

namespace miw {

// SAFE: two idle cycles in front of the MFMA.  The compiler may place a register copy of its own (a VALU
// write) right in front of the statement, and an MFMA must not read a register in the two cycles after a
// VALU instruction wrote it; the compiler keeps that distance for the MFMAs it knows, not for this one.
// The steps of the K loop proper go without (the idle cycles cost 6 % there), and
// tests/test_reflection.py checks in the built code that no MFMA of this kernel follows such a write.
template <bool SAFE>
__device__ inline void mfma_agpr(float4_t &c, half8_t a, half8_t b)
{
    if constexpr (SAFE) asm volatile("s_nop 1\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
    else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}
// The same MFMA with one direct-to-LDS load around it: M0 before, the load behind (lane l fetches
// base + G_IMM + voff[l] into LDS byte lds_base + DST_IMM + 16 l; the instruction's offset field
// advances both addresses, so M0 is set back by as much).
template <int DST_IMM, int G_IMM, bool SAFE>
__device__ inline void mfma_agpr_dma(float4_t &c, half8_t a, half8_t b, const void *base, unsigned voff, unsigned lds_base)
{
    static_assert(G_IMM >= 0 && G_IMM < 4096, "instruction offset field");
    if constexpr (SAFE)
        asm volatile("s_add_u32 m0, %3, %6\n\ts_nop 0\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5 offset:%7"
                     : "+a"(c)
                     : "v"(a), "v"(b), "s"(lds_base), "v"(voff), "s"(base), "n"(DST_IMM - G_IMM), "n"(G_IMM)
                     : "memory", "m0", "scc");
    else
        asm volatile("s_add_u32 m0, %3, %6\n\tv_mfma_f32_16x16x32_f16 %0, %1, %2, %0\n\tglobal_load_lds_dwordx4 %4, %5 offset:%7"
                     : "+a"(c)
                     : "v"(a), "v"(b), "s"(lds_base), "v"(voff), "s"(base), "n"(DST_IMM - G_IMM), "n"(G_IMM)
                     : "memory", "m0", "scc");
}

// Slots of a k-step (slot m: what is issued with MFMA m).  Fragment u of the 16 (X's, then Y's) owns
// slots 3 u .. 3 u + 2: its LDS read in the first (an I-major operand's second read in the next one), and
// every other fragment's third slot carries a request (request n with MFMA 6 n + 2).  The scalar ring
// bookkeeping follows at slot 49 and the read addresses of the next step behind it.
constexpr int W128_ADVANCE_SLOT = 49;

template <bool XK, bool YK, class CT, class DT>
__global__ __launch_bounds__(256)
void k_gemm_w128(tiled_params p)
{
    constexpr int BI = 256, BJ = 256, WI = 2, WJ = 2;
    constexpr int NT = WI * WJ * 64;
    constexpr int WTI = BI / WI, WTJ = BJ / WJ;
    constexpr int TI = WTI / 16, TJ = WTJ / 16;
    constexpr int NMFMA = TI * TJ;
    constexpr bool KK = XK && YK;
    using xop = pp_operand<BI, XK, NT>;
    using yop = pp_operand<BJ, YK, NT, pp_y_slots(XK)>;
    constexpr int XB = xop::BYTES;
    constexpr int ND = xop::PER_CLUSTER + yop::PER_CLUSTER;  // loads per thread and k-step
    static_assert(!KK || (xop::NL == ND && yop::NL == ND), "alternating steps carry equal loads");
    static_assert(pp_fits(BI, BJ, XK, YK), "ring does not fit in LDS");
    static_assert(3 * (TI + TJ) <= W128_ADVANCE_SLOT && 6 * (ND - 1) + 2 < W128_ADVANCE_SLOT && W128_ADVANCE_SLOT + 9 < NMFMA,
                  "one memory instruction per MFMA");

    extern __shared__ __attribute__((aligned(128))) char smem[];
    MIW_LDS char *lds = (MIW_LDS char *)smem;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wi = wave % WI, wj = wave / WI;

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

    const int NP = (p.K + KGRAN - 1) / KGRAN;  // pairs of k-steps (the host passes K >= 128)
    const int NS = 2 * NP;
    const int tail_skip = NP * KGRAN - p.K;
    const unsigned lds0 = (unsigned)(uintptr_t)lds;
    const unsigned wave_dst = lds0 + (unsigned)wave * 1024u;

    // ---- ring state, requests: as in k_gemm_pp ----
    unsigned xpair = 0, xprev = 2 * xop::UNIT_BYTES, ypair = 0, yprev = (yop::UNITS - 1) * yop::UNIT_BYTES;
    int xnext = 0, ynext = 0;
    unsigned xvo[XK ? xop::NL : 1], yvo[YK ? yop::NL : 1];
#pragma unroll
    for (int i = 0; i < (XK ? xop::NL : 1); i++) xvo[i] = xoff + 2u * (unsigned)xop::load_delta(i, p.ldx);
#pragma unroll
    for (int i = 0; i < (YK ? yop::NL : 1); i++) yvo[i] = yoff + 2u * (unsigned)yop::load_delta(i, p.ldy);
    auto x_load = [&]<int I>(unsigned unit, std::integral_constant<int, I>) {
        if constexpr (XK) lds_dma16_at<I * NT * 16, 0>(X, xvo[I], wave_dst + unit);
        else lds_dma16_at<I * NT * 16, I * 128>(X, xvo[0], wave_dst + unit);
    };
    auto y_load = [&]<int I>(unsigned unit, std::integral_constant<int, I>) {
        if constexpr (YK) lds_dma16_at<XB + I * NT * 16, 0>(Y, yvo[I], wave_dst + unit);
        else lds_dma16_at<XB + I * NT * 16, I * 128>(Y, yvo[0], wave_dst + unit);
    };
    // Elements from one unit to the next; the first unit of the last pair lies tail_skip k-values short of
    // where it would follow on, and past the end of K the last unit is requested again (into a unit nobody
    // reads any more).  The step is a 32-bit product: the operand tile's offsets fit (the host checks).
    constexpr int XUK = XK ? KGRAN : BKS, YUK = YK ? KGRAN : BKS;
    // FAST: the unit requested next is neither the shifted last one nor past the end (true for all but the
    // last few steps, which a second copy of the loop runs): one 64-bit addition.
    auto x_advance = [&]<bool FAST>(std::bool_constant<FAST>) {
        xnext++;
        if constexpr (FAST) {
            X += XK ? XUK : XUK * (int)p.ldx;
        } else {
            const int ks = xnext == (XK ? NP - 1 : NS - 2) ? XUK - tail_skip : xnext < (XK ? NP : NS) ? XUK : 0;
            X += XK ? ks : ks * (int)p.ldx;
        }
    };
    auto y_advance = [&]<bool FAST>(std::bool_constant<FAST>) {
        ynext++;
        if constexpr (FAST) {
            Y += YK ? YUK : YUK * (int)p.ldy;
        } else {
            const int ks = ynext == (YK ? NP - 1 : NS - 2) ? YUK - tail_skip : ynext < (YK ? NP : NS) ? YUK : 0;
            Y += YK ? ks : ks * (int)p.ldy;
        }
    };
    // Request N (0 .. ND-1) of the memory part of k-step 2 pr + H, fused with one MFMA.
    auto mfma_with_request = [&]<int H, int N, bool SAFE>(float4_t &c, half8_t fa, half8_t fb, std::integral_constant<int, H>,
                                                          std::integral_constant<int, N>, std::bool_constant<SAFE>) {
        auto x_req = [&]<int I>(unsigned unit, std::integral_constant<int, I>) {
            if constexpr (XK) mfma_agpr_dma<I * NT * 16, 0, SAFE>(c, fa, fb, X, xvo[I], wave_dst + unit);
            else mfma_agpr_dma<I * NT * 16, I * 128, SAFE>(c, fa, fb, X, xvo[0], wave_dst + unit);
        };
        auto y_req = [&]<int I>(unsigned unit, std::integral_constant<int, I>) {
            if constexpr (YK) mfma_agpr_dma<XB + I * NT * 16, 0, SAFE>(c, fa, fb, Y, yvo[I], wave_dst + unit);
            else mfma_agpr_dma<XB + I * NT * 16, I * 128, SAFE>(c, fa, fb, Y, yvo[0], wave_dst + unit);
        };
        if constexpr (KK) {
            if constexpr (H == 0) y_req(yprev, std::integral_constant<int, N>{});
            else x_req(xprev, std::integral_constant<int, N>{});
        } else if constexpr (N < xop::PER_CLUSTER) {
            if constexpr (XK) x_req(xprev, std::integral_constant<int, H * xop::NL / 2 + N>{});
            else x_req(H == 0 ? (xpair ^ (2u * xop::UNIT_BYTES)) + xop::UNIT_BYTES : xpair, std::integral_constant<int, N>{});
        } else {
            constexpr int M = N - xop::PER_CLUSTER;
            if constexpr (YK) y_req(yprev, std::integral_constant<int, H * yop::NL / 2 + M>{});
            else y_req(H == 0 ? (ypair ^ (2u * yop::UNIT_BYTES)) + yop::UNIT_BYTES : ypair, std::integral_constant<int, M>{});
        }
    };
    auto cluster_advance = [&]<int H, bool FAST>(std::integral_constant<int, H>, std::bool_constant<FAST> fast) {
        if constexpr (!XK || H == 1) x_advance(fast);
        if constexpr (!YK || H == (KK ? 0 : 1)) y_advance(fast);
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

    // Prologue: the ring's first units in the order in which the loop needs them (see k_gemm_pp).
    auto prologue_unit = [&]<int U>(std::integral_constant<int, U>, bool is_x) {
        if (is_x) {
            [&]<int... I>(std::integer_sequence<int, I...>) {
                (x_load((unsigned)(U * xop::UNIT_BYTES), std::integral_constant<int, I>{}), ...);
            }(std::make_integer_sequence<int, xop::NL>{});
            x_advance(std::false_type{});
        } else {
            [&]<int... I>(std::integer_sequence<int, I...>) {
                (y_load((unsigned)(U * yop::UNIT_BYTES), std::integral_constant<int, I>{}), ...);
            }(std::make_integer_sequence<int, yop::NL>{});
            y_advance(std::false_type{});
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
    else if constexpr (!KK) prologue_unit(unit1, false);
    constexpr int PROLOGUE_LOADS = (XK ? 2 : 3) * xop::NL + (KK ? 1 : YK ? 2 : 3) * yop::NL;
    static_assert(xop::NL + yop::NL >= ND, "the units of step 2 must cover one step's requests");
    wait_loads_and_barrier<PROLOGUE_LOADS - xop::NL - yop::NL>();

    // Two fragment sets: the memory part of k-step s fills set s % 2.
    uint4_t fx[2][TI], fy[2][TJ];
    // Lane addresses of the fragment reads of the coming memory part: the unit's LDS address plus the
    // reader's lane offsets (one for a K-major operand, which depends on the half of the slot; four for an
    // I-major one).  They are worked out behind the ring bookkeeping of the step before.
    MIW_LDS const char *xa[XK ? 1 : 4], *ya[YK ? 1 : 4];
    auto read_addresses = [&]<int H, int W>(std::integral_constant<int, H>, std::integral_constant<int, W>) {
        // address number W of the memory part of a k-step of parity H: X's, then Y's
        constexpr int NX = XK ? 1 : 4;
        // (one VALU addition each, written out so that the compiler neither copies the result nor works it out again at every read)
        auto add = [&](MIW_LDS const char *&dst, unsigned unit, int lane_offset) {
            unsigned r;
            asm volatile("v_add_u32 %0, %1, %2" : "=v"(r) : "s"(lds0 + unit), "v"(lane_offset));
            dst = (MIW_LDS const char *)(uintptr_t)r;
        };
        if constexpr (W < NX) {
            if constexpr (XK) add(xa[0], xpair, xr.kr.base[H]);
            else add(xa[W], xpair + H * xop::UNIT_BYTES, xr.ibase[W]);
        } else if constexpr (W - NX < (YK ? 1 : 4)) {
            constexpr int V = W - NX;
            if constexpr (YK) add(ya[0], XB + ypair, yr.kr.base[H]);
            else add(ya[V], XB + ypair + H * yop::UNIT_BYTES, yr.ibase[V]);
        }
    };
    // Read number P (0, or 1: the second half of an I-major operand's fragment) of fragment U (X's TI, then
    // Y's TJ) of the memory part of a k-step of parity H, into fragment set H.
    auto lds_read = [&]<int H, int U, int P>(std::integral_constant<int, H>, std::integral_constant<int, U>, std::integral_constant<int, P>) {
        auto one = [&]<bool KM, int T>(uint4_t *f, MIW_LDS const char *const *addr, std::bool_constant<KM>, std::integral_constant<int, T>) {
            if constexpr (KM) {
                if constexpr (P == 0) f[T] = *(MIW_LDS const uint4_t *)(addr[0] + T * 2048);
            } else {
                const fp16x4_t v = __builtin_amdgcn_ds_read_tr16_b64_v4f16((MIW_LDS fp16x4_t *)(addr[T & 3] + (T >> 2) * 4096 + P * 512));
                const uint2_t w = __builtin_bit_cast(uint2_t, v);
                f[T][2 * P] = w[0];
                f[T][2 * P + 1] = w[1];
            }
        };
        if constexpr (U < TI) one(fx[H], xa, std::bool_constant<XK>{}, std::integral_constant<int, U>{});
        else one(fy[H], ya, std::bool_constant<YK>{}, std::integral_constant<int, U - TI>{});
    };

    // One step of the loop: the MFMAs of k-step s - 1 (COMPUTE; out of set H ^ 1) with the memory part of
    // k-step s = 2 pr + H between them (MEMORY; into set H), the waits, the barrier.  MASK: the fragments
    // read belong to the last pair of k-steps and are masked for the K tail.  SAFE: see mfma_agpr.
    auto step = [&]<int H, bool COMPUTE, bool MEMORY, bool MASK, bool SAFE, bool FAST>(std::integral_constant<int, H> h, std::bool_constant<COMPUTE>,
                                                                                      std::bool_constant<MEMORY>, std::bool_constant<MASK>,
                                                                                      std::bool_constant<SAFE> safe, std::bool_constant<FAST> fast) {
        // (the first MFMA of a step may follow copies that the compiler placed at the end of the step before)
        if constexpr (COMPUTE && !SAFE) asm volatile("s_nop 1" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
        [&]<int... M>(std::integer_sequence<int, M...>) {
            (([&] {
                 constexpr int a = M / TJ, b = serpentine_column(M, TJ);
                 constexpr int N = MEMORY && !(MIW_PP_ABLATE & 1) && M % 6 == 2 && M / 6 < ND ? M / 6 : -1;
                 if constexpr (COMPUTE && !(MIW_PP_ABLATE & 4)) {
                     const half8_t fa = __builtin_bit_cast(half8_t, fx[H ^ 1][a]), fb = __builtin_bit_cast(half8_t, fy[H ^ 1][b]);
                     if constexpr (N >= 0) mfma_with_request(acc[a][b], fa, fb, h, std::integral_constant<int, N>{}, safe);
                     else mfma_agpr<SAFE>(acc[a][b], fa, fb);
                 } else if constexpr (N >= 0) {
                     // (no MFMAs to go with: the first memory part, or a measurement build)
                     if constexpr (KK) {
                         if constexpr (H == 0) y_load(yprev, std::integral_constant<int, N>{});
                         else x_load(xprev, std::integral_constant<int, N>{});
                     } else if constexpr (N < xop::PER_CLUSTER) {
                         if constexpr (XK) x_load(xprev, std::integral_constant<int, H * xop::NL / 2 + N>{});
                         else x_load(H == 0 ? (xpair ^ (2u * xop::UNIT_BYTES)) + xop::UNIT_BYTES : xpair, std::integral_constant<int, N>{});
                     } else {
                         constexpr int MM = N - xop::PER_CLUSTER;
                         if constexpr (YK) y_load(yprev, std::integral_constant<int, H * yop::NL / 2 + MM>{});
                         else y_load(H == 0 ? (ypair ^ (2u * yop::UNIT_BYTES)) + yop::UNIT_BYTES : ypair, std::integral_constant<int, MM>{});
                     }
                 }
                 if constexpr (MEMORY && M % 3 < 2 && M / 3 < TI + TJ) {
                     if constexpr (MIW_PP_ABLATE & 2) asm volatile("" : "+v"(fx[H][(M / 3) % TI]), "+v"(fy[H][(M / 3) % TJ]));
                     else lds_read(h, std::integral_constant<int, M / 3>{}, std::integral_constant<int, M % 3>{});
                 }
                 if constexpr (MEMORY && M == W128_ADVANCE_SLOT) {
                     cluster_advance(h, fast);
                     if constexpr (H == 1) pair_advance();
                 }
                 // the next memory part has the other parity
                 if constexpr (MEMORY && M > W128_ADVANCE_SLOT && M <= W128_ADVANCE_SLOT + 8)
                     read_addresses(std::integral_constant<int, H ^ 1>{}, std::integral_constant<int, M - W128_ADVANCE_SLOT - 1>{});
                 __builtin_amdgcn_sched_barrier(0);
             }()),
             ...);
        }(std::make_integer_sequence<int, NMFMA>{});
        if constexpr (MEMORY) {
            constexpr int YOUNGER = KK && H == 1 ? ND : 2 * ND;
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_waitcnt((YOUNGER & 15) | (7 << 4) | (0 << 8) | ((YOUNGER >> 4) << 14));
            asm volatile("" ::: "memory");
            if constexpr (MASK) {
                const unsigned keep = tail_keep<H>(tail_skip);
#pragma unroll
                for (int a = 0; a < TI; a++)
#pragma unroll
                    for (int e = 0; e < 4; e++) fx[H][a][e] &= keep;
#pragma unroll
                for (int b = 0; b < TJ; b++)
#pragma unroll
                    for (int e = 0; e < 4; e++) fy[H][b][e] &= keep;
            }
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    constexpr std::integral_constant<int, 0> h0{};
    constexpr std::integral_constant<int, 1> h1{};
    constexpr std::true_type yes{};
    constexpr std::false_type no{};

    [&]<int... W>(std::integer_sequence<int, W...>) { (read_addresses(h0, std::integral_constant<int, W>{}), ...); }(std::make_integer_sequence<int, 8>{});
    if constexpr (MIW_PP_ABLATE & 2) {
#pragma unroll
        for (int s = 0; s < 2; s++) {
            [&]<int... U>(std::integer_sequence<int, U...>) {
                ((lds_read(std::integral_constant<int, 0>{}, std::integral_constant<int, U / 2>{}, std::integral_constant<int, U % 2>{})), ...);
            }(std::make_integer_sequence<int, 2 * (TI + TJ)>{});
#pragma unroll
            for (int a = 0; a < TI; a++) fx[1][a] = fx[0][a];
#pragma unroll
            for (int b = 0; b < TJ; b++) fy[1][b] = fy[0][b];
        }
    }
    // k-step 0's fragments, then the steps in pairs: {MFMAs 2 pr, memory 2 pr + 1}, {MFMAs 2 pr + 1, memory 2 pr + 2}
    step(h0, no, yes, no, yes, no);
    // (a request in the memory part of k-step s is for step s + 3 or pair s / 2 + 2: up to s = NS - 8 it is an ordinary unit)
    const int fast_pairs = NP > 4 ? NP - 4 : 0;
    for (int pr = 0; pr < fast_pairs; pr++) {
        step(h1, yes, yes, no, no, yes);
        step(h0, yes, yes, no, no, yes);
    }
    for (int pr = fast_pairs; pr < NP - 2; pr++) {
        step(h1, yes, yes, no, no, no);
        step(h0, yes, yes, no, no, no);
    }
    step(h1, yes, yes, no, yes, no);
    step(h0, yes, yes, yes, yes, no);  // reads k-step NS - 2: the last pair, masked
    step(h1, yes, yes, yes, yes, no);  // reads k-step NS - 1
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // no load may outlive the workgroup's LDS
    step(h0, yes, no, no, yes, no);    // the MFMAs of k-step NS - 1 (out of set 1)
    // The last MFMA has to leave the matrix core before the accumulators are read.  The accumulators pass
    // through the statements that wait, or the compiler, to which the MFMAs are opaque, moves its copies
    // out of the AGPRs up to right behind the MFMA that wrote the tile.
    static_assert(TJ == 8, "one statement per row of tiles");
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int a = 0; a < TI; a++)
        asm volatile("" : "+a"(acc[a][0]), "+a"(acc[a][1]), "+a"(acc[a][2]), "+a"(acc[a][3]), "+a"(acc[a][4]), "+a"(acc[a][5]), "+a"(acc[a][6]), "+a"(acc[a][7]));

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
    if (!p.use_c) epilogue(false, false);
    else if (p.c_trans) epilogue(true, true);
    else epilogue(true, false);
}

}  // namespace miw

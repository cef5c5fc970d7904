// bf16 GEMM fast path for gfx950: operand tiles go from global memory STRAIGHT into LDS
// (global_load_lds_dwordx4, 16 bytes per lane, no VGPR staging, no ds_write), for both
// operand layouts, and the transposition a row-contiguous operand needs is done by the
// LDS read itself (ds_read_b64_tr_b16).  The k loop therefore contains only MFMAs, LDS
// reads, the direct loads and one barrier.
//
// Same formulation as agh_gemm_kernel.h:  D[p][q] = sum_k P[p][k] * Q[q][k], on
// v_mfma_f32_16x16x32_bf16: lane l supplies row l % 16, k = 8 (l / 16) .. + 7 of a 32-deep substep, and
// accumulator element r of lane l = D[p0 + 4 (l / 16) + r][q0 + l % 16].  The 16x16x32 form does the same
// flop per cycle as 32x32x16 and reads the same LDS bytes per flop, but moves half as many accumulator
// registers per flop; on data that toggles like real data the part is power-limited, and a loop of nothing
// but MFMAs sustains about 15 % more flop per second with this form than with 32x32x16.
//
// LDS tile of an operand with BR rows, k-tile of 64:
//   LD_K (k contiguous in memory):   [row][64 k], 128-byte rows, 16-byte chunk c of row r at
//        slot c ^ swz(r)  (the layout of agh_gemm_kernel.h); fragment = one ds_read_b128 of chunk
//        l / 16 + 4 s of row l % 16: the 16 lanes the LDS serves together hit 16 different 16-byte bank groups.
//   LD_R (rows contiguous in memory): [k][BR rows], pitch 2*BR bytes.  A 32-byte group of 16
//        rows (index m) of k-row kr sits at group slot  m ^ (kr&3) ^ (((kr>>3)&1)<<2).
//        Fragment = two ds_read_b64_tr_b16: within a 16-lane group, lanes 4j..4j+3 point at
//        the 16 rows of k-row k0+j, and lane i receives the 4 k values of row i.  The slot
//        function spreads the four k-rows a group touches, and the k-rows 8 apart that two
//        neighbouring lane groups read, over distinct banks.
// A direct load deposits lane L's 16 bytes at (wave-uniform LDS base) + 16*L, so the swizzles
// are applied on the global side: each lane computes once which chunk of the tile belongs at
// its LDS position.
//
// Requirements checked by the host: every split's k range but the last a multiple of 64, operand
// base pointers 16-byte aligned, unit stride along k (LD_K: k a multiple of 8) or along rows (LD_R)
// with the other stride a multiple of 8 elements, rows a multiple of 8 for LD_R.  A last k-tile
// shorter than 64 is multiplied after the pipelined loop, its lanes reading zeros behind k = K.
#pragma once
#include "agh_gemm_kernel.h"

namespace agh {
namespace gemm {

typedef short s16x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

typedef float f32x4_t __attribute__((ext_vector_type(4)));
// 32-byte group m (16 rows) of k-row kr sits at group slot m ^ (kr & 3) ^ (((kr >> 3) & 1) << 2): an involution in m
__device__ __forceinline__ uint32_t rslot(uint32_t m, uint32_t kr) { return m ^ (kr & 3u) ^ (((kr >> 3) & 1u) << 2); }
__device__ __forceinline__ uint32_t rslot_inv(uint32_t ms, uint32_t kr) { return rslot(ms, kr); }
// The same for a tile of BR rows.  BR == 64: a k-row is 128 bytes, four groups, and covers only half of the LDS banks, so
// the slot function has two bits, and k-rows 8 apart (which two neighbouring 16-lane groups of a transposing read
// touch together) would meet on the same banks: k-rows with bit 3 set swap places with their even / odd neighbour
// (krow_pos, an involution), which puts them on the other half of the banks.
template <int BR>
__device__ __forceinline__ uint32_t rslot_br(uint32_t m, uint32_t kr) {
    if constexpr (BR == 64) return m ^ (kr & 3u);
    else return rslot(m, kr);
}
template <int BR>
__device__ __forceinline__ uint32_t krow_pos(uint32_t kr) {
    if constexpr (BR == 64) return kr ^ ((kr >> 3) & 1u);
    else return kr;
}

// 16-byte direct load: lane L's data lands at LDS address lds_base + 16*L (lds_base is
// wave-uniform and travels in M0).  Issued as inline assembly on purpose: the compiler's
// wait-count pass treats an LDS-DMA it knows about as aliasing EVERY later LDS read and would
// stall the fragment reads of the other stage until the load has landed.  Completion is
// awaited explicitly (s_waitcnt vmcnt(0)) before the barrier that publishes the stage.
__device__ __forceinline__ void direct_load16(const void *gptr, uint32_t lds_addr_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(lds_addr_uniform)
                 : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_address(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char *)p;
}

// Per-lane byte offsets (relative to the operand's tile origin for k-tile 0) of the NL direct
// loads this wave issues for one operand tile.
template <int MODE, int BR, int NWAVES>
struct DirectLoad {
    static constexpr int BYTES = BR * 128;
    static constexpr int NL = BYTES / 1024 / NWAVES;  // instructions per wave per k-tile
    static_assert(BYTES % (1024 * NWAVES) == 0, "tile must split evenly over the waves");
    static constexpr int PITCH = BR * 2;              // LD_R: bytes per k-row
    static constexpr int CPR = PITCH / 16;            // LD_R: 16-byte chunks per k-row
    static constexpr int KRPI = 1024 / PITCH;         // LD_R: k-rows per instruction

    static __device__ __forceinline__ void offsets(int64_t (&off)[NL], int64_t rs, int64_t ks, int r0, int NR,
                                                   int wave, int lane) {
#pragma unroll
        for (int i = 0; i < NL; ++i) {
            const int inst = wave * NL + i;
            if constexpr (MODE == LD_K) {
                const int row = inst * 8 + (lane >> 3);
                const int c = (lane & 7) ^ (int)swz((uint32_t)row);
                const int rowg = min(r0 + row, NR - 1);
                off[i] = ((int64_t)rowg * rs + c * 8) * 2;
            } else {
                const int kr = (int)krow_pos<BR>((uint32_t)(inst * KRPI + lane / CPR));  // the k-row stored at this LDS row
                const int pc = lane % CPR;
                const uint32_t m = rslot_br<BR>((uint32_t)(pc >> 1), (uint32_t)kr);
                int rowg = r0 + (int)(2 * m + (pc & 1)) * 8;
                if (rowg >= NR) rowg = NR - 8;
                off[i] = ((int64_t)kr * ks + rowg) * 2;
            }
        }
    }
    // whether this lane's 16 bytes of load i lie below k = rem within a k-tile (rem < 64: the last, shorter tile)
    static __device__ __forceinline__ bool below(int i, int wave, int lane, int rem) {
        const int inst = wave * NL + i;
        if constexpr (MODE == LD_K) {
            const int row = inst * 8 + (lane >> 3);
            return (((lane & 7) ^ (int)swz((uint32_t)row)) * 8) < rem;
        } else {
            return (int)krow_pos<BR>((uint32_t)(inst * KRPI + lane / CPR)) < rem;
        }
    }
};

// what the lanes of a shorter last k-tile read in place of elements at k >= K: both operands are zero there, so the
// products vanish whatever lies behind the end of a row
__device__ __align__(16) static const uint32_t kZeroChunk[4] = {0u, 0u, 0u, 0u};

// Per-lane LDS byte offsets for the MFMA fragments of one operand (16-row tile index i), v_mfma_f32_16x16x32_bf16:
// lane l supplies row l % 16, k = 8 * (l / 16) .. + 7 of a 32-deep substep.
template <int MODE, int BR, int NTILE>
struct FragRead {
    static constexpr int PITCH = BR * 2;
    // LD_K: chunk (l / 16) + 4 s of row rb + l % 16; substep s toggles bit 6 of the offset
    // LD_R: two transposing reads of 4 k-rows each: k-row 8 (l / 16) + (l % 16) / 4 (+ 4), 16-row group rb / 16
    static __device__ __forceinline__ void offsets(uint32_t (&off)[NTILE], int row_base, int lane) {
#pragma unroll
        for (int i = 0; i < NTILE; ++i) {
            const int rb = row_base + i * 16;
            if constexpr (MODE == LD_K) {
                const uint32_t lrow = (uint32_t)rb + (lane & 15), lg = lane >> 4;
                off[i] = lrow * 128u + ((lg ^ swz(lrow)) << 4);
            } else {
                const uint32_t j = (lane & 15) >> 2;
                const uint32_t kr = 8u * (lane >> 4) + j;
                off[i] = krow_pos<BR>(kr) * PITCH + 32u * rslot_br<BR>((uint32_t)(rb >> 4), kr) + 8u * (lane & 3);
            }
        }
    }
    static __device__ __forceinline__ uint4 read(const unsigned char *tile, uint32_t off, int s) {
        if constexpr (MODE == LD_K) {
            return *(const uint4 *)(tile + (off ^ (uint32_t)(s << 6)));
        } else {
            const unsigned char *p = tile + off + s * 32 * PITCH;
            s16x4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3))) *)p);
            s16x4_t hi =
                __builtin_amdgcn_ds_read_tr16_b64_v4i16((s16x4_t __attribute__((address_space(3))) *)(p + 4 * PITCH));
            uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
            return make_uint4(l2.x, l2.y, h2.x, h2.y);
        }
    }
};

// STAGED: the kernel is only launched with store_mode == ST_STAGED (the common case); the other
// epilogues are compiled out, which keeps their register demand from spilling accumulators.
// NS: LDS stages.  Two serve wherever the CU's matrix pipes are kept busy by a second workgroup or by a k-tile long
// enough to cover a load's latency; a 128 x 128 workgroup alone on its CU (a grid of at most one per CU) multiplies a
// k-tile in 512 cycles, a quarter of that latency, and runs a ring of four.
template <int BP, int BQ, int WGP, int WGQ, int LP, int LQ, bool STAGED, int NS = 2>
__global__ __launch_bounds__(WGP *WGQ * 64) void gemm_bf16_dl_kernel(Args g) {
    typedef uint16_t T;
    constexpr int NW = WGP * WGQ;
    constexpr int BK = 64;
    constexpr int MT = 16;  // MFMA tile: 16 x 16 outputs, 32 deep
    constexpr int TP = BP / WGP / MT, TQ = BQ / WGQ / MT;
    constexpr int P_BYTES = BP * 128, Q_BYTES = BQ * 128, STAGE_BYTES = P_BYTES + Q_BYTES;
    typedef DirectLoad<LP, BP, NW> DlP;
    typedef DirectLoad<LQ, BQ, NW> DlQ;
    typedef FragRead<LP, BP, TP> FrP;
    typedef FragRead<LQ, BQ, TQ> FrQ;

    static_assert(NS >= 2, "tile kt is multiplied while tile kt + 1 lands");
    __shared__ __align__(1024) unsigned char stages[NS][STAGE_BYTES];
    unsigned char *const stage0 = stages[0], *const stage1 = stages[1];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wp = wave % WGP, wq = wave / WGP;
    int tp, tq;
    tile_coords(blockIdx.x, g.tiles_p, g.tiles_q, tp, tq);
    const int p0 = tp * BP, q0 = tq * BQ;
    const int split = blockIdx.y;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int KT = kend > kbeg ? (kend - kbeg) / BK : 0;     // whole k-tiles
    const int rem = kend > kbeg ? (kend - kbeg) % BK : 0;    // depth of a shorter last one (the last split's only)

    int64_t offp[DlP::NL], offq[DlQ::NL];
    DlP::offsets(offp, g.ps, g.pk, p0, g.NP, wave, lane);
    DlQ::offsets(offq, g.qs, g.qk, q0, g.NQ, wave, lane);
    const int64_t stepP = (int64_t)BK * g.pk * 2, stepQ = (int64_t)BK * g.qk * 2;
    const unsigned char *gp[DlP::NL], *gq[DlQ::NL];
#pragma unroll
    for (int i = 0; i < DlP::NL; ++i)
        gp[i] = (const unsigned char *)g.P + offp[i] + ((int64_t)kbeg * g.pk + (int64_t)blockIdx.z * g.batch_p) * 2;
#pragma unroll
    for (int i = 0; i < DlQ::NL; ++i)
        gq[i] = (const unsigned char *)g.Q + offq[i] + ((int64_t)kbeg * g.qk + (int64_t)blockIdx.z * g.batch_q) * 2;

    uint32_t fp[TP], fq[TQ];
    FrP::offsets(fp, wp * TP * MT, lane);
    FrQ::offsets(fq, wq * TQ * MT, lane);

    f32x4_t acc[TP][TQ];
    static_for<TP>([&](auto ic) {
        static_for<TQ>([&](auto jc) { acc[decltype(ic)::value][decltype(jc)::value] = (f32x4_t)(0.0f); });
    });

    constexpr int NLP = DlP::NL, NLQ = DlQ::NL, NLT = NLP + NLQ;
    auto issue_load = [&](uint32_t stage_addr, auto lc, int64_t adv_p, int64_t adv_q) {
        constexpr int l = decltype(lc)::value;
        if constexpr (l < NLP) {
            direct_load16(gp[l], stage_addr + (wave * NLP + l) * 1024);
            gp[l] += adv_p;
        } else {
            direct_load16(gq[l - NLP], stage_addr + P_BYTES + (wave * NLQ + (l - NLP)) * 1024);
            gq[l - NLP] += adv_q;
        }
    };

    // two fragment sets of TP + TQ fragments each (one 32-deep substep of the wave's 128 x 128 tile)
    uint4 pfa[TP], qfa[TQ], pfb[TP], qfb[TQ];
    constexpr int NU = TP + TQ;
    auto read_unit = [&](uint4 (&pf)[TP], uint4 (&qf)[TQ], const unsigned char *stage, auto sc, auto uc) {
        constexpr int s = decltype(sc)::value, u = decltype(uc)::value;
        // unit order: P0, Q0, Q1, ..., Q(TQ-1), P1, ..., P(TP-1): the order the row-major MFMA walk first needs them
        if constexpr (u == 0) pf[0] = FrP::read(stage, fp[0], s);
        else if constexpr (u <= TQ) qf[u - 1] = FrQ::read(stage + P_BYTES, fq[u - 1], s);
        else pf[u - TQ] = FrP::read(stage, fp[u - TQ], s);
    };
    // Issued from inline assembly with the accumulator tied to the accumulation registers and updated in place: given
    // the builtin, the register allocator moves 16x16 tiles between the two register files inside the loop (several
    // hundred copies per k-tile).  An accumulator is next touched NM MFMAs later, so no result hazard arises here.
    auto mma = [&](f32x4_t &c, const uint4 &a, const uint4 &b) {
        asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(__builtin_bit_cast(u32x4_t, a)), "v"(__builtin_bit_cast(u32x4_t, b)));
    };

    // One k-tile = 2 substeps (32 k each) of NM MFMAs.  On entry: tile kt is visible in `cur`, its substep-0 fragments
    // are in set A and the loads of tiles kt+1 .. kt+NS-1 are in flight, those of tile kt+1 into `nxt`.  Every RSTEP-th of the first MFMAs of substep 0
    // is followed by one fragment read of substep 1 (set B; reading them back to back would ask the LDS for 1 KB per
    // wave every 16 cycles, its whole bandwidth), after which this wave needs nothing more from `cur`: the barrier at
    // MFMA NB frees `cur` and publishes `nxt`.  From there on the loads of tile kt+NS go out into `cur`, one every LSTEP
    // MFMAs, and the first MFMAs of substep 1 are followed by the reads of tile kt+1's substep 0 from `nxt` (set A).
    // sched_barrier(0) after every MFMA pins this interleaving.
    constexpr int NM = TP * TQ;
    constexpr int RSTEP = NU * 2 <= NM ? 2 : 1;                       // one fragment read every RSTEP MFMAs
    constexpr int NB = NU * RSTEP + NM / 16 < NM ? NU * RSTEP + NM / 16 : NM;  // barrier: a few MFMAs after the last read
    constexpr int LSTEP = NM / NLT > 0 ? NM / NLT : 1;                // one direct load every LSTEP MFMAs
    static_assert(NU * RSTEP <= NM, "fragment reads must fit behind the MFMAs of one substep");
    static_assert(NB + LSTEP * NLT <= 2 * NM, "the loads of a tile must go out within the tile");
    auto step = [&](unsigned char *cur, unsigned char *nxt, bool adv) __attribute__((always_inline)) {
        const uint32_t cur_addr = __builtin_amdgcn_readfirstlane(lds_address(cur));
        const int64_t ap = adv ? stepP : 0, aq = adv ? stepQ : 0;
        static_for<2 * NM>([&](auto nc) {
            constexpr int n = decltype(nc)::value, ph = n / NM, m = n % NM, i = m / TQ, j = m % TQ;
            if constexpr (n == NB) {
                asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((NS - 2) * NLT) : "memory");  // tile kt+1 has landed
                __builtin_amdgcn_s_barrier();
                asm volatile("" ::: "memory");
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (ph == 0) {
                mma(acc[i][j], pfa[i], qfa[j]);
                if constexpr (m % RSTEP == 0 && m / RSTEP < NU) read_unit(pfb, qfb, cur, std::integral_constant<int, 1>{}, std::integral_constant<int, m / RSTEP>{});
            } else {
                mma(acc[i][j], pfb[i], qfb[j]);
                if constexpr (m % RSTEP == 0 && m / RSTEP < NU) read_unit(pfa, qfa, nxt, std::integral_constant<int, 0>{}, std::integral_constant<int, m / RSTEP>{});
            }
            if constexpr (n >= NB && (n - NB) % LSTEP == LSTEP - 1 && (n - NB) / LSTEP < NLT)
                issue_load(cur_addr, std::integral_constant<int, (n - NB) / LSTEP>{}, ap, aq);
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    if (KT > 0) {
        // tile min(t, KT-1) -> stage t
        const uint32_t a0 = __builtin_amdgcn_readfirstlane(lds_address(stage0));
        static_for<NS * NLT>([&](auto nc) {
            constexpr int t = decltype(nc)::value / NLT, l = decltype(nc)::value % NLT;
            issue_load(a0 + t * STAGE_BYTES, std::integral_constant<int, l>{}, KT > t + 1 ? stepP : 0, KT > t + 1 ? stepQ : 0);
        });
        static_assert((NS - 1) * NLT < 64, "the wait counter holds six bits");
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((NS - 1) * NLT) : "memory");  // tile 0 has landed
        __syncthreads();
        static_for<NU>([&](auto uc) { read_unit(pfa, qfa, stage0, std::integral_constant<int, 0>{}, uc); });
    }
    int kt = 0;
    for (; kt + NS <= KT; kt += NS)  // step kt requests tile kt+NS and moves on if a tile kt+NS+1 exists
        static_for<NS>([&](auto sc) {
            constexpr int s = decltype(sc)::value;
            step(stages[s], stages[(s + 1) % NS], kt + s + NS + 1 < KT);
        });
    static_for<NS - 1>([&](auto sc) {
        constexpr int s = decltype(sc)::value;
        if (kt + s < KT) step(stages[s], stages[(s + 1) % NS], false);
    });
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (rem > 0) {
        // The shorter last k-tile, outside the pipeline (one load latency per workgroup, once): the same direct loads
        // into stage 0, lanes whose bytes lie at k >= K reading zeros instead.  After the loop the pointers stand at
        // the last whole tile (at this tile when there is none).
        const uint32_t a0 = __builtin_amdgcn_readfirstlane(lds_address(stage0));
        const int64_t tp_adv = KT > 0 ? stepP : 0, tq_adv = KT > 0 ? stepQ : 0;
        static_for<NLT>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            if constexpr (l < NLP) {
                const void *src = DlP::below(l, wave, lane, rem) ? (const void *)(gp[l] + tp_adv) : (const void *)kZeroChunk;
                direct_load16(src, a0 + (wave * NLP + l) * 1024);
            } else {
                const void *src = DlQ::below(l - NLP, wave, lane, rem) ? (const void *)(gq[l - NLP] + tq_adv) : (const void *)kZeroChunk;
                direct_load16(src, a0 + P_BYTES + (wave * NLQ + (l - NLP)) * 1024);
            }
        });
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        static_for<NU>([&](auto uc) { read_unit(pfa, qfa, stage0, std::integral_constant<int, 0>{}, uc); });
        static_for<NM>([&](auto mc) { mma(acc[decltype(mc)::value / TQ][decltype(mc)::value % TQ], pfa[decltype(mc)::value / TQ], qfa[decltype(mc)::value % TQ]); });
        if (rem > 32) {
            static_for<NU>([&](auto uc) { read_unit(pfb, qfb, stage0, std::integral_constant<int, 1>{}, uc); });
            static_for<NM>([&](auto mc) { mma(acc[decltype(mc)::value / TQ][decltype(mc)::value % TQ], pfb[decltype(mc)::value / TQ], qfb[decltype(mc)::value % TQ]); });
        }
        __syncthreads();  // the epilogue reuses the stages
    }

    // ------------------------------------------------------------ epilogue ----
    // accumulator element r of lane l, tile (i, j) = D[pwb + 16 i + 4 (l / 16) + r][qwb + 16 j + l % 16]
    const uint32_t l16 = lane & 15, lg = lane >> 4;
    const int pwb = p0 + wp * TP * MT, qwb = q0 + wq * TQ * MT;
    const int pw0 = pwb + (int)lg * 4, qw0 = qwb + (int)l16;
    T *D = (T *)g.D + (int64_t)blockIdx.z * g.batch_d;
    const T *bias = (const T *)g.bias;
    const int mode = STAGED ? (int)ST_STAGED : g.store_mode;
    const bool has_bias = g.has_bias != 0, bias_p = g.bias_on_p != 0;
    if (mode == ST_STAGED) {
        // beta == 0, D rows 16-byte aligned, NP a multiple of 8.  A lane holds 4 consecutive p of ONE q row and the
        // 16 lanes of a group hold 16 different q rows, so storing straight from the accumulators would write 8 bytes
        // into each of 64 different cache lines per instruction.  Instead each wave transposes 32 q rows (two tile
        // columns) at a time through its own LDS region and stores whole 16-byte chunks of contiguous row segments.
        constexpr int WPB = TP * MT * 2;               // bytes of one q row of the wave's tile
        constexpr int EPITCH = WPB + 16;               // bytes per staged q row (padded)
        constexpr int CPRW = WPB / 16;                 // 16-byte chunks per staged row
        constexpr int RPI = 64 / CPRW;                 // rows one store instruction covers
        constexpr int NST = 32 / RPI;                  // store instructions per pass
        static_assert(TQ % 2 == 0, "the staged epilogue takes two tile columns per pass");
        static_assert(4 * 32 * EPITCH <= STAGE_BYTES && NW <= 8, "epilogue staging must fit in the LDS stages");
        unsigned char *region = (wave < 4 ? stage0 : stage1) + (wave & 3) * 32 * EPITCH;
        auto staged = [&](auto plainc) {
            constexpr bool PLAIN = decltype(plainc)::value;
            // Bias and activation are applied after the transposition, on the already rounded product (the
            // reference's three separate ops: T(dot), then T(. + bias), then relu), where a lane holds 8
            // consecutive p of one q row.  A bias along p (C's unit-stride axis) is then the same 8 values
            // for every row the lane stores: they are widened to f32 once.  A bias along q is one value
            // per stored row.
            const int chunk = lane % CPRW;
            const bool post_bias = has_bias && bias_p, row_bias = has_bias && !bias_p, relu = g.act == AGH_ACT_RELU;
            float bpf[8];
            if constexpr (!PLAIN) {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    bpf[e] = 0.0f;
                    if (post_bias) bpf[e] = bf16_raw_f32(bias[(int64_t)min(pwb + chunk * 8 + e, g.NP - 1) * g.bias_stride]);
                }
            }
            const float alpha = g.alpha;
            static_for<TQ / 2>([&](auto jc) {
                constexpr int jj = decltype(jc)::value;
                static_for<2>([&](auto hc) {
                    constexpr int half = decltype(hc)::value, j = 2 * jj + half;
                    static_for<TP>([&](auto ic) {
                        constexpr int i = decltype(ic)::value;
                        const int pl = i * MT + (int)lg * 4;  // p inside the wave tile
                        const uint32_t w0 = f32x2_to_bf16x2(alpha * acc[i][j][0], alpha * acc[i][j][1]);
                        const uint32_t w1 = f32x2_to_bf16x2(alpha * acc[i][j][2], alpha * acc[i][j][3]);
                        *(uint2 *)(region + (half * 16 + l16) * EPITCH + pl * 2) = make_uint2(w0, w1);
                    });
                });
                // same wave, LDS executes in order: the reads below see the writes above
                static_for<NST>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    const int row = r * RPI + lane / CPRW;
                    uint4 v = *(const uint4 *)(region + row * EPITCH + chunk * 16);
                    const int qq = qwb + jj * 32 + row, pp = pwb + chunk * 8;
                    if constexpr (!PLAIN) {
                        uint32_t w[4] = {v.x, v.y, v.z, v.w};
                        float brow = 0.0f;
                        if (row_bias) brow = bf16_raw_f32(bias[(int64_t)min(qq, g.NQ - 1) * g.bias_stride]);  // wave-uniform branch
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            // the two bf16 values as f32 (exact); an addition quiets a signalling NaN by itself
                            float lo = __uint_as_float(w[e] << 16), hi = __uint_as_float(w[e] & 0xFFFF0000u);
                            if (has_bias) {  // wave-uniform
                                lo = (post_bias ? bpf[2 * e] : brow) + lo;
                                hi = (post_bias ? bpf[2 * e + 1] : brow) + hi;
                            }
                            // relu keeps x when x >= 0 (so -0 stays, NaN goes to 0).  Taken on the f32 sum before it is
                            // rounded: rounding to bf16 changes neither the sign nor NaN-ness, and a sum of two bf16
                            // values is zero or at least the smallest bf16 subnormal, so it cannot round to -0.
                            if (relu) {  // wave-uniform
                                lo = lo >= 0.0f ? lo : 0.0f;
                                hi = hi >= 0.0f ? hi : 0.0f;
                            }
                            w[e] = f32x2_to_bf16x2(lo, hi);
                        }
                        v = make_uint4(w[0], w[1], w[2], w[3]);
                    }
                    // streaming store: C is not read again by this launch, and keeping it out of the last-level
                    // cache leaves that cache to the operand panels, which every tile row / column re-reads
                    if (qq < g.NQ && pp < g.NP)
                        __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, (u32x4_t *)(D + (int64_t)qq * g.dq + pp));
                });
            });
        };
        if (!has_bias && g.act == AGH_ACT_NONE) staged(std::true_type{});
        else staged(std::false_type{});
    } else if (mode == ST_SPLITK) {
        static_for<TQ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int q = qw0 + j * MT;
            float *wrow = g.ws + ((size_t)split * g.NQ + q) * g.NPpad;
            static_for<TP>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                const int p = pw0 + i * MT;
                if (q < g.NQ && p < g.NPpad)
                    *(float4 *)(wrow + p) = make_float4(acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]);
            });
        });
    } else if (mode == ST_VEC) {
        static_for<TQ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int q = qw0 + j * MT;
            const bool qok = q < g.NQ;
            T bq = 0;
            if (qok && has_bias && !bias_p) bq = bias[(int64_t)q * g.bias_stride];
            T *drow = D + (int64_t)q * g.dq;
            static_for<TP>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                const int p = pw0 + i * MT;
                if (qok && p < g.NP) {
                    T *dst = drow + p;
                    __align__(8) T old[4] = {0, 0, 0, 0};
                    if (g.beta != 0.0f) *(uint2 *)old = *(const uint2 *)dst;
                    T b0 = bq, b1 = bq, b2 = bq, b3 = bq;
                    if (has_bias && bias_p) {
                        b0 = bias[(int64_t)(p + 0) * g.bias_stride];
                        b1 = bias[(int64_t)(p + 1) * g.bias_stride];
                        b2 = bias[(int64_t)(p + 2) * g.bias_stride];
                        b3 = bias[(int64_t)(p + 3) * g.bias_stride];
                    }
                    __align__(8) T out[4];
                    out[0] = finish<T>(acc[i][j][0], g.alpha, g.beta, old[0], has_bias, b0, g.act);
                    out[1] = finish<T>(acc[i][j][1], g.alpha, g.beta, old[1], has_bias, b1, g.act);
                    out[2] = finish<T>(acc[i][j][2], g.alpha, g.beta, old[2], has_bias, b2, g.act);
                    out[3] = finish<T>(acc[i][j][3], g.alpha, g.beta, old[3], has_bias, b3, g.act);
                    *(uint2 *)dst = *(const uint2 *)out;
                }
            });
        });
    } else {
        static_for<TQ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int q = qw0 + j * MT;
            const bool qok = q < g.NQ;
            T bq = 0;
            if (qok && has_bias && !bias_p) bq = bias[(int64_t)q * g.bias_stride];
            T *drow = D + (int64_t)q * g.dq;
            static_for<TP>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                static_for<4>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    const int p = pw0 + i * MT + r;
                    if (qok && p < g.NP) {
                        T *dst = drow + (int64_t)p * g.dp;
                        T old = 0;
                        if (g.beta != 0.0f) old = *dst;
                        T bv = bq;
                        if (has_bias && bias_p) bv = bias[(int64_t)p * g.bias_stride];
                        *dst = finish<T>(acc[i][j][r], g.alpha, g.beta, old, has_bias, bv, g.act);
                    }
                });
            });
        });
    }
}

}  // namespace gemm
}  // namespace agh

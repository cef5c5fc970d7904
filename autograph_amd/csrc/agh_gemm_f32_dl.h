// f32 GEMM on gfx950 with the operand tiles going from global memory straight into LDS
// (global_load_lds_dwordx4): no staging registers, no address arithmetic per load, no LDS write instructions.
// Staged through registers, a 64 x 64 tile (sixteen MFMAs per wave and k-tile) spends as long on those as on the
// MFMAs themselves (agh_gemm_kernel.h); here a k-tile is the MFMAs, the fragment reads, the direct loads and one
// barrier.
//
// Same formulation as agh_gemm_kernel.h: D[p][q] = sum_k P[p][k] * Q[q][k] on v_mfma_f32_32x32x2_f32, four waves
// in a 2 x 2 grid, a wave owns TP x TQ tiles of 32 x 32, the workgroup 64 TP x 64 TQ.  Lane l supplies row l % 32
// and, in substep s (8 k) of a k-tile (32 k), the four k values 8 s + 4 (l / 32) + e, e = 0..3, one per MFMA.
//
// LDS image of an operand's BR rows x 32 k (BR / 8 direct loads of 1 KB; a load deposits lane L's 16 bytes at
// base + 16 L):
//   LD_K (k contiguous in memory): [row][32 k], 128-byte rows, eight rows per load, 16-byte chunk c of row r at slot
//        c ^ swz(r): the layout and the fragment read (one ds_read_b128) of agh_gemm_kernel.h; the swizzle is
//        applied on the global side.
//   LD_R (rows contiguous in memory): [k][BR rows] as it comes, 1024 / (4 BR) k-rows per load.  The image of a load
//        starts 1024 + pad bytes after the one before, pad chosen so that k-rows four apart (the two half-waves of
//        a fragment read) fall on the two halves of the banks.  Fragment = four ds_read_b32.
// A ring of NS stages.  With three or more, the loads of k-tile kt + NS - 1 go out during the first substep of k-tile
// kt, into the stage k-tile kt - 1 has left; with two, those of k-tile kt + 2 during the last substep of k-tile kt,
// behind the barrier after which nobody reads that stage any more.  Either way a load has more than NS - 2 k-tiles
// to land (with two stages: most of one, which for 128-row tiles is 4000 matrix-pipe cycles).
//
// KS = 2 splits every k-tile between two waves per 32 x 32-tile position (eight waves, two per SIMD: while one waits
// for its fragments or at the barrier the other multiplies): a wave takes two of a k-tile's four substeps, and the
// two partial accumulators are added through LDS in front of the epilogue, always in the same order.  For grids that
// give a CU a single workgroup.
//
// Requirements checked by the host: every split's k range but the last a multiple of 32, operand base pointers
// 16-byte aligned, unit stride along k (LD_K: k a multiple of 4) or along rows (LD_R) with the other stride a
// multiple of 4 elements, rows a multiple of 4 for LD_R.  A last k-tile shorter than 32 is multiplied after the
// pipelined loop, its lanes reading zeros behind k = K.
#pragma once
#include "agh_gemm_bf16_dl.h"

namespace agh {
namespace gemm {

// LDS geometry of one operand of BR rows in layout MODE
template <int MODE, int BR>
struct F32DlOperand {
    static constexpr int LOADS = BR / 8;                            // direct loads per k-tile (workgroup)
    static constexpr int KRPI = MODE == LD_R ? 256 / BR : 1;        // LD_R: k-rows per load image
    static constexpr int IMG = 1024 + (MODE == LD_R ? 128 / (4 / KRPI) : 0);  // bytes from one image to the next
    static constexpr int BYTES = LOADS * IMG;
    static_assert(MODE != LD_R || (BR == 64 || BR == 128 || BR == 256), "row-contiguous tiles of 64, 128 or 256 rows");
    // byte offset of k-row k (LD_R)
    static constexpr int koff(int k) { return (k / KRPI) * IMG + (k % KRPI) * BR * 4; }
};

template <int TP, int TQ, int NS, int LP, int LQ>
struct F32DlGeo {
    static constexpr int BP = 64 * TP, BQ = 64 * TQ;
    typedef F32DlOperand<LP, BP> OpP;
    typedef F32DlOperand<LQ, BQ> OpQ;
    static constexpr int STAGE_BYTES = OpP::BYTES + OpQ::BYTES;
    static constexpr int SMEM_BYTES = NS * STAGE_BYTES;
};

// what the lanes of a shorter last k-tile read in place of elements at k >= K
__device__ __align__(16) static const uint32_t kZeroChunkF32[4] = {0u, 0u, 0u, 0u};

template <int TP, int TQ, int NS, int LP, int LQ, int KS = 1>
__global__ __launch_bounds__(256 * KS) void gemm_f32_dl_kernel(Args g) {
    typedef float T;
    static_assert((LP == LD_K || LP == LD_R) && (LQ == LD_K || LQ == LD_R), "vector layouts only");
    static_assert(KS == 1 || KS == 2, "a k-tile goes to one wave or is split between two");
    constexpr int SPW = 4 / KS;  // substeps of a k-tile per wave
    typedef F32DlGeo<TP, TQ, NS, LP, LQ> Geo_;
    typedef typename Geo_::OpP OpP;
    typedef typename Geo_::OpQ OpQ;
    constexpr int BP = Geo_::BP, BQ = Geo_::BQ, BK = 32;
    constexpr int STAGE_BYTES = Geo_::STAGE_BYTES;
    constexpr int LPWP = OpP::LOADS / (4 * KS), LPWQ = OpQ::LOADS / (4 * KS), LPW = LPWP + LPWQ;  // direct loads per wave and k-tile
    static_assert(LPWP >= 1 && LPWQ >= 1, "every wave issues loads of both operands");
    static_assert(NS >= 2 && (NS - 1) * LPW <= 63, "the loads in flight must fit the counter");
    constexpr bool EARLY = NS >= 3;                  // requests in the first substep (see above)
    constexpr int AHEAD = EARLY ? NS - 1 : NS;       // k-tile kt requests k-tile kt + AHEAD; the prologue the AHEAD first
    constexpr int INFLIGHT = (NS - 2) * LPW;         // loads that may still be in flight when k-tile kt + 1 is awaited
    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wp = wave & 1, wq = (wave >> 1) & 1;
    const int kh = wave >> 2;  // which half of every k-tile's substeps (KS == 2)
    int tp, tq;
    tile_coords(blockIdx.x, g.tiles_p, g.tiles_q, tp, tq);
    const int p0 = tp * BP, q0 = tq * BQ;
    const int split = blockIdx.y;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int KT = kend > kbeg ? (kend - kbeg) / BK : 0;   // whole k-tiles
    const int rem = kend > kbeg ? (kend - kbeg) % BK : 0;  // depth of a shorter last one (the last split's only)

    // ---- the wave's direct loads (instructions wave * n .. wave * n + n - 1 of an operand's loads) ----
    // per-lane global address for k-tile 0, LDS offset of the load's image inside the operand, bytes per k-tile
    const unsigned char *gp[LPWP], *gq[LPWQ];
    uint32_t lp[LPWP], lq[LPWQ];
    auto setup = [&](auto opc, auto modec, auto nc, const void *base, int64_t rs, int64_t ks, int64_t batch_off, int r0,
                     int NR, auto &gptr, auto &loff, int64_t &kstep) {
        typedef typename decltype(opc)::type Op;
        constexpr int MODE = decltype(modec)::value, N = decltype(nc)::value;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int inst = wave * N + i;
            int64_t off;
            if constexpr (MODE == LD_K) {
                const int row = inst * 8 + (lane >> 3);
                const int c = (lane & 7) ^ (int)swz((uint32_t)row);
                const int rowg = min(r0 + row, NR - 1);
                off = (int64_t)rowg * rs + kbeg + c * 4;
            } else {
                constexpr int LPK = 64 / Op::KRPI;  // lanes per k-row
                const int kr = inst * Op::KRPI + lane / LPK;
                int rowg = r0 + (lane % LPK) * 4;
                if (rowg >= NR) rowg = NR - 4;  // NR is a multiple of 4 on this path
                off = (int64_t)(kbeg + kr) * ks + rowg;
            }
            loff[i] = (uint32_t)inst * Op::IMG;
            gptr[i] = (const unsigned char *)base + (off + batch_off) * 4;
        }
        kstep = (MODE == LD_K ? (int64_t)BK : (int64_t)BK * ks) * 4;
    };
    int64_t stepP, stepQ;
    setup(std::common_type<OpP>{}, std::integral_constant<int, LP>{}, std::integral_constant<int, LPWP>{}, g.P, g.ps, g.pk,
          (int64_t)blockIdx.z * g.batch_p, p0, g.NP, gp, lp, stepP);
    setup(std::common_type<OpQ>{}, std::integral_constant<int, LQ>{}, std::integral_constant<int, LPWQ>{}, g.Q, g.qs, g.qk,
          (int64_t)blockIdx.z * g.batch_q, q0, g.NQ, gq, lq, stepQ);
    const uint32_t smem_addr = __builtin_amdgcn_readfirstlane(lds_address(smem));
    // load l of this wave's LPW for k-tile t (clamped to the last k-tile: that image is then never read)
    auto request_one = [&](int t, auto lc) {
        constexpr int l = decltype(lc)::value;
        const int tc = min(t, KT - 1);
        const uint32_t st = smem_addr + (uint32_t)(t % NS) * STAGE_BYTES;
        if constexpr (l < LPWP) direct_load16(gp[l] + (int64_t)tc * stepP, st + lp[l]);
        else direct_load16(gq[l - LPWP] + (int64_t)tc * stepQ, st + OpP::BYTES + lq[l - LPWP]);
    };

    // ---- fragment reads: lane l supplies row l % 32, k = 8 s + 4 (l / 32) + e ----
    const uint32_t lrow = lane & 31, lg = lane >> 5;
    uint32_t fp[TP], fq[TQ];
    auto frag_offsets = [&](auto opc, auto modec, auto nc, int wave_row, auto &off) {
        typedef typename decltype(opc)::type Op;
        constexpr int MODE = decltype(modec)::value, N = decltype(nc)::value;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const uint32_t r = (uint32_t)wave_row + 32u * i + lrow;
            // the wave's first substep is SPW * kh; its later ones toggle bits 5.. (LD_K) or add koff(8 s) (LD_R)
            if constexpr (MODE == LD_K) off[i] = (r * 128u + ((lg ^ swz(r)) << 4)) ^ (uint32_t)((SPW * kh) << 5);
            else off[i] = lg * (uint32_t)Op::koff(4) + r * 4u + (uint32_t)(kh * Op::koff(8 * (SPW % 4)));
        }
    };
    frag_offsets(std::common_type<OpP>{}, std::integral_constant<int, LP>{}, std::integral_constant<int, TP>{}, wp * 32 * TP, fp);
    frag_offsets(std::common_type<OpQ>{}, std::integral_constant<int, LQ>{}, std::integral_constant<int, TQ>{}, wq * 32 * TQ, fq);
    auto frag_read = [&](auto opc, auto modec, const unsigned char *op, uint32_t off, auto sc) -> uint4 {
        typedef typename decltype(opc)::type Op;
        constexpr int MODE = decltype(modec)::value, s = decltype(sc)::value;
        if constexpr (MODE == LD_K) {
            return *(const uint4 *)(op + (off ^ (uint32_t)(s << 5)));
        } else {
            const unsigned char *p = op + off + Op::koff(8 * s);
            return make_uint4(*(const uint32_t *)(p + Op::koff(0)), *(const uint32_t *)(p + Op::koff(1)),
                              *(const uint32_t *)(p + Op::koff(2)), *(const uint32_t *)(p + Op::koff(3)));
        }
    };
    // unit u of a substep's TP + TQ fragments, in the order the MFMA walk first needs them: P0, Q0 .. Q(TQ-1), P1 ..
    constexpr int NU = TP + TQ, NM = TP * TQ, SLOTS = 4 * NM;
    auto read_unit = [&](uint4(&pf)[TP], uint4(&qf)[TQ], const unsigned char *stage, auto sc, auto uc) {
        constexpr int u = decltype(uc)::value;
        if constexpr (u == 0) pf[0] = frag_read(std::common_type<OpP>{}, std::integral_constant<int, LP>{}, stage, fp[0], sc);
        else if constexpr (u <= TQ)
            qf[u - 1] = frag_read(std::common_type<OpQ>{}, std::integral_constant<int, LQ>{}, stage + OpP::BYTES, fq[u - 1], sc);
        else pf[u - TQ] = frag_read(std::common_type<OpP>{}, std::integral_constant<int, LP>{}, stage, fp[u - TQ], sc);
    };

    f32x16 acc[TP][TQ];
#pragma unroll
    for (int i = 0; i < TP; ++i)
#pragma unroll
        for (int j = 0; j < TQ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    uint4 pfa[TP], qfa[TQ], pfb[TP], qfb[TQ];  // fragment sets of even and odd substeps
    if (KT > 0) {
        static_for<AHEAD>([&](auto tc) { static_for<LPW>([&](auto lc) { request_one(decltype(tc)::value, lc); }); });
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"((AHEAD - 1) * LPW) : "memory");  // this wave's part of k-tile 0 has landed
        __builtin_amdgcn_s_barrier();                                             // and everybody else's
        asm volatile("" ::: "memory");
        static_for<NU>([&](auto uc) { read_unit(pfa, qfa, smem, std::integral_constant<int, 0>{}, uc); });
    }
    // One substep: its 4 NM MFMAs out of set x, part-major (consecutive MFMAs write different accumulators when the
    // wave has more than one); the fragments of the following substep are requested into set y, one behind each of
    // the first MFMAs (a single-tile wave requests both in front of the first), and `extra(m)` runs behind MFMA m.
    auto substep = [&](const uint4(&xp)[TP], const uint4(&xq)[TQ], uint4(&yp)[TP], uint4(&yq)[TQ],
                       const unsigned char *stage, auto sc, auto &&extra) {
        static_for<SLOTS>([&](auto mc) {
            constexpr int m = decltype(mc)::value, e = m / NM, n = m % NM, i = n / TQ, j = n % TQ;
            if constexpr (NM == 1 && m == 0) static_for<NU>([&](auto uc) { read_unit(yp, yq, stage, sc, uc); });
            Mma<T>::template part<e>(acc[i][j], xp[i], xq[j]);
            if constexpr (NM > 1 && m < NU) read_unit(yp, yq, stage, sc, mc);
            extra(mc);
            __builtin_amdgcn_sched_barrier(0);
        });
    };
    auto nothing = [](auto) {};
    for (int kt = 0; kt < KT; ++kt) {
        const unsigned char *cur = smem + (kt % NS) * STAGE_BYTES;
        const unsigned char *nxt = smem + ((kt + 1) % NS) * STAGE_BYTES;
        // the wave's LPW loads of k-tile kt + AHEAD, spread between the MFMAs of one substep
        auto requests = [&](auto mc) {
            constexpr int m = decltype(mc)::value, LA = m * LPW / SLOTS, LB = (m + 1) * LPW / SLOTS;
            static_for<LB - LA>([&](auto tc) { request_one(kt + AHEAD, std::integral_constant<int, LA + decltype(tc)::value>{}); });
        };
        if constexpr (EARLY) substep(pfa, qfa, pfb, qfb, cur, std::integral_constant<int, 1>{}, requests);
        else substep(pfa, qfa, pfb, qfb, cur, std::integral_constant<int, 1>{}, nothing);
        if constexpr (SPW == 4) {
            substep(pfb, qfb, pfa, qfa, cur, std::integral_constant<int, 2>{}, nothing);
            substep(pfa, qfa, pfb, qfb, cur, std::integral_constant<int, 3>{}, nothing);
        }
        // k-tile kt + 1 becomes visible: this wave's loads of it have landed (those of the NS - 2 k-tiles after it may
        // still be in flight), every fragment of `cur` has been read, and the barrier says the same of the other waves.
        // Then the first fragments of k-tile kt + 1 between the last MFMAs of this one (and, with two stages, the loads
        // of k-tile kt + 2 into the stage that has just been left).
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(INFLIGHT) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if constexpr (EARLY) substep(pfb, qfb, pfa, qfa, nxt, std::integral_constant<int, 0>{}, nothing);
        else substep(pfb, qfb, pfa, qfa, nxt, std::integral_constant<int, 0>{}, requests);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the requests past the last k-tile
    if (rem > 0) {
        // The shorter last k-tile, outside the pipeline (one load latency per workgroup, once): the same direct loads
        // into stage 0, lanes whose 16 bytes lie at k >= K reading zeros instead (in both operands, so the products
        // vanish whatever follows the end of a row), then every substep of the wave's share out of one fragment set.
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();  // nobody reads a stage any more
        asm volatile("" ::: "memory");
        auto below = [&](auto opc, auto modec, int inst) {
            typedef typename decltype(opc)::type Op;
            if constexpr (decltype(modec)::value == LD_K) {
                const int row = inst * 8 + (lane >> 3);
                return (((lane & 7) ^ (int)swz((uint32_t)row)) * 4) < rem;
            } else {
                return inst * Op::KRPI + lane / (64 / Op::KRPI) < rem;
            }
        };
        static_for<LPW>([&](auto lc) {
            constexpr int l = decltype(lc)::value;
            if constexpr (l < LPWP) {
                const bool in = below(std::common_type<OpP>{}, std::integral_constant<int, LP>{}, wave * LPWP + l);
                direct_load16(in ? (const void *)(gp[l] + (int64_t)KT * stepP) : (const void *)kZeroChunkF32, smem_addr + lp[l]);
            } else {
                const bool in = below(std::common_type<OpQ>{}, std::integral_constant<int, LQ>{}, wave * LPWQ + (l - LPWP));
                direct_load16(in ? (const void *)(gq[l - LPWP] + (int64_t)KT * stepQ) : (const void *)kZeroChunkF32,
                              smem_addr + OpP::BYTES + lq[l - LPWP]);
            }
        });
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        static_for<SPW>([&](auto sc) {
            static_for<NU>([&](auto uc) { read_unit(pfa, qfa, smem, sc, uc); });
            static_for<SLOTS>([&](auto mc) {
                constexpr int m = decltype(mc)::value, e = m / NM, n = m % NM, i = n / TQ, j = n % TQ;
                Mma<T>::template part<e>(acc[i][j], pfa[i], qfa[j]);
            });
        });
    }
    if constexpr (KS == 2) {
        // the second half's partial sums go to the first half through LDS: [tile][i][j][r][lane], 4 bytes each
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();  // nobody reads a stage any more
        asm volatile("" ::: "memory");
        float *xch = (float *)smem + ((wave & 3) * TP * TQ * 16) * 64 + lane;
        static_assert(4 * TP * TQ * 16 * 64 * 4 <= Geo_::SMEM_BYTES, "the partial sums must fit in the stages");
        if (kh == 1) {
#pragma unroll
            for (int i = 0; i < TP; ++i)
#pragma unroll
                for (int j = 0; j < TQ; ++j)
#pragma unroll
                    for (int r = 0; r < 16; ++r) xch[((i * TQ + j) * 16 + r) * 64] = acc[i][j][r];
        }
        __syncthreads();
        if (kh == 1) return;
#pragma unroll
        for (int i = 0; i < TP; ++i)
#pragma unroll
            for (int j = 0; j < TQ; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] += xch[((i * TQ + j) * 16 + r) * 64];
    }

    store_tile<T, TP, TQ>(g, acc, p0, q0, wp, wq, lane, split);
}

}  // namespace gemm
}  // namespace agh

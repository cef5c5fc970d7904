// f32 GEMM for small problems on gfx950: 64 x 64 tiles whose operand tiles go from global memory straight into
// LDS (global_load_lds_dwordx4), four k-tiles in flight.  A 64 x 64 tile is sixteen MFMAs per wave and k-tile;
// staged through registers, the loads' address arithmetic and the LDS writes cost as much again
// (agh_gemm_kernel.h).  Here a k-tile is sixteen MFMAs, the fragment reads, four direct loads and one barrier.
//
// Same formulation as agh_gemm_kernel.h: D[p][q] = sum_k P[p][k] * Q[q][k] on v_mfma_f32_32x32x2_f32, four waves
// in a 2 x 2 grid, a wave owns one 32 x 32 tile.  Lane l supplies row l % 32 and, in substep s (8 k) of a k-tile
// (32 k), the four k values 8 s + 4 (l / 32) + e, e = 0..3, one per MFMA.
//
// LDS image of an operand's 64 rows x 32 k:
//   LD_K (k contiguous in memory): [row][32 k], 128-byte rows, 16-byte chunk c of row r at slot c ^ swz(r): the
//        layout and the fragment read (one ds_read_b128) of agh_gemm_kernel.h.  A direct load deposits lane L's
//        16 bytes at base + 16 L, so the swizzle is applied on the global side.
//   LD_R (rows contiguous in memory): [k][64 rows], 256 bytes per k-row, four k-rows per direct load.  The image
//        of a load starts kBlock = 1152 bytes after the one before: the two half-waves of a fragment read (k-rows
//        four apart, i.e. neighbouring loads) then fall on the two halves of the banks.  Fragment = four
//        ds_read_b32, 256 bytes apart.
//
// Requirements checked by the host: K and every split's k range multiples of 32, operand base pointers 16-byte
// aligned, unit stride along k (LD_K) or along rows (LD_R) with the other stride a multiple of 4 elements, rows a
// multiple of 4 for LD_R.
#pragma once
#include "agh_gemm_bf16_dl.h"

namespace agh {
namespace gemm {

template <int LP, int LQ>
__global__ __launch_bounds__(256) void gemm_f32_dl_kernel(Args g) {
    typedef float T;
    static_assert((LP == LD_K || LP == LD_R) && (LQ == LD_K || LQ == LD_R), "vector layouts only");
    constexpr int BP = 64, BQ = 64, BK = 32, NS = 4;
    constexpr int kBlock = 1152;                    // LDS bytes between the images of consecutive direct loads (LD_R)
    constexpr int OP_BYTES = 8 * kBlock;            // one operand of one stage (LD_K uses 8192 of them)
    constexpr int STAGE_BYTES = 2 * OP_BYTES;
    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wp = wave & 1, wq = wave >> 1;
    int tp, tq;
    tile_coords(blockIdx.x, g.tiles_p, g.tiles_q, tp, tq);
    const int p0 = tp * BP, q0 = tq * BQ;
    const int split = blockIdx.y;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int KT = kend > kbeg ? (kend - kbeg) / BK : 0;

    // ---- the wave's direct loads: two per operand and k-tile (instructions 2 wave, 2 wave + 1 of the operand's 8) ----
    // per-lane global address for k-tile 0, LDS offset of the instruction's image inside the operand, bytes per k-tile
    const unsigned char *gp[2], *gq[2];
    uint32_t lp[2], lq[2];
    auto setup = [&](auto modec, const void *base, int64_t rs, int64_t ks, int64_t batch_off, int r0, int NR,
                     const unsigned char *(&gptr)[2], uint32_t (&loff)[2], int64_t &kstep) {
        constexpr int MODE = decltype(modec)::value;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int inst = wave * 2 + i;
            int64_t off;
            if constexpr (MODE == LD_K) {
                const int row = inst * 8 + (lane >> 3);
                const int c = (lane & 7) ^ (int)swz((uint32_t)row);
                const int rowg = min(r0 + row, NR - 1);
                off = (int64_t)rowg * rs + kbeg + c * 4;
                loff[i] = (uint32_t)inst * 1024u;
            } else {
                const int kr = inst * 4 + (lane >> 4);
                int rowg = r0 + (lane & 15) * 4;
                if (rowg >= NR) rowg = NR - 4;  // NR is a multiple of 4 on this path
                off = (int64_t)(kbeg + kr) * ks + rowg;
                loff[i] = (uint32_t)inst * kBlock;
            }
            gptr[i] = (const unsigned char *)base + (off + batch_off) * 4;
        }
        kstep = (MODE == LD_K ? (int64_t)BK : (int64_t)BK * ks) * 4;
    };
    int64_t stepP, stepQ;
    setup(std::integral_constant<int, LP>{}, g.P, g.ps, g.pk, (int64_t)blockIdx.z * g.batch_p, p0, g.NP, gp, lp, stepP);
    setup(std::integral_constant<int, LQ>{}, g.Q, g.qs, g.qk, (int64_t)blockIdx.z * g.batch_q, q0, g.NQ, gq, lq, stepQ);
    const uint32_t smem_addr = __builtin_amdgcn_readfirstlane(lds_address(smem));
    // requests k-tile t (clamped to the last: the image is then never read) into its stage
    auto request = [&](int t) {
        const int tc = min(t, KT - 1);
        const uint32_t st = smem_addr + (uint32_t)(t & (NS - 1)) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 2; ++i) direct_load16(gp[i] + (int64_t)tc * stepP, st + lp[i]);
#pragma unroll
        for (int i = 0; i < 2; ++i) direct_load16(gq[i] + (int64_t)tc * stepQ, st + OP_BYTES + lq[i]);
    };

    // ---- fragment reads: lane l supplies row l % 32, k = 8 s + 4 (l / 32) + e ----
    const uint32_t lrow = lane & 31, lg = lane >> 5;
    auto frag_offset = [&](auto modec, int wave_row) -> uint32_t {
        constexpr int MODE = decltype(modec)::value;
        if constexpr (MODE == LD_K) {
            const uint32_t r = (uint32_t)wave_row + lrow;
            return r * 128u + ((lg ^ swz(r)) << 4);  // substep s toggles bit 5
        } else {
            return lg * kBlock + ((uint32_t)wave_row + lrow) * 4u;  // substep s adds 2 kBlock
        }
    };
    const uint32_t fp = frag_offset(std::integral_constant<int, LP>{}, wp * 32);
    const uint32_t fq = frag_offset(std::integral_constant<int, LQ>{}, wq * 32);
    auto frag_read = [&](auto modec, const unsigned char *op, uint32_t off, int s) -> uint4 {
        constexpr int MODE = decltype(modec)::value;
        if constexpr (MODE == LD_K) {
            return *(const uint4 *)(op + (off ^ (uint32_t)(s << 5)));
        } else {
            const unsigned char *p = op + off + s * 2 * kBlock;
            return make_uint4(*(const uint32_t *)p, *(const uint32_t *)(p + 256), *(const uint32_t *)(p + 512),
                              *(const uint32_t *)(p + 768));
        }
    };

    f32x16 acc[1][1];
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[0][0][r] = 0.0f;

    if (KT > 0) {
        request(0);
        request(1);
        request(2);
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // this wave's part of k-tile 0 has landed
        __builtin_amdgcn_s_barrier();                     // and everybody else's
        asm volatile("" ::: "memory");
    }
    uint4 pa, qa, pb, qb;  // fragment sets of even and odd substeps
    if (KT > 0) {
        pa = frag_read(std::integral_constant<int, LP>{}, smem, fp, 0);
        qa = frag_read(std::integral_constant<int, LQ>{}, smem + OP_BYTES, fq, 0);
    }
    for (int kt = 0; kt < KT; ++kt) {
        const unsigned char *cur = smem + (kt & (NS - 1)) * STAGE_BYTES;
        const unsigned char *nxt = smem + ((kt + 1) & (NS - 1)) * STAGE_BYTES;
        // substep 0: request k-tile kt + 3 into the stage k-tile kt - 1 has left (the barrier that ended it is behind us)
        pb = frag_read(std::integral_constant<int, LP>{}, cur, fp, 1);
        qb = frag_read(std::integral_constant<int, LQ>{}, cur + OP_BYTES, fq, 1);
        request(kt + 3);
        Mma<T>::template part<0>(acc[0][0], pa, qa);
        Mma<T>::template part<1>(acc[0][0], pa, qa);
        Mma<T>::template part<2>(acc[0][0], pa, qa);
        Mma<T>::template part<3>(acc[0][0], pa, qa);
        __builtin_amdgcn_sched_barrier(0);
        // substep 1
        pa = frag_read(std::integral_constant<int, LP>{}, cur, fp, 2);
        qa = frag_read(std::integral_constant<int, LQ>{}, cur + OP_BYTES, fq, 2);
        Mma<T>::template part<0>(acc[0][0], pb, qb);
        Mma<T>::template part<1>(acc[0][0], pb, qb);
        Mma<T>::template part<2>(acc[0][0], pb, qb);
        Mma<T>::template part<3>(acc[0][0], pb, qb);
        __builtin_amdgcn_sched_barrier(0);
        // substep 2
        pb = frag_read(std::integral_constant<int, LP>{}, cur, fp, 3);
        qb = frag_read(std::integral_constant<int, LQ>{}, cur + OP_BYTES, fq, 3);
        Mma<T>::template part<0>(acc[0][0], pa, qa);
        Mma<T>::template part<1>(acc[0][0], pa, qa);
        Mma<T>::template part<2>(acc[0][0], pa, qa);
        Mma<T>::template part<3>(acc[0][0], pa, qa);
        __builtin_amdgcn_sched_barrier(0);
        // substep 3: k-tile kt + 1 becomes visible (two later k-tiles, eight loads of this wave, may still be in flight;
        // every fragment of `cur` has been read), its first fragments are requested, then the last MFMAs of this one
        asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        pa = frag_read(std::integral_constant<int, LP>{}, nxt, fp, 0);
        qa = frag_read(std::integral_constant<int, LQ>{}, nxt + OP_BYTES, fq, 0);
        Mma<T>::template part<0>(acc[0][0], pb, qb);
        Mma<T>::template part<1>(acc[0][0], pb, qb);
        Mma<T>::template part<2>(acc[0][0], pb, qb);
        Mma<T>::template part<3>(acc[0][0], pb, qb);
        __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the requests past the last k-tile

    store_tile<T, 1, 1>(g, acc, p0, q0, wp, wq, lane, split);
}

}  // namespace gemm
}  // namespace agh

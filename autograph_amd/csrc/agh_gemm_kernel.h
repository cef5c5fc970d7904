// MFMA GEMM for gfx950 behind agh_gemm_{f32,bf16}[_bias_act].
//
// Formulation.  The host rewrites C = alpha*A*B + beta*C as
//     D[p][q] = sum_k P[p][k] * Q[q][k]
// where P and Q are the two operands seen as "row index x k" matrices with arbitrary
// signed element strides (row stride rs, k stride ks).  Which of A, B becomes P is chosen
// so that p runs along the unit-stride axis of C: the 32x32 MFMA accumulator holds four
// consecutive p per lane, so C is written with 8/16-byte stores.  Transposed views are
// therefore never materialised; they only change which loader a side uses:
//     LD_K  k is unit stride      -> 16-byte global loads along k
//     LD_R  rows are unit stride  -> 16-byte global loads along rows + in-register transpose
//     LD_S  anything else         -> guarded element loads (any stride, any size)
//
// LDS layout (both operands, both element types): tile rows of 128 bytes = 8 chunks of 16
// bytes (64 bf16 or 32 f32 of k).  Chunk c of row r lives at chunk slot c ^ swz(r) with
// swz(r) = (r & 7) ^ ((r >> 3) & 1): sixteen consecutive rows reading the same logical
// chunk touch sixteen different 16-byte bank groups, whether the LDS is viewed as 32 or
// as 64 banks wide, and so do the 8-lane row writes of the loaders.
//
// MFMA operand mapping.  A 16-byte chunk is exactly one lane's operand:
//   bf16: v_mfma_f32_32x32x16_bf16, lane l supplies row l%32, the 8 k of chunk 2s + l/32.
//   f32 : v_mfma_f32_32x32x2_f32 four times per chunk pair; MFMA e takes element e of the
//         chunk, i.e. k = {4(2s)+e, 4(2s+1)+e} - a permutation of k that is the same on
//         both operands, so the dot products are unchanged.
// Accumulator element r of lane l is D[p0 + 8*(r/4) + 4*(l/32) + r%4][q0 + l%32].
//
// Pipeline: global loads for k-tile t+1 are issued into registers before the MFMA loop
// over k-tile t, and written to the other LDS stage after it; one barrier per k-tile.
#pragma once
#include <utility>

#include "agh_internal.h"

namespace agh {
namespace gemm {

typedef float f32x16 __attribute__((ext_vector_type(16)));

// Compile-time loop: the body is instantiated once per index, so accumulator registers are
// only ever named by constants no matter how large the unrolled code gets (a `#pragma unroll`
// loop that exceeds the unroller's size budget silently stays a loop, and an accumulator
// array indexed by a loop variable is demoted to scratch memory).
template <int... Is, typename F>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, Is...>, F &&f) {
    (f(std::integral_constant<int, Is>{}), ...);
}
template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, static_cast<F &&>(f));
}
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

enum { LD_K = 0, LD_R = 1, LD_S = 2 };
enum { ST_SCALAR = 0, ST_VEC = 1, ST_SPLITK = 2, ST_STAGED = 3 };  // ST_STAGED: direct-to-LDS bf16 kernel only

struct Args {
    const void *P;
    const void *Q;
    void *D;
    const void *bias;
    float *ws;  // split-K partials [splits][NQ][NPpad]
    int64_t ps, pk, qs, qk, dp, dq, bias_stride;
    int64_t batch_p, batch_q, batch_d;  // element strides between consecutive matrices (grid.z = batch)
    int NP, NQ, K, NPpad, batch;
    int tiles_p, tiles_q;
    int k_per_split;  // multiple of the k-tile
    float alpha, beta;
    int bias_on_p, has_bias, act;
    int store_mode;
};

template <typename T> struct Geo;
template <> struct Geo<uint16_t> { static constexpr int EPC = 8; };
template <> struct Geo<float> { static constexpr int EPC = 4; };

__device__ __forceinline__ uint32_t swz(uint32_t r) { return (r & 7u) ^ ((r >> 3) & 1u); }
__device__ __forceinline__ uint32_t lds_off(uint32_t r, uint32_t c) { return r * 128u + ((c ^ swz(r)) << 4); }

// ---- epilogue arithmetic in the order the reference's separate ops round ----
template <typename T>
__device__ __forceinline__ T finish(float acc, float alpha, float beta, T cold, bool has_bias, T bias, int act) {
    // selects only: a branch per output element would dominate the epilogue
    const float v0 = alpha * acc;
    const float v1 = v0 + beta * Elem<T>::to_f32(cold);
    T r = Elem<T>::from_f32(beta != 0.0f ? v1 : v0);  // beta == 0 never uses C (and keeps the sign of a zero)
    const T rb = Elem<T>::from_f32(Elem<T>::to_f32(bias) + Elem<T>::to_f32(r));
    r = has_bias ? rb : r;
    const bool neg = !(Elem<T>::to_f32(r) >= 0.0f);
    return (act == AGH_ACT_RELU && neg) ? Elem<T>::zero() : r;
}
// alpha only (no C, no bias, no activation): the plain `dot` epilogue
template <typename T>
__device__ __forceinline__ T finish_plain(float acc, float alpha) {
    return Elem<T>::from_f32(alpha * acc);
}

// ---- global -> register loaders (one operand tile of BR rows x 8 chunks) ----
template <typename T, int MODE, int BR, int NT>
struct Loader {
    static constexpr int EPC = Geo<T>::EPC;
    static constexpr int TOTAL = BR * 8;                   // chunks in the tile
    static constexpr int NREG = (TOTAL + NT - 1) / NT;     // 16-byte registers per thread
    static constexpr int NBLK_TOTAL = 8 * (BR / EPC);      // LD_R: EPC x EPC blocks in the tile
    static constexpr int NBLK = (NBLK_TOTAL + NT - 1) / NT;

    // A tile is moved in NPIECE independent pieces (one 16-byte register, or one EPC x EPC block for LD_R), so
    // that the kernel can hand them out between MFMAs instead of issuing a burst.
    static constexpr int NPIECE = MODE == LD_R ? NBLK : NREG;
    typedef uint4 Regs[NREG > NBLK * EPC ? NREG : NBLK * EPC];

    // base: element pointer of the operand; r0: first tile row; NR: rows in the operand;
    // k0: first k of the tile; kend: one past the last valid k.
    // LD_K and LD_R pieces are loaded UNCONDITIONALLY from clamped addresses and the k tail is zeroed when the
    // piece is stored: no branch surrounds a load (behind a branch the compiler can no longer count the loads
    // in flight and waits for all of them), and nothing touches the loaded value before it is needed.
    static __device__ __forceinline__ void load(Regs &reg, const T *base, int64_t rs, int64_t ks, int r0, int NR, int k0,
                                                int kend, int tid) {
        static_for<NPIECE>([&](auto ic) { load_piece<decltype(ic)::value>(reg, base, rs, ks, r0, NR, k0, kend, tid); });
    }
    template <int i>
    static __device__ __forceinline__ void load_piece(Regs &reg, const T *base, int64_t rs, int64_t ks, int r0, int NR,
                                                      int k0, int kend, int tid) {
        if constexpr (MODE == LD_K) {
            const int id = min(tid + i * NT, TOTAL - 1);
            const int r = id >> 3, c = id & 7;
            const int row = min(r0 + r, NR - 1);
            const int kk = min(k0 + c * EPC, kend - EPC);  // K is a multiple of EPC here
            reg[i] = *(const uint4 *)(base + (int64_t)row * rs + kk);
        } else if constexpr (MODE == LD_R) {
            const int id = min(tid + i * NT, NBLK_TOTAL - 1);
            const int kb = id & 7, rb = id >> 3;
            int row = r0 + rb * EPC;
            if (row >= NR) row = NR - EPC;  // NR is a multiple of EPC on this path
#pragma unroll
            for (int e = 0; e < EPC; ++e) {
                const int kk = min(k0 + kb * EPC + e, kend - 1);
                reg[i * EPC + e] = *(const uint4 *)(base + (int64_t)kk * ks + row);
            }
        } else {
            int id = tid + i * NT;
            int r = id >> 3, c = id & 7;
            int row = r0 + r;
            bool rok = (TOTAL % NT == 0 || id < TOTAL) && row < NR;
            const T *src = base + (int64_t)row * rs;
            T tmp[EPC];
#pragma unroll
            for (int e = 0; e < EPC; ++e) {
                int kk = k0 + c * EPC + e;
                T v = 0;
                if (rok && kk < kend) v = src[(int64_t)kk * ks];
                tmp[e] = v;
            }
            uint4 v;
            if constexpr (sizeof(T) == 2) {
                v.x = (uint32_t)tmp[0] | ((uint32_t)tmp[1] << 16);
                v.y = (uint32_t)tmp[2] | ((uint32_t)tmp[3] << 16);
                v.z = (uint32_t)tmp[4] | ((uint32_t)tmp[5] << 16);
                v.w = (uint32_t)tmp[6] | ((uint32_t)tmp[7] << 16);
            } else {
                v.x = __float_as_uint(tmp[0]);
                v.y = __float_as_uint(tmp[1]);
                v.z = __float_as_uint(tmp[2]);
                v.w = __float_as_uint(tmp[3]);
            }
            reg[i] = v;
        }
    }

    // The same for a k-tile that lies wholly inside [kbeg, kend): no clamp on k, and the address is written as a
    // per-lane part that does not change from k-tile to k-tile plus a wave-uniform part in k0, so that a piece costs
    // one or two vector instructions instead of a 64-bit multiply per load (vector loaders only).
    template <int i>
    static __device__ __forceinline__ void load_piece_full(Regs &reg, const T *base, int64_t rs, int64_t ks, int r0, int NR,
                                                           int k0, int tid) {
        static_assert(MODE == LD_K || MODE == LD_R, "vector loaders only");
        if constexpr (MODE == LD_K) {
            const int id = min(tid + i * NT, TOTAL - 1);
            const int r = id >> 3, c = id & 7;
            const int row = min(r0 + r, NR - 1);
            const T *lane_base = base + (int64_t)row * rs + c * EPC;
            reg[i] = *(const uint4 *)(lane_base + k0);
        } else {
            const int id = min(tid + i * NT, NBLK_TOTAL - 1);
            const int kb = id & 7, rb = id >> 3;
            int row = r0 + rb * EPC;
            if (row >= NR) row = NR - EPC;  // NR is a multiple of EPC on this path
            const T *lane_base = base + row + (int64_t)(kb * EPC) * ks;
            const T *p = lane_base + (int64_t)k0 * ks;
#pragma unroll
            for (int e = 0; e < EPC; ++e) reg[i * EPC + e] = *(const uint4 *)(p + (int64_t)e * ks);
        }
    }

    // registers -> LDS stage (tile base address `lds`, bytes); k0 / kend as given to load
    static __device__ __forceinline__ void store(const Regs &reg, unsigned char *lds, int k0, int kend, int tid) {
        static_for<NPIECE>([&](auto ic) { store_piece<decltype(ic)::value>(reg, lds, k0, kend, tid); });
    }
    // FULL: the k-tile lies wholly below kend, nothing to zero
    template <int i, bool FULL = false>
    static __device__ __forceinline__ void store_piece(const Regs &reg, unsigned char *lds, int k0, int kend, int tid) {
        if constexpr (MODE == LD_R) {
            int id = tid + i * NT;
            int kb = id & 7, rb = id >> 3;
            if (!(NBLK_TOTAL % NT == 0 || id < NBLK_TOTAL)) return;
            uint4 in[EPC];  // in[e] = EPC rows at k = kb*EPC + e
#pragma unroll
            for (int e = 0; e < EPC; ++e) {
                const bool ok = FULL || k0 + kb * EPC + e < kend;
                const uint4 &src = reg[i * EPC + e];
                in[e] = make_uint4(ok ? src.x : 0u, ok ? src.y : 0u, ok ? src.z : 0u, ok ? src.w : 0u);
            }
            if constexpr (sizeof(T) == 4) {
                // 4x4 transpose of 32-bit values: pure register renaming
                uint4 o0 = make_uint4(in[0].x, in[1].x, in[2].x, in[3].x);
                uint4 o1 = make_uint4(in[0].y, in[1].y, in[2].y, in[3].y);
                uint4 o2 = make_uint4(in[0].z, in[1].z, in[2].z, in[3].z);
                uint4 o3 = make_uint4(in[0].w, in[1].w, in[2].w, in[3].w);
                uint32_t r = rb * 4;
                *(uint4 *)(lds + lds_off(r + 0, kb)) = o0;
                *(uint4 *)(lds + lds_off(r + 1, kb)) = o1;
                *(uint4 *)(lds + lds_off(r + 2, kb)) = o2;
                *(uint4 *)(lds + lds_off(r + 3, kb)) = o3;
            } else {
                // 8x8 transpose of 16-bit values: one half-word interleave per output word,
                // the 32- and 64-bit levels are register renaming
                uint32_t w[8][4];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const uint4 &s = in[e];
                    w[e][0] = s.x; w[e][1] = s.y; w[e][2] = s.z; w[e][3] = s.w;
                }
                uint32_t r = rb * 8;
#pragma unroll
                for (int rr = 0; rr < 8; ++rr) {
                    uint32_t o[4];
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        uint32_t lo = w[2 * q][rr >> 1], hi = w[2 * q + 1][rr >> 1];
                        o[q] = (rr & 1) ? ((lo >> 16) | (hi & 0xFFFF0000u)) : ((lo & 0xFFFFu) | (hi << 16));
                    }
                    *(uint4 *)(lds + lds_off(r + rr, kb)) = make_uint4(o[0], o[1], o[2], o[3]);
                }
            }
        } else {
            int id = tid + i * NT;
            int r = id >> 3, c = id & 7;
            const bool ok = FULL || MODE != LD_K || k0 + c * EPC < kend;
            const uint4 v = make_uint4(ok ? reg[i].x : 0u, ok ? reg[i].y : 0u, ok ? reg[i].z : 0u, ok ? reg[i].w : 0u);
            if (TOTAL % NT == 0 || id < TOTAL) *(uint4 *)(lds + lds_off(r, c)) = v;
        }
    }
};

// One MFMA group = all the MFMAs that consume one 16-byte fragment pair: a single 32x32x16 for bf16, four
// 32x32x2 for f32 (PARTS).  `part` lets a caller walk the parts of many accumulators in turn, so that
// consecutive MFMAs never accumulate into the same registers (a dependent MFMA waits for its predecessor).
template <typename T> struct Mma;
template <> struct Mma<uint16_t> {
    static constexpr int PARTS = 1;
    static __device__ __forceinline__ void run(f32x16 &acc, const uint4 &a, const uint4 &b) {
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                      acc, 0, 0, 0);
    }
    template <int E> static __device__ __forceinline__ void part(f32x16 &acc, const uint4 &a, const uint4 &b) { run(acc, a, b); }
};
template <> struct Mma<float> {
    static constexpr int PARTS = 4;
    template <int E> static __device__ __forceinline__ void part(f32x16 &acc, const uint4 &a, const uint4 &b) {
        const uint32_t ae = E == 0 ? a.x : E == 1 ? a.y : E == 2 ? a.z : a.w;
        const uint32_t be = E == 0 ? b.x : E == 1 ? b.y : E == 2 ? b.z : b.w;
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(ae), __uint_as_float(be), acc, 0, 0, 0);
    }
    static __device__ __forceinline__ void run(f32x16 &acc, const uint4 &a, const uint4 &b) {
        part<0>(acc, a, b);
        part<1>(acc, a, b);
        part<2>(acc, a, b);
        part<3>(acc, a, b);
    }
};

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.  Give every XCD a
// contiguous run of tile ids, and walk tiles in panels of GROUP_P tile rows so that tiles
// running together on an XCD share operand panels.
__device__ __forceinline__ void tile_coords(int bid, int tiles_p, int tiles_q, int &tp, int &tq) {
    const int nb = tiles_p * tiles_q;
    int id = bid;
    if ((nb & 7) == 0) id = (bid & 7) * (nb >> 3) + (bid >> 3);
    constexpr int GROUP_P = 8;
    const int per_group = GROUP_P * tiles_q;
    const int group = id / per_group;
    const int first_p = group * GROUP_P;
    const int gsz = min(tiles_p - first_p, GROUP_P);
    const int in_group = id - group * per_group;
    tp = first_p + in_group % gsz;
    tq = in_group / gsz;
}

// ------------------------------------------------------------ epilogue ----
// Stores a wave's TP x TQ tiles of 32 x 32 accumulators (element r of lane l of tile (i, j) is
// D[p0 + 32 (wp TP + i) + 8 (r / 4) + 4 (l / 32) + r % 4][q0 + 32 (wq TQ + j) + l % 32]).  One loop nest per store
// mode, each small enough to unroll fully: the accumulators must only ever be indexed by compile-time constants
// or they would be demoted to scratch.
template <typename T, int TP, int TQ>
__device__ __forceinline__ void store_tile(const Args &g, const f32x16 (&acc)[TP][TQ], int p0, int q0, int wp, int wq,
                                           int lane, int split) {
    const uint32_t lrow = lane & 31, lg = lane >> 5;
    const int pw0 = p0 + wp * TP * 32 + (int)lg * 4, qw0 = q0 + wq * TQ * 32 + (int)lrow;
    T *D = (T *)g.D + (int64_t)blockIdx.z * g.batch_d;
    const T *bias = (const T *)g.bias;
    const int mode = g.store_mode;
    const bool has_bias = g.has_bias != 0, bias_p = g.bias_on_p != 0;
    if (mode == ST_SPLITK) {
        static_for<TQ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int q = qw0 + j * 32;
            float *wrow = g.ws + ((size_t)split * g.NQ + q) * g.NPpad;
            static_for<TP>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                static_for<4>([&](auto bc) {
                    constexpr int blk = decltype(bc)::value;
                    const int p = pw0 + i * 32 + blk * 8;
                    if (q < g.NQ && p < g.NPpad)
                        *(float4 *)(wrow + p) = make_float4(acc[i][j][blk * 4 + 0], acc[i][j][blk * 4 + 1],
                                                            acc[i][j][blk * 4 + 2], acc[i][j][blk * 4 + 3]);
                });
            });
        });
    } else if (mode == ST_VEC) {
        static_for<TQ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int q = qw0 + j * 32;
            const bool qok = q < g.NQ;
            T bq = 0;
            if (qok && has_bias && !bias_p) bq = bias[(int64_t)q * g.bias_stride];
            T *drow = D + (int64_t)q * g.dq;
            static_for<TP>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                static_for<4>([&](auto bc) {
                    constexpr int blk = decltype(bc)::value;
                    const int p = pw0 + i * 32 + blk * 8;
                    if (qok && p < g.NP) {  // NP is a multiple of 4 on this path
                        T *dst = drow + p;
                        __align__(16) T old[4] = {0, 0, 0, 0};
                        if (g.beta != 0.0f) {
                            if constexpr (sizeof(T) == 4) *(uint4 *)old = *(const uint4 *)dst;
                            else *(uint2 *)old = *(const uint2 *)dst;
                        }
                        T b0 = bq, b1 = bq, b2 = bq, b3 = bq;
                        if (has_bias && bias_p) {
                            b0 = bias[(int64_t)(p + 0) * g.bias_stride];
                            b1 = bias[(int64_t)(p + 1) * g.bias_stride];
                            b2 = bias[(int64_t)(p + 2) * g.bias_stride];
                            b3 = bias[(int64_t)(p + 3) * g.bias_stride];
                        }
                        __align__(16) T out[4];
                        out[0] = finish<T>(acc[i][j][blk * 4 + 0], g.alpha, g.beta, old[0], has_bias, b0, g.act);
                        out[1] = finish<T>(acc[i][j][blk * 4 + 1], g.alpha, g.beta, old[1], has_bias, b1, g.act);
                        out[2] = finish<T>(acc[i][j][blk * 4 + 2], g.alpha, g.beta, old[2], has_bias, b2, g.act);
                        out[3] = finish<T>(acc[i][j][blk * 4 + 3], g.alpha, g.beta, old[3], has_bias, b3, g.act);
                        if constexpr (sizeof(T) == 4) *(uint4 *)dst = *(const uint4 *)out;
                        else *(uint2 *)dst = *(const uint2 *)out;
                    }
                });
            });
        });
    } else {
        static_for<TQ>([&](auto jc) {
            constexpr int j = decltype(jc)::value;
            const int q = qw0 + j * 32;
            const bool qok = q < g.NQ;
            T bq = 0;
            if (qok && has_bias && !bias_p) bq = bias[(int64_t)q * g.bias_stride];
            T *drow = D + (int64_t)q * g.dq;
            static_for<TP>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                static_for<16>([&](auto rc) {
                    constexpr int r = decltype(rc)::value;
                    const int p = pw0 + i * 32 + (r >> 2) * 8 + (r & 3);
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

template <typename T, int BP, int BQ, int WGP, int WGQ, int LP, int LQ>
__global__ __launch_bounds__(WGP *WGQ * 64) void gemm_kernel(Args g) {
    constexpr int NT = WGP * WGQ * 64;
    constexpr int EPC = Geo<T>::EPC;
    constexpr int BK = 8 * EPC;
    constexpr int TP = BP / WGP / 32, TQ = BQ / WGQ / 32;
    static_assert(TP >= 1 && TQ >= 1, "wave tile must hold at least one 32x32 MFMA tile");
    constexpr int STAGE_BYTES = (BP + BQ) * 128;
    typedef Loader<T, LP, BP, NT> LdP;
    typedef Loader<T, LQ, BQ, NT> LdQ;
    constexpr int NRP = LdP::NREG > LdP::NBLK * EPC ? LdP::NREG : LdP::NBLK * EPC;
    constexpr int NRQ = LdQ::NREG > LdQ::NBLK * EPC ? LdQ::NREG : LdQ::NBLK * EPC;

    extern __shared__ __align__(16) unsigned char smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wp = wave % WGP, wq = wave / WGP;
    int tp, tq;
    tile_coords(blockIdx.x, g.tiles_p, g.tiles_q, tp, tq);
    const int p0 = tp * BP, q0 = tq * BQ;
    const int split = blockIdx.y;
    const int kbeg = split * g.k_per_split;
    const int kend = min(g.K, kbeg + g.k_per_split);
    const int KT = kend > kbeg ? (kend - kbeg + BK - 1) / BK : 0;

    const T *P = (const T *)g.P + (int64_t)blockIdx.z * g.batch_p;
    const T *Q = (const T *)g.Q + (int64_t)blockIdx.z * g.batch_q;

    f32x16 acc[TP][TQ];
#pragma unroll
    for (int i = 0; i < TP; ++i)
#pragma unroll
        for (int j = 0; j < TQ; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;

    // Small tiles (a k-tile is a few hundred matrix-pipe cycles, far less than a trip to memory, and every CU asks
    // for a k-tile's new lines at about the same time, so somebody's request is always the first) keep NSET
    // k-tiles in flight: the loads requested during k-tile kt are those of k-tile kt + NSET and are written to LDS
    // during k-tile kt + NSET - 1, out of one of NSET sets of staging registers (two to four registers each), so a
    // load has NSET - 1/2 k-tiles to arrive instead of half of one.
    constexpr bool SPREAD = LP != LD_S && LQ != LD_S;
    constexpr bool DEEP = SPREAD && BP + BQ <= 160;
    constexpr int NSET = DEEP ? 2 : 1;  // four measured no faster than two (f32 1024^3: 29-33 us either way)
    uint4 rp[NSET][NRP], rq[NSET][NRQ];
    if (KT > 0) {
        LdP::load(rp[0], P, g.ps, g.pk, p0, g.NP, kbeg, kend, tid);
        LdQ::load(rq[0], Q, g.qs, g.qk, q0, g.NQ, kbeg, kend, tid);
        LdP::store(rp[0], smem, kbeg, kend, tid);
        LdQ::store(rq[0], smem + BP * 128, kbeg, kend, tid);
        if constexpr (DEEP) {  // k-tiles 1 .. NSET - 1 (past the last one: the last again, never used)
            static_for<NSET - 1>([&](auto sc) {
                constexpr int s = decltype(sc)::value + 1;
                const int ks = kbeg + min(s, KT - 1) * BK;
                LdP::load(rp[s], P, g.ps, g.pk, p0, g.NP, ks, kend, tid);
                LdQ::load(rq[s], Q, g.qs, g.qk, q0, g.NQ, ks, kend, tid);
            });
        }
    }
    __syncthreads();

    // per-lane read offsets: row = lane%32 inside a 32-row MFMA tile, chunk = 2s + lane/32
    const uint32_t lrow = lane & 31, lg = lane >> 5;
    const uint32_t lane_off = lrow * 128u + ((lg ^ swz(lrow)) << 4);  // tile row bases are multiples of 32

    // Fragment sets A and B alternate between substeps: while the MFMAs of substep s run out of one set,
    // the LDS reads of substep s+1 fill the other, one read after each of the first TP+TQ MFMA groups.
    // sched_barrier(0) pins that interleaving (left alone, the scheduler puts every read directly in
    // front of its first use and the matrix pipe waits out the LDS latency sixteen times per k-tile).
    constexpr int NU = TP + TQ, NM = TP * TQ;
    uint4 pfa[TP], qfa[TQ], pfb[TP], qfb[TQ];
    auto read_unit = [&](uint4(&pf)[TP], uint4(&qf)[TQ], const unsigned char *sp, const unsigned char *sq, int s, auto uc) {
        constexpr int u = decltype(uc)::value;
        const uint32_t off = lane_off ^ (uint32_t)(s << 5);
        // order of first use by the MFMA groups: P0, Q0 .. Q(TQ-1), P1 .. P(TP-1)
        if constexpr (u == 0) pf[0] = *(const uint4 *)(sp + off);
        else if constexpr (u <= TQ) qf[u - 1] = *(const uint4 *)(sq + (u - 1) * 32 * 128 + off);
        else pf[u - TQ] = *(const uint4 *)(sp + (u - TQ) * 32 * 128 + off);
    };
    constexpr int PARTS = Mma<T>::PARTS, SLOTS = NM * PARTS;
    auto phase = [&](const uint4(&xp)[TP], const uint4(&xq)[TQ], uint4(&yp)[TP], uint4(&yq)[TQ], const unsigned char *sp,
                     const unsigned char *sq, int s, auto &&after) {
        static_for<SLOTS>([&](auto mc) {  // part-major: consecutive MFMAs write different accumulators
            constexpr int m = decltype(mc)::value, e = m / NM, n = m % NM, i = n / TQ, j = n % TQ;
            // with a single MFMA tile per wave a substep is only PARTS MFMAs long: all of the next substep's
            // fragments are requested in front of its first MFMA, or the last read has half a substep to arrive
            if constexpr (NM == 1 && m == 0) static_for<NU>([&](auto uc) { read_unit(yp, yq, sp, sq, s, uc); });
            Mma<T>::template part<e>(acc[i][j], xp[i], xq[j]);
            if constexpr (NM > 1 && m < NU) read_unit(yp, yq, sp, sq, s, mc);
            after(mc);
            __builtin_amdgcn_sched_barrier(0);
        });
        static_for<(NU > NM * PARTS ? NU - NM * PARTS : 0)>([&](auto rc) {
            read_unit(yp, yq, sp, sq, s, std::integral_constant<int, NM * PARTS + decltype(rc)::value>{});
        });
    };
    const int wave_p = (wp * TP * 32) * 128, wave_q = BP * 128 + (wq * TQ * 32) * 128;
    if (KT > 0) static_for<NU>([&](auto uc) { read_unit(pfa, qfa, smem + wave_p, smem + wave_q, 0, uc); });

    // One k-tile.  With vector loaders the pieces of the next tile are requested from global memory one at a
    // time between the MFMAs of substep 0 and written to the other LDS stage between the MFMAs of substep 2
    // (a burst of loads fills the memory pipeline's queues, and a wave that cannot issue its load cannot issue
    // its next MFMA either); past the last tile the same tile is fetched again and never used.  The element
    // loader keeps its guarded loads together in front of the MFMAs.  Then the barrier publishes that
    // stage, and the last substep multiplies out of registers while the first fragments of the next tile are read.
    constexpr int NPP = LdP::NPIECE, NPT = LdP::NPIECE + LdQ::NPIECE;
    // `parc` is kt % NSET (it selects the staging register sets)
    auto ktile = [&](int kt, auto parc) {
        constexpr int LS = decltype(parc)::value;               // set the loads fill: k-tile kt's, already in LDS
        constexpr int SS = (decltype(parc)::value + 1) % NSET;  // set the stores drain: k-tile kt + 1's
        const bool more = kt + 1 < KT;
        const int k0 = kbeg + (more ? kt + 1 : kt) * BK;                   // the k-tile the stores publish
        const int kl = DEEP ? kbeg + min(kt + NSET, KT - 1) * BK : k0;      // the k-tile the loads request
        const unsigned char *cur = smem + (kt & 1) * STAGE_BYTES;
        unsigned char *nxt = smem + ((kt + 1) & 1) * STAGE_BYTES;
        if constexpr (!SPREAD) {
            if (more) {
                LdP::load(rp[0], P, g.ps, g.pk, p0, g.NP, k0, kend, tid);
                LdQ::load(rq[0], Q, g.qs, g.qk, q0, g.NQ, k0, kend, tid);
            }
        }
        // small tiles: whole k-tiles (all but possibly the last) take the loaders' short forms; next to sixteen
        // MFMAs the clamps, the zeroing selects and a 64-bit multiply per load of the general forms are most of the
        // instructions of a k-tile
        const bool req_full = DEEP && kl + BK <= kend, pub_full = DEEP && k0 + BK <= kend;
        auto request = [&](auto mc) {
            if constexpr (SPREAD) {
                constexpr int m = decltype(mc)::value, LA = m * NPT / SLOTS, LB = (m + 1) * NPT / SLOTS;
                static_for<LB - LA>([&](auto tc) {
                    constexpr int l = LA + decltype(tc)::value;
                    if constexpr (DEEP) {
                        if (req_full) {
                            if constexpr (l < NPP) LdP::template load_piece_full<l>(rp[LS], P, g.ps, g.pk, p0, g.NP, kl, tid);
                            else LdQ::template load_piece_full<l - NPP>(rq[LS], Q, g.qs, g.qk, q0, g.NQ, kl, tid);
                            return;
                        }
                    }
                    if constexpr (l < NPP) LdP::template load_piece<l>(rp[LS], P, g.ps, g.pk, p0, g.NP, kl, kend, tid);
                    else LdQ::template load_piece<l - NPP>(rq[LS], Q, g.qs, g.qk, q0, g.NQ, kl, kend, tid);
                });
            }
        };
        auto publish = [&](auto mc) {
            if constexpr (SPREAD) {
                constexpr int m = decltype(mc)::value, LA = m * NPT / SLOTS, LB = (m + 1) * NPT / SLOTS;
                static_for<LB - LA>([&](auto tc) {
                    constexpr int l = LA + decltype(tc)::value;
                    if constexpr (DEEP) {
                        if (pub_full) {
                            if constexpr (l < NPP) LdP::template store_piece<l, true>(rp[SS], nxt, k0, kend, tid);
                            else LdQ::template store_piece<l - NPP, true>(rq[SS], nxt + BP * 128, k0, kend, tid);
                            return;
                        }
                    }
                    if constexpr (l < NPP) LdP::template store_piece<l>(rp[SS], nxt, k0, kend, tid);
                    else LdQ::template store_piece<l - NPP>(rq[SS], nxt + BP * 128, k0, kend, tid);
                });
            }
        };
        if constexpr (DEEP) {
            // the pieces to publish arrived a k-tile ago and the other stage is free since the last barrier: they
            // go to LDS first, so that the barrier below never waits for an LDS write; the new requests follow
            phase(pfa, qfa, pfb, qfb, cur + wave_p, cur + wave_q, 1, publish);
            phase(pfb, qfb, pfa, qfa, cur + wave_p, cur + wave_q, 2, request);
            phase(pfa, qfa, pfb, qfb, cur + wave_p, cur + wave_q, 3, [](auto) {});
        } else {
            phase(pfa, qfa, pfb, qfb, cur + wave_p, cur + wave_q, 1, request);
            phase(pfb, qfb, pfa, qfa, cur + wave_p, cur + wave_q, 2, [](auto) {});
            phase(pfa, qfa, pfb, qfb, cur + wave_p, cur + wave_q, 3, publish);
        }
        if constexpr (!SPREAD) {
            if (more) {
                LdP::store(rp[0], nxt, k0, kend, tid);
                LdQ::store(rq[0], nxt + BP * 128, k0, kend, tid);
            }
        }
        // the barrier publishes LDS writes only; __syncthreads() would also wait for every global load in flight
        // (the requests of the k-tiles ahead), once per k-tile
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
        // after the last tile `nxt` holds stale data: the fragments read from it are never used
        phase(pfb, qfb, pfa, qfa, nxt + wave_p, nxt + wave_q, 0, [](auto) {});
    };
    if constexpr (DEEP) {
        for (int kt = 0; kt < KT; kt += NSET)
            static_for<NSET>([&](auto ic) {
                if (kt + decltype(ic)::value < KT) ktile(kt + decltype(ic)::value, ic);
            });
    } else {
        for (int kt = 0; kt < KT; ++kt) ktile(kt, std::integral_constant<int, 0>{});
    }

    store_tile<T, TP, TQ>(g, acc, p0, q0, wp, wq, lane, split);
}

// Second pass of split-K: sum the partials in split order (deterministic), then the same
// epilogue as the single-pass kernel.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_kernel(Args g, int splits, int lanes) {
    // `lanes` (a power of two, at most 16) neighbouring threads share one output element: lane l adds the
    // partials l, l + lanes, l + 2*lanes, ... in that order, then the lane sums are combined pairwise.  The
    // order is fixed by (splits, lanes) alone, so a product is reproducible from run to run.
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    const size_t total = (size_t)g.NQ * g.NP;
    const int lane = (int)(t & (size_t)(lanes - 1));
    size_t e = t / (size_t)lanes;
    const bool live = e < total;
    if (!live) e = total - 1;  // whole lane groups stay in step for the exchange below
    const int q = (int)(e / g.NP), p = (int)(e - (size_t)q * g.NP);
    float s = 0.0f;
    // eight partials are requested (from clamped addresses) before the first is added: left as a plain loop
    // the loads issue one per add and the launch is nothing but their latencies in a row
    const float *wp = g.ws + (size_t)q * g.NPpad + p;
    const size_t zstride = (size_t)g.NQ * g.NPpad;
    for (int z = lane; z < splits; z += 8 * lanes) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = wp[(size_t)min(z + u * lanes, splits - 1) * zstride];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += z + u * lanes < splits ? v[u] : 0.0f;  // s is never -0: adding +0 is exact
    }
    for (int o = lanes >> 1; o > 0; o >>= 1) s += __shfl_xor(s, o);
    if (!live || lane != 0) return;
    T *dst = (T *)g.D + (int64_t)p * g.dp + (int64_t)q * g.dq;
    T old = 0;
    if (g.beta != 0.0f) old = *dst;
    T bv = 0;
    if (g.has_bias) bv = ((const T *)g.bias)[(int64_t)(g.bias_on_p ? p : q) * g.bias_stride];
    *dst = finish<T>(s, g.alpha, g.beta, old, g.has_bias != 0, bv, g.act);
}

// The same pass for fewer than 16 splits, C rows contiguous along p and whole groups of four: one thread per four
// neighbouring outputs, the partials read 16 bytes at a time and four splits requested before the first add.  Every
// output is the sum of its partials in split order from +0, exactly as splitk_reduce_kernel with one lane forms it.
template <typename T>
__global__ __launch_bounds__(256) void splitk_reduce_vec4_kernel(Args g, int splits) {
    const size_t t = (size_t)blockIdx.x * 256 + threadIdx.x;
    const int groups_per_row = g.NP / 4;
    if (t >= (size_t)g.NQ * groups_per_row) return;
    const int q = (int)(t / groups_per_row), p = (int)(t - (size_t)q * groups_per_row) * 4;
    const float4 *wp = (const float4 *)(g.ws + (size_t)q * g.NPpad + p);
    const size_t zstride = (size_t)g.NQ * g.NPpad / 4;  // in float4
    float s[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int z = 0; z < splits; z += 4) {
        float4 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) v[u] = wp[(size_t)min(z + u, splits - 1) * zstride];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const bool on = z + u < splits;  // s is never -0: adding +0 is exact
            s[0] += on ? v[u].x : 0.0f;
            s[1] += on ? v[u].y : 0.0f;
            s[2] += on ? v[u].z : 0.0f;
            s[3] += on ? v[u].w : 0.0f;
        }
    }
    T *dst = (T *)g.D + p + (int64_t)q * g.dq;
    __align__(16) T old[4] = {0, 0, 0, 0}, out[4];
    if (g.beta != 0.0f) {
        if constexpr (sizeof(T) == 4) *(uint4 *)old = *(const uint4 *)dst;
        else *(uint2 *)old = *(const uint2 *)dst;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        T bv = 0;
        if (g.has_bias) bv = ((const T *)g.bias)[(int64_t)(g.bias_on_p ? p + e : q) * g.bias_stride];
        out[e] = finish<T>(s[e], g.alpha, g.beta, old[e], g.has_bias != 0, bv, g.act);
    }
    if constexpr (sizeof(T) == 4) *(uint4 *)dst = *(const uint4 *)out;
    else *(uint2 *)dst = *(const uint2 *)out;
}

}  // namespace gemm
}  // namespace agh

// Conv2 forward as an implicit GEMM on the matrix cores (bf16 and f32, unit stride and dilation): the patch
// matrix of im2col is never written.  A workgroup takes 256 consecutive output positions of one image
// and up to 128 output channels; it stages the input rows those positions touch ONCE in LDS, pixel
// major with the channels of a pixel contiguous, and then runs the k loop (filter tap, then 16
// channels per step; 8 for f32, where a step is four v_mfma_f32_32x32x2_f32 per tile) without a single
// barrier: the A operand of v_mfma_f32_32x32x16_bf16 (32 positions x 16 channels of one tap) is a
// 16-byte LDS read per lane, the B operand (32 output channels x the same 16 k) comes straight from
// a fragment-ordered copy of the filter bank, which is small and stays in L2.  A wave owns ALL 256
// positions of the tile and 32 output channels: per k step it reads eight A fragments from LDS (the
// four waves read the same ones; LDS serves 16-byte reads at 256 bytes per clock, this takes half) and
// ONE B fragment from memory, so the filter bank crosses the vector memory path once per workgroup.  When the rows of all
// input channels do not fit in half a CU's LDS, the channels are taken in passes of a power-of-two
// count each (stage, k loop over all taps, stage the next ...), accumulators staying in registers:
// two workgroups share a CU, so one's staging and epilogue run under the other's k loop.  HBM traffic is the image in and the activation out, a tenth of
// what im2col + GEMM move; bias and ReLU are applied in the epilogue in the order the separate
// layers round.  Sums are f32 in k order (tap, channel), one rounding at the end (none for f32), so
// results agree with the im2col chain within the GEMM tolerances, not bit for bit.
#include <stdlib.h>

#include <type_traits>

#include "agh_internal.h"

using namespace agh;

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kTileOc = 128;   // output channels per workgroup (4 MFMA tiles of 32, one per wave)

template <int N, typename F>
__device__ __forceinline__ void static_for(F &&f) {
    if constexpr (N > 0) {
        static_for<N - 1>(f);
        f(std::integral_constant<int, N - 1>{});
    }
}

// Element-type geometry: a 16-byte chunk holds CPC channels, a k step covers two chunks (one per half-wave).
template <typename T> struct Geo {
    static constexpr int ES = (int)sizeof(T);
    static constexpr int CPC = 16 / ES;           // channels per 16-byte chunk = pixels per 16-byte vector of a row
    static constexpr int CPI = 4 / ES;            // channels one staging item packs into a 4-byte LDS write
    static constexpr int EPI_POS = 256 / ES;      // positions the epilogue transposes at a time (256 bytes of an output row)
    static constexpr int EPITCH = 256 + 16;       // bytes per staged output-channel row in the epilogue (EPI_POS positions + pad)
};

struct ConvMfmaParams {
    int bs, ic, ih, iw, oc, oh, ow, fh, fw, ph, pw;
    int act, has_bias;
    int npos, tiles_per_img, oc_tiles;
    int lcols;     // staged columns: iw + 2*pw
    int icc, npass;  // channels staged per pass (a power of two), passes = ic / icc
    int nchunk;    // 16-byte chunks per staged pixel
    int K;         // fh*fw*ic
    int per_xcd;   // workgroups per XCD when the grid divides by 8, else 0
    int nt_store;  // output stores carry the streaming hint
    int remap;     // staging takes the coalesced lane order where it applies (AGH_CONV_REMAP=0 switches it off)
    FastDiv div_ow, div_tiles, div_octiles, div_vec;
};

// Filter bank [oc][ic][fh][fw] -> MFMA B-fragment order: for every tile of 32 output channels and every
// k step s = (pass * taps + tap) * steps_per_tap + (c % icc) / (2*CPC), pass = c / icc, one contiguous 1 KB block holding lane (kg, n)'s CPC values
// (channels 2*CPC*(c/(2*CPC)) + CPC*kg .. of output channel n) at position lane = 32*kg + n.  A wave then
// fetches a fragment with ONE fully coalesced 16-byte-per-lane load.
template <typename T>
__global__ __launch_bounds__(kThreads) void pack_filter_kernel(const T *__restrict__ w, T *__restrict__ wp, int ic, int icc, int ff,
                                                                int nsteps, size_t total) {
    constexpr int CPC = Geo<T>::CPC;
    const size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;  // source index: [o][c][tap]
    if (e >= total) return;
    const size_t per_o = (size_t)ic * ff;
    const size_t o = e / per_o;
    const int r = (int)(e - o * per_o);
    const int c = r / ff, tap = r - c * ff;
    const int s = ((c / icc) * ff + tap) * (icc / (2 * CPC)) + (c % icc) / (2 * CPC), kg = (c / CPC) & 1, i = c % CPC;
    const size_t dst = ((((o >> 5) * nsteps + s) * 64) + kg * 32 + (o & 31)) * CPC + i;
    wp[dst] = w[e];
}

// kTilePos output positions per workgroup (kMT MFMA tiles of 32), kWgs workgroups per CU, kBRing register sets of B
// fragments (requested kBRing - 1 steps ahead).
template <typename T, int kTilePos, int kWgs, int kBRing>
__global__ __launch_bounds__(kThreads, kWgs) void conv2_mfma_kernel(const T *__restrict__ x, const T *__restrict__ wp,
                                                                                  const T *__restrict__ bias, T *__restrict__ y,
                                                                                  ConvMfmaParams p) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr int ES = Geo<T>::ES, CPC = Geo<T>::CPC, PV = Geo<T>::CPC, kEpitch = Geo<T>::EPITCH, kEpiPos = Geo<T>::EPI_POS;
    constexpr int kMT = kTilePos / 32, kEpiMT = kEpiPos / 32, kBAhead = kBRing - 1;
    static_assert(kTilePos % 32 == 0, "whole MFMA tiles");
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    uint32_t t0, oct, b, tile;
    // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: give every XCD a run of consecutive
    // tiles, so that the input rows two neighbouring position tiles share are fetched from HBM once
    const uint32_t bid = p.per_xcd ? (blockIdx.x & 7u) * (uint32_t)p.per_xcd + (blockIdx.x >> 3) : blockIdx.x;
    p.div_octiles.divmod(bid, t0, oct);
    p.div_tiles.divmod(t0, b, tile);
    const int p0 = tile * kTilePos;
    const int plast = min(p0 + kTilePos, p.npos) - 1;
    const int ho_first = p.div_ow.div((uint32_t)p0), ho_last = p.div_ow.div((uint32_t)plast);
    const int lrows = ho_last - ho_first + p.fh;  // staged input rows
    const int pix_bytes = p.icc * ES;

    // ---- staging of one pass ----
    // A staged pixel is its icc channels (pix_bytes) plus 16 bytes of padding.  The lanes of a ds_read_b128 of the
    // k loop address consecutive pixels and the same chunk: with a pitch of pix_bytes + 16 (4 banks more than a
    // multiple of 8 banks) any 16 consecutive pixels fall on 16 different 16-byte bank groups, whatever the tap,
    // so the k loop needs no swizzle and its addresses are one add away from a per-lane constant.
    const int pitch = pix_bytes + 16;
    auto stage = [&](int pass) {
        // An item is CPC channels x PV (= CPC) pixels: CPC 16-byte loads, one per channel plane, transposed in
        // registers (bf16: one v_perm_b32 per output dword; f32: the transposition is register renaming) into
        // PV 16-byte LDS writes, one whole channel chunk of one pixel each.  Consecutive lanes take the
        // consecutive channel chunks of the same pixels, so a write instruction covers whole staged pixels
        // (contiguous bytes: no bank conflict).
        const int nvec = p.iw / PV, ngrp = p.icc / CPC;
        // Item order.  General: channel group fastest, so the lanes of an LDS write cover whole staged pixels.  With
        // eight channel groups of 16-bit elements (64 channels per pass) the lanes are dealt differently: a wave takes
        // eight consecutive 16-byte vectors of the rows (rows of a plane follow one another in memory, so the eight are
        // contiguous) in all eight groups, lane = (vector & 1) + 2 * group + 16 * (vector >> 1).  A load instruction then
        // touches 8 runs of 128 bytes instead of 64 separate 16-byte pieces in 64 cache lines, and the 16 lanes the LDS
        // serves together still write 16 different 16-byte bank groups (two neighbouring vectors are 8 pixels = 72
        // sixteen-byte units apart: 8 mod 16, the eight groups fill the gap).
        const bool remap = ES == 2 && ngrp == 8 && p.remap;
        const uint32_t nt = (uint32_t)lrows * nvec;  // 16-byte vectors of one channel plane in the staged rows
        const uint32_t items = remap ? ((nt + 7) / 8) * 64 : (uint32_t)lrows * ngrp * nvec;
        const T *ximg = x + ((size_t)b * p.ic + (size_t)pass * p.icc) * p.ih * (size_t)p.iw;
        const size_t plane = (size_t)p.ih * p.iw;
        // SB items per thread and trip: all SB * CPC loads are requested before the first LDS write (with two, a
        // workgroup's staging waits for memory about once: 448 items at the 64-channel 56 x 56 layer)
        constexpr int SB = kWgs >= 3 ? 1 : 2;  // three workgroups per CU leave 170 registers: one item at a time
        for (uint32_t it0 = tid; it0 < items; it0 += kThreads * SB) {
            uint4 r[SB][CPC];
            int dst[SB];
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                const uint32_t it = it0 + u * kThreads;
                uint32_t rv, v, lr, cg;
                if (remap) {
                    const uint32_t L = it & 63u;
                    cg = (L >> 1) & 7u;
                    rv = (it >> 6) * 8 + (((L >> 4) << 1) | (L & 1u));
                } else {
                    rv = it / (uint32_t)ngrp;
                    cg = it - rv * ngrp;
                }
                const bool live = it < items && rv < nt;
                p.div_vec.divmod(live ? rv : 0u, lr, v);
                const int hi = ho_first - p.ph + (int)lr;
#pragma unroll
                for (int i = 0; i < CPC; ++i) r[u][i] = make_uint4(0, 0, 0, 0);
                if (live && hi >= 0 && hi < p.ih) {
                    const T *src = ximg + ((size_t)(CPC * cg) * p.ih + hi) * (size_t)p.iw + v * PV;
#pragma unroll
                    for (int i = 0; i < CPC; ++i) r[u][i] = *(const uint4 *)(src + i * plane);
                }
                dst[u] = live ? ((int)lr * p.lcols + p.pw + (int)v * PV) * pitch + ((int)cg << 4) : -1;
            }
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                if (dst[u] < 0) continue;
#pragma unroll
                for (int j = 0; j < PV; ++j) {
                    uint4 o;
                    if constexpr (ES == 2) {
                        // pixel j's value is half (j & 1) of dword j >> 1 of every channel row; dword d of the chunk
                        // packs channels 2d (low half) and 2d + 1 (high half)
                        constexpr uint32_t kLow = 0x05040100u, kHigh = 0x07060302u;
                        const uint32_t sel = (j & 1) ? kHigh : kLow;
                        auto word = [&](const uint4 &q) { return (j >> 1) == 0 ? q.x : (j >> 1) == 1 ? q.y : (j >> 1) == 2 ? q.z : q.w; };
                        o.x = __builtin_amdgcn_perm(word(r[u][1 % CPC]), word(r[u][0]), sel);
                        o.y = __builtin_amdgcn_perm(word(r[u][3 % CPC]), word(r[u][2 % CPC]), sel);
                        o.z = __builtin_amdgcn_perm(word(r[u][5 % CPC]), word(r[u][4 % CPC]), sel);
                        o.w = __builtin_amdgcn_perm(word(r[u][7 % CPC]), word(r[u][6 % CPC]), sel);
                    } else {
                        auto word = [&](const uint4 &q) { return j == 0 ? q.x : j == 1 ? q.y : j == 2 ? q.z : q.w; };
                        o = make_uint4(word(r[u][0]), word(r[u][1 % CPC]), word(r[u][2 % CPC]), word(r[u][3 % CPC]));
                    }
                    *(uint4 *)(lds + dst[u] + j * pitch) = o;
                }
            }
        }
        if (pass == 0) {  // padding columns left and right of the image: no pass writes them again
            const int npadcol = p.lcols - p.iw, nch = p.nchunk;
            const uint32_t pads = (uint32_t)lrows * npadcol * nch;
            for (uint32_t it = tid; it < pads; it += kThreads) {
                const uint32_t ch = it % nch, rc = it / nch;
                const uint32_t k = rc % npadcol, lr = rc / npadcol;
                const int col = (int)k < p.pw ? (int)k : p.iw + (int)k;
                *(uint4 *)(lds + ((int)lr * p.lcols + col) * pitch + (ch << 4)) = make_uint4(0, 0, 0, 0);
            }
        }
    };

    // ---- per-lane operand addressing ----
    const int kg = lane >> 5, l32 = lane & 31;
    int abase[kMT];  // byte address of the lane's chunk (half-wave kg) of its staged pixel for tap (0,0), per position tile
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt) {
        const int pp = min(p0 + mt * 32 + l32, p.npos - 1);  // clamped: a duplicate, never stored
        uint32_t ho, wo;
        p.div_ow.divmod((uint32_t)pp, ho, wo);
        abase[mt] = (((int)ho - ho_first) * p.lcols + (int)wo) * pitch + (kg << 4);
    }
    const int ncc = p.icc / (2 * CPC);          // k steps per tap in one pass
    const int nsteps = p.fh * p.fw * ncc;       // k steps per pass
    const int oc0 = oct * kTileOc + wave * 32;
    const bool wave_live = oc0 < p.oc;  // oc is a multiple of 64
    // fragment-ordered bank: block (tile of 32 channels, step), 16 bytes per lane.  The block address is
    // wave-uniform (scalar registers), the lane adds 16 * lane.
    const unsigned char *bbank = (const unsigned char *)wp + (size_t)(min(oc0, p.oc - 32) >> 5) * nsteps * p.npass * 1024;
    const uint32_t blane = (uint32_t)lane * 16u;

    f32x16 acc[kMT];
#pragma unroll
    for (int mt = 0; mt < kMT; ++mt) acc[mt] = (f32x16)(0.0f);

    // ---- k loop of a pass: taps outer, 2*CPC channels per step ----
    int fi = 0, fj = 0, cc = 0;  // position of the NEXT step to load
    // A fragments: the fragment of tile mt for step s+1 is read from LDS into the same registers right after
    // the MFMA of tile mt of step s has been issued (eight MFMAs, 256 clocks, ahead of its use); its address
    // is the lane's constant plus a wave-uniform step offset.  B fragments come from L2 (several hundred
    // cycles away), so they are requested kBAhead steps ahead into a ring of register sets.  The main loop
    // takes a whole ring of steps per trip so every register index is static, and it contains no branch around
    // a load: a load that would run past the last step re-reads a valid location instead (with conditional
    // loads the compiler can no longer count outstanding loads and waits for all of them before every MFMA
    // group, which serialises the L2 latency into each step).
    int aoff_next = 0;  // wave-uniform byte offset of the step the next load_a calls will fetch
    auto prepare_a = [&](int s) { aoff_next = s < nsteps ? (fi * p.lcols + fj) * pitch + (cc << 5) : 0; };
    auto load_a = [&](uint4(&a)[kMT], auto mtc) {
        constexpr int mt = decltype(mtc)::value;
        a[mt] = *(const uint4 *)(lds + abase[mt] + aoff_next);
    };
    auto advance_a = [&]() {
        if (++cc == ncc) {
            cc = 0;
            if (++fj == p.fw) { fj = 0; ++fi; }
        }
    };
    auto load_b = [&](uint4 &bq, int s) { bq = *(const uint4 *)(bbank + (size_t)min(s, nsteps - 1) * 1024 + blane); };
    auto mma = [&](const uint4(&a)[kMT], const uint4 &bq, auto mtc) {
        constexpr int mt = decltype(mtc)::value;
        if constexpr (ES == 2) {
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[mt]), __builtin_bit_cast(bf16x8_t, bq), acc[mt], 0, 0, 0);
        } else {  // lanes 0-31 hold channels c..c+3, lanes 32-63 channels c+4..c+7: element j of both is one k pair
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].x), __uint_as_float(bq.x), acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].y), __uint_as_float(bq.y), acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].z), __uint_as_float(bq.z), acc[mt], 0, 0, 0);
            acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].w), __uint_as_float(bq.w), acc[mt], 0, 0, 0);
        }
    };
    // One step: the eight MFMA groups of step s on (a, bq); the A fragment of each tile is refreshed for step s+1
    // right behind its MFMA, the B fragment of the step kBAhead ahead is requested (into bn) in the middle; the
    // tap bookkeeping for step s+2 runs at the end of the step, after the last refresh.  sched_barrier pins the order, so the matrix pipe gets
    // new work back to back while the other requests trickle out.
    auto step = [&](uint4(&a)[kMT], const uint4 &bq, uint4 &bn, int s) {
        prepare_a(s + 1);
        static_for<kMT>([&](auto mtc) {
            constexpr int mt = decltype(mtc)::value;
            mma(a, bq, mtc);
            load_a(a, mtc);
            if constexpr (mt == 3) load_b(bn, s + kBAhead);
            if constexpr (mt == kMT - 1) advance_a();
            __builtin_amdgcn_sched_barrier(0);
        });
    };

    for (int pass = 0; pass < p.npass; ++pass) {
        if (pass) __syncthreads();  // every wave is done reading the previous pass's channels
        stage(pass);
        __syncthreads();
        if (wave_live) {
            uint4 a[kMT], bf[kBRing];
            static_for<kBAhead>([&](auto ic) { load_b(bf[decltype(ic)::value], decltype(ic)::value); });
            fi = 0; fj = 0; cc = 0;
            prepare_a(0);
            static_for<kMT>([&](auto mtc) { load_a(a, mtc); });
            advance_a();
            int s = 0;
            for (; s + kBRing <= nsteps; s += kBRing)
                static_for<kBRing>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    step(a, bf[i], bf[(i + kBAhead) % kBRing], s + i);
                });
            // fewer than a ring of steps left: their B fragments are in bf[0 ..]; the requests these steps
            // make land in the one set no remaining step reads
            const int left = nsteps - s;
            static_for<kBRing - 1>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                if (i < left) step(a, bf[i], bf[kBRing - 1], s + i);
            });
            bbank += (size_t)nsteps * 1024;
        }
    }
    __syncthreads();  // every wave is done with the staged image: LDS becomes the epilogue's transposition space

    // ---- epilogue: round, bias, ReLU, transpose 32 channels x 128 positions at a time through LDS, 16-byte stores ----
    if (wave_live) {
        unsigned char *region = lds + wave * 32 * kEpitch;
        const bool relu = p.act == AGH_ACT_RELU;
        const int o_lane = oc0 + l32;
        float bq = 0.0f;
        if (p.has_bias) bq = Elem<T>::to_f32(bias[min(o_lane, p.oc - 1)]);
        // the position tiles leave in groups of kEpiMT (256 bytes of every output row), the last group may be smaller
        static_for<(kMT + kEpiMT - 1) / kEpiMT>([&](auto partc) {
            constexpr int part = decltype(partc)::value;
            constexpr int NMT = (kMT - part * kEpiMT) < kEpiMT ? (kMT - part * kEpiMT) : kEpiMT;
#pragma unroll
            for (int m4 = 0; m4 < NMT; ++m4)
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    const int mt = part * kEpiMT + m4;
                    const int pl = m4 * 32 + blk * 8 + kg * 4;  // position inside this part
                    if constexpr (ES == 2) {
                        // two packed conversions give the four rounded values as two dwords
                        uint32_t w[2] = {f32x2_to_bf16x2(acc[mt][blk * 4 + 0], acc[mt][blk * 4 + 1]),
                                         f32x2_to_bf16x2(acc[mt][blk * 4 + 2], acc[mt][blk * 4 + 3])};
                        if (p.has_bias || relu) {  // wave-uniform
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                // the rounded products as f32 (exact); bias + product is rounded again by the conversion below
                                float lo = __uint_as_float(w[h] << 16), hi = __uint_as_float(w[h] & 0xFFFF0000u);
                                if (p.has_bias) {
                                    lo = bq + lo;
                                    hi = bq + hi;
                                }
                                // relu keeps x when x >= 0 (so -0 stays, NaN goes to 0).  Taken on the f32 value before the
                                // final rounding: rounding changes neither sign nor NaN-ness, and a sum of two bf16 values is
                                // zero or at least the smallest bf16 subnormal, so it cannot round to -0.
                                if (relu) {
                                    lo = lo >= 0.0f ? lo : 0.0f;
                                    hi = hi >= 0.0f ? hi : 0.0f;
                                }
                                w[h] = f32x2_to_bf16x2(lo, hi);
                            }
                        }
                        *(uint2 *)(region + l32 * kEpitch + pl * 2) = make_uint2(w[0], w[1]);
                    } else {
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = acc[mt][blk * 4 + e];
                        if (p.has_bias) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = bq + v[e];
                        }
                        if (relu) {
#pragma unroll
                            for (int e = 0; e < 4; ++e) v[e] = v[e] >= 0.0f ? v[e] : 0.0f;
                        }
                        *(float4 *)(region + l32 * kEpitch + pl * 4) = make_float4(v[0], v[1], v[2], v[3]);
                    }
                }
            // same wave, LDS executes in order: the reads below see the writes above, and the next part's
            // writes come after these reads.  A staged row of NMT tiles is NMT * 64 bytes = 4 * NMT chunks (in either
            // element type: 32 positions are 64 or 128 bytes, and kEpiMT is 4 or 2).
            constexpr int CPRW = NMT * 32 * ES / 16, TOTAL = 32 * CPRW, NST = (TOTAL + 63) / 64;
#pragma unroll
            for (int r = 0; r < NST; ++r) {
                const int idx = r * 64 + lane, row = idx / CPRW, chunk = idx % CPRW;
                if (TOTAL % 64 != 0 && idx >= TOTAL) continue;
                const uint4 v = *(const uint4 *)(region + row * kEpitch + chunk * 16);
                const int pos = p0 + part * kEpiPos + chunk * CPC, o = oc0 + row;
                if (pos < p.npos && o < p.oc) {
                    typedef uint32_t u32x4_nt __attribute__((ext_vector_type(4)));
                    if (p.nt_store) __builtin_nontemporal_store(u32x4_nt{v.x, v.y, v.z, v.w}, (u32x4_nt *)(y + ((size_t)b * p.oc + o) * p.npos + pos));
                    else *(uint4 *)(y + ((size_t)b * p.oc + o) * p.npos + pos) = v;
                }
            }
        });
    }
}

}  // namespace

namespace agh {

// Returns 1 when the geometry is not one this kernel takes (the caller goes on to its other paths),
// otherwise a status code.  The API lock is held by the caller.
template <typename T, int kTilePos, int kWgs, int kBRing>
static int conv2_mfma_launch(const char *name, const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic, int64_t ih,
                   int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t oh, int64_t ow, int act) {
    constexpr int ES = Geo<T>::ES, CPC = Geo<T>::CPC;
    const int64_t npos = oh * ow;
    if (ic < 2 * CPC || ic % (2 * CPC) != 0 || ic > 8192 || oc % 64 != 0 || iw % CPC != 0 || npos % CPC != 0 || fh * fw > 64) return 1;
    if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) != 0) return 1;
    // little work per output: the LDS-resident scalar kernels do better on small problems
    if (ic * fh * fw < 128 || npos < 256) return 1;
    const int64_t lcols = iw + 2 * pw;
    const int64_t rows_out = std::min<int64_t>(oh, (kTilePos - 1) / ow + 2);
    // kWgs workgroups per CU (160 KB of LDS): the largest power-of-two channel count whose rows fit in a share
    const int64_t lds_limit = 160 * 1024 / kWgs;
    int64_t icc = ic & -ic;  // channels per pass: a power of two that divides ic
    while (icc > 2 * CPC && (rows_out + fh - 1) * lcols * (icc * ES + 16) > lds_limit) icc >>= 1;
    const int64_t tile_bytes = (rows_out + fh - 1) * lcols * (icc * ES + 16);  // staged pixels are padded by 16 bytes
    const int64_t smem = std::max<int64_t>(tile_bytes, 4 * 32 * Geo<T>::EPITCH);
    if (smem > lds_limit) return 1;
    const int64_t tiles = (npos + kTilePos - 1) / kTilePos, octiles = (oc + kTileOc - 1) / kTileOc;
    const int64_t blocks = bs * tiles * octiles;
    if (blocks > 0x7FFFFFFFll || bs * ic * ih * iw > ((int64_t)1 << 40)) return 1;

    void *wperm = nullptr;
    const size_t wtotal = (size_t)(oc * ic * fh * fw);
    if (int rc = workspace(wtotal * ES, &wperm)) return rc;
    const int nsteps = (int)(fh * fw * (ic / (2 * CPC)));  // over all passes
    hipLaunchKernelGGL(pack_filter_kernel<T>, dim3((unsigned)((wtotal + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream(),
                       (const T *)w, (T *)wperm, (int)ic, (int)icc, (int)(fh * fw), nsteps, wtotal);
    AGH_LAUNCH_CHECK(name);

    ConvMfmaParams p;
    p.bs = bs; p.ic = ic; p.ih = ih; p.iw = iw; p.oc = oc; p.oh = oh; p.ow = ow; p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw;
    p.act = act; p.has_bias = bias != nullptr;
    p.npos = npos; p.tiles_per_img = tiles; p.oc_tiles = octiles; p.lcols = lcols;
    p.icc = icc; p.npass = ic / icc;
    p.nchunk = icc / CPC;
    p.K = fh * fw * ic;
    p.per_xcd = blocks % 8 == 0 ? (int)(blocks / 8) : 0;
    {
        const char *e = getenv("AGH_CONV_REMAP");
        p.remap = e && *e ? atoi(e) : 1;
        // An output that could not stay in the 256 MB last-level cache next to the input anyway is stored with the
        // streaming hint, which leaves that cache to the input rows neighbouring tiles share (config 3 in bf16: 0.135 ->
        // 0.124 ms); a smaller one is stored plainly, for the layer that reads it next.  AGH_CONV_NT=0|1 overrides.
        const char *nt = getenv("AGH_CONV_NT");
        const size_t out_bytes = (size_t)bs * oc * npos * sizeof(T);
        p.nt_store = nt && *nt ? atoi(nt) : out_bytes > ((size_t)64 << 20);
    }
    p.div_ow = FastDiv((uint32_t)ow);
    p.div_tiles = FastDiv((uint32_t)tiles);
    p.div_octiles = FastDiv((uint32_t)octiles);
    p.div_vec = FastDiv((uint32_t)(iw / CPC));
    static bool attr_done = false;
    if (!attr_done) {
        AGH_HIP(hipFuncSetAttribute((const void *)(conv2_mfma_kernel<T, kTilePos, kWgs, kBRing>), hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_limit));
        attr_done = true;
    }
    hipLaunchKernelGGL((conv2_mfma_kernel<T, kTilePos, kWgs, kBRing>), dim3((unsigned)blocks), dim3(kThreads), (size_t)smem, stream(), (const T *)x,
                       (const T *)wperm, (const T *)bias, (T *)y, p);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int conv2_mfma_try(const char *name, const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic, int64_t ih,
                   int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t oh, int64_t ow, int act) {
    // f32: 128 positions per workgroup and three workgroups per CU; while one stages its rows or writes its outputs
    // (memory latency), two others keep the matrix pipes fed (measured 132 against 124 TFLOP/s at the 256 x 64 x 56 x 56
    // layer).  bf16, whose k loop is eight times shorter per byte staged: 256 positions and two per CU (halo rows are
    // a smaller share; 878 against 796 TFLOP/s).  AGH_CONV_TILE=128|256 overrides.
    const char *e = getenv("AGH_CONV_TILE");
    const int tile = e && *e ? atoi(e) : (sizeof(T) == 4 ? 128 : 256);
    if (tile == 128)
        return conv2_mfma_launch<T, 128, 3, 8>(name, x, w, bias, y, bs, ic, ih, iw, oc, fh, fw, ph, pw, oh, ow, act);
    return conv2_mfma_launch<T, 256, 2, 8>(name, x, w, bias, y, bs, ic, ih, iw, oc, fh, fw, ph, pw, oh, ow, act);
}

template int conv2_mfma_try<uint16_t>(const char *, const void *, const void *, const void *, void *, int64_t, int64_t, int64_t, int64_t,
                                      int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int);
template int conv2_mfma_try<float>(const char *, const void *, const void *, const void *, void *, int64_t, int64_t, int64_t, int64_t,
                                   int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int);

}  // namespace agh

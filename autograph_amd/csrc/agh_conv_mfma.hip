// Conv2 forward as an implicit GEMM on the matrix cores (bf16 and f32, unit stride and dilation): the patch
// matrix of im2col is never written.  A workgroup takes 256 consecutive output positions of one image
// and up to 128 output channels; it stages the input rows those positions touch ONCE in LDS, pixel
// major with the channels of a pixel contiguous, and then runs the k loop (filter tap, then 16
// channels per step; 8 for f32, where a step is four v_mfma_f32_32x32x2_f32 per tile) without a single
// barrier: the A operand of v_mfma_f32_32x32x16_bf16 (32 positions x 16 channels of one tap) is a
// 16-byte LDS read per lane, the B operand (32 output channels x the same 16 k) comes straight from
// a fragment-ordered copy of the filter bank, which is small and stays in L2.  When the rows of all
// input channels do not fit in half a CU's LDS, the channels are taken in passes of a power-of-two
// count each (stage, k loop over all taps, stage the next ...), accumulators staying in registers:
// two workgroups share a CU, so one's staging and epilogue run under the other's k loop.  HBM traffic is the image in and the activation out, a tenth of
// what im2col + GEMM move; bias and ReLU are applied in the epilogue in the order the separate
// layers round.  Sums are f32 in k order (tap, channel), one rounding at the end (none for f32), so
// results agree with the im2col chain within the GEMM tolerances, not bit for bit.
#include <type_traits>

#include "agh_internal.h"

using namespace agh;

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kTilePos = 256;  // output positions per workgroup (8 MFMA tiles of 32)
constexpr int kTileOc = 128;   // output channels per workgroup (4 MFMA tiles of 32)

// Element-type geometry: a 16-byte chunk holds CPC channels, a k step covers two chunks (one per half-wave).
template <typename T> struct Geo {
    static constexpr int ES = (int)sizeof(T);
    static constexpr int CPC = 16 / ES;           // channels per 16-byte chunk = pixels per 16-byte vector of a row
    static constexpr int CPI = 4 / ES;            // channels one staging item packs into a 4-byte LDS write
    static constexpr int EPITCH = 128 * ES + 16;  // bytes per staged output-channel row in the epilogue (128 positions + pad)
};

struct ConvMfmaParams {
    int bs, ic, ih, iw, oc, oh, ow, fh, fw, ph, pw;
    int act, has_bias;
    int npos, tiles_per_img, oc_tiles;
    int lcols;     // staged columns: iw + 2*pw
    int icc, npass;  // channels staged per pass (a power of two), passes = ic / icc
    int nch_mask;  // 16-byte chunks per staged pixel - 1 (a power of two)
    int kshift;    // log2(pixels per 256 bytes): see the swizzle key below
    int K;         // fh*fw*ic
    int per_xcd;   // workgroups per XCD when the grid divides by 8, else 0
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

template <typename T>
__global__ __launch_bounds__(kThreads, 2) void conv2_mfma_kernel(const T *__restrict__ x, const T *__restrict__ wp,
                                                                                  const T *__restrict__ bias, T *__restrict__ y,
                                                                                  ConvMfmaParams p) {
    extern __shared__ __align__(16) unsigned char lds[];
    constexpr int ES = Geo<T>::ES, CPC = Geo<T>::CPC, CPI = Geo<T>::CPI, PV = Geo<T>::CPC, kEpitch = Geo<T>::EPITCH;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
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

    // ---- staging of one pass: items = (row, channel pair or channel, 16-byte vector of the row) ----
    // The 16-byte channel chunks of pixel q are stored at chunk ^ key(q), key(q) = ((q >> kshift) + (q >> 4)) &
    // nch_mask.  The lanes of a ds_read_b128 of the k loop address 16 consecutive pixels and the same chunk:
    // the first term puts those 16 reads on 16 different 16-byte columns of the 256-byte LDS row.  The lanes
    // of a staging write address pixels 8 apart: the second term spreads those as well.
    auto stage = [&](int pass) {
        const int nvec = p.iw / PV, npair = p.icc / CPI;  // an item packs CPI channels of PV pixels into PV 4-byte writes
        const uint32_t items = (uint32_t)lrows * npair * nvec;
        const T *ximg = x + ((size_t)b * p.ic + (size_t)pass * p.icc) * p.ih * (size_t)p.iw;
        // batches of SB items per thread: all global loads of a batch are issued before the first LDS write
        constexpr int SB = 4;
        for (uint32_t it0 = tid; it0 < items; it0 += kThreads * SB) {
            uint4 r0[SB], r1[SB];
            int base[SB], pix0[SB], cpart[SB];
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                const uint32_t it = it0 + u * kThreads;
                uint32_t rc, v, lr, c2;
                p.div_vec.divmod(it, rc, v);
                lr = rc / (uint32_t)npair;
                c2 = rc - lr * npair;
                const int hi = ho_first - p.ph + (int)lr;
                r0[u] = make_uint4(0, 0, 0, 0);
                r1[u] = r0[u];
                if (it < items && hi >= 0 && hi < p.ih) {
                    const T *src = ximg + ((size_t)(CPI * c2) * p.ih + hi) * (size_t)p.iw + v * PV;
                    r0[u] = *(const uint4 *)src;
                    if constexpr (CPI == 2) r1[u] = *(const uint4 *)(src + (size_t)p.ih * p.iw);
                }
                const int c = CPI * (int)c2;
                pix0[u] = (int)lr * p.lcols + p.pw + (int)v * PV;
                base[u] = it < items ? pix0[u] * pix_bytes + (c % CPC) * ES : -1;
                cpart[u] = c / CPC;
            }
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                if (base[u] < 0) continue;
                const uint32_t lo[4] = {r0[u].x, r0[u].y, r0[u].z, r0[u].w}, hi2[4] = {r1[u].x, r1[u].y, r1[u].z, r1[u].w};
#pragma unroll
                for (int j = 0; j < PV; ++j) {
                    uint32_t word;
                    if constexpr (CPI == 2) word = ((lo[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu) | (((hi2[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu) << 16);
                    else word = lo[j];
                    const int q = pix0[u] + j;
                    const int addr = base[u] + j * pix_bytes + ((cpart[u] ^ (((q >> p.kshift) + (q >> 4)) & p.nch_mask)) << 4);
                    *(uint32_t *)(lds + addr) = word;
                }
            }
        }
        if (pass == 0) {  // padding columns left and right of the image: no pass writes them again
            const int npadcol = p.lcols - p.iw, nch = p.nch_mask + 1;
            const uint32_t pads = (uint32_t)lrows * npadcol * nch;
            for (uint32_t it = tid; it < pads; it += kThreads) {
                const uint32_t ch = it % nch, rc = it / nch;
                const uint32_t k = rc % npadcol, lr = rc / npadcol;
                const int col = (int)k < p.pw ? (int)k : p.iw + (int)k;
                *(uint4 *)(lds + ((int)lr * p.lcols + col) * pix_bytes + (ch << 4)) = make_uint4(0, 0, 0, 0);
            }
        }
    };

    // ---- per-lane operand addressing ----
    const int kg = lane >> 5, l32 = lane & 31;
    int apix[4], abase[4];  // the lane's staged pixel for tap (0,0) of each position tile, and its byte address
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        const int pp = min(p0 + (wm * 4 + mt) * 32 + l32, p.npos - 1);  // clamped: a duplicate, never stored
        uint32_t ho, wo;
        p.div_ow.divmod((uint32_t)pp, ho, wo);
        apix[mt] = ((int)ho - ho_first) * p.lcols + (int)wo;
        abase[mt] = apix[mt] * pix_bytes;
    }
    const int ncc = p.icc / (2 * CPC);          // k steps per tap in one pass
    const int nsteps = p.fh * p.fw * ncc;       // k steps per pass
    const int oc0 = oct * kTileOc + wn * 64;
    const bool wave_live = oc0 < p.oc;  // oc is a multiple of 64
    const T *brow[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)  // fragment-ordered bank: block (tile of 32 channels, step), CPC elements per lane
        brow[nt] = wp + ((size_t)(min(oc0 + nt * 32, p.oc - 32) >> 5) * nsteps * p.npass * 64 + lane) * CPC;

    f32x16 acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) acc[mt][nt] = (f32x16)(0.0f);

    // ---- k loop of a pass: taps outer, 2*CPC channels per step, operands of step s+1 requested before the MFMAs of step s ----
    int fi = 0, fj = 0, cc = 0;  // position of the NEXT step to load
    int akey[4];                 // swizzle key of the current tap, << 4
    const int kg16 = kg << 4;
    // A fragments: next step's LDS reads are issued before this step's MFMAs.  B fragments come from L2
    // (several hundred cycles away), so they are requested three steps ahead into a ring of four
    // register sets.  The main loop takes four steps per trip so every register index is static, and
    // it contains no branch around a load: a load that would run past the last step re-reads a valid
    // location instead (with conditional loads the compiler can no longer count outstanding loads and
    // waits for all of them before every MFMA group, which serialises the L2 latency into each step).
    int tapbytes_next = 0, chunk16_next = kg16;  // of the step the next load_a_part calls will fetch
    auto prepare_a = [&](int s) {  // scalar / per-lane state for fetching step s's A fragments
        tapbytes_next = s < nsteps ? (fi * p.lcols + fj) * pix_bytes : 0;
        chunk16_next = kg16 + ((s < nsteps ? cc : 0) << 5);
    };
    auto load_a_part = [&](uint4(&a)[4], auto mtc) {
        constexpr int mt = decltype(mtc)::value;
        a[mt] = *(const uint4 *)(lds + abase[mt] + tapbytes_next + (chunk16_next ^ akey[mt]));
    };
    auto set_keys = [&]() {
#pragma unroll
        for (int mt = 0; mt < 4; ++mt) {
            const int q = apix[mt] + fi * p.lcols + fj;
            akey[mt] = (((q >> p.kshift) + (q >> 4)) & p.nch_mask) << 4;
        }
    };
    auto advance_a = [&]() {
        if (++cc == ncc) {
            cc = 0;
            if (++fj == p.fw) { fj = 0; ++fi; }
            set_keys();
        }
    };
    auto load_b_part = [&](uint4(&bq)[2], int s, auto ntc) {
        constexpr int nt = decltype(ntc)::value;
        bq[nt] = *(const uint4 *)(brow[nt] + (size_t)min(s, nsteps - 1) * (64 * CPC));
    };
    auto mma = [&](const uint4(&a)[4], const uint4(&bq)[2], auto nc) {
        constexpr int n = decltype(nc)::value, mt = n >> 1, nt = n & 1;
        if constexpr (ES == 2) {
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[mt]), __builtin_bit_cast(bf16x8_t, bq[nt]),
                                                                  acc[mt][nt], 0, 0, 0);
        } else {  // lanes 0-31 hold channels c..c+3, lanes 32-63 channels c+4..c+7: element j of both is one k pair
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].x), __uint_as_float(bq[nt].x), acc[mt][nt], 0, 0, 0);
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].y), __uint_as_float(bq[nt].y), acc[mt][nt], 0, 0, 0);
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].z), __uint_as_float(bq[nt].z), acc[mt][nt], 0, 0, 0);
            acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x2f32(__uint_as_float(a[mt].w), __uint_as_float(bq[nt].w), acc[mt][nt], 0, 0, 0);
        }
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>;
    using I5 = std::integral_constant<int, 5>;
    using I6 = std::integral_constant<int, 6>;
    using I7 = std::integral_constant<int, 7>;
    // One step: the eight MFMA groups of step s on (a, b), with the fetches of step s+1's A fragments (into an)
    // and of step s+3's B fragments (into bn) handed out between them, one per group.  sched_barrier pins
    // the order, so the matrix pipe gets new work back to back while the other requests trickle out.
    auto step = [&](const uint4(&a)[4], const uint4(&bq)[2], uint4(&an)[4], uint4(&bn)[2], int s) {
        prepare_a(s + 1);
        mma(a, bq, I0{}); load_a_part(an, I0{}); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I1{}); load_a_part(an, I1{}); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I2{}); load_a_part(an, I2{}); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I3{}); load_a_part(an, I3{}); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I4{}); load_b_part(bn, s + 3, I0{}); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I5{}); load_b_part(bn, s + 3, I1{}); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I6{}); advance_a(); __builtin_amdgcn_sched_barrier(0);
        mma(a, bq, I7{}); __builtin_amdgcn_sched_barrier(0);
    };

    for (int pass = 0; pass < p.npass; ++pass) {
        if (pass) __syncthreads();  // every wave is done reading the previous pass's channels
        stage(pass);
        __syncthreads();
        if (wave_live) {
            uint4 a0[4], a1[4], b0[2], b1[2], b2[2], b3[2];
            load_b_part(b0, 0, I0{}); load_b_part(b0, 0, I1{});
            load_b_part(b1, 1, I0{}); load_b_part(b1, 1, I1{});
            load_b_part(b2, 2, I0{}); load_b_part(b2, 2, I1{});
            fi = 0; fj = 0; cc = 0;
            set_keys();
            prepare_a(0);
            load_a_part(a0, I0{}); load_a_part(a0, I1{}); load_a_part(a0, I2{}); load_a_part(a0, I3{});
            advance_a();
            int s = 0;
            for (; s + 4 <= nsteps; s += 4) {
                step(a0, b0, a1, b3, s);
                step(a1, b1, a0, b0, s + 1);
                step(a0, b2, a1, b1, s + 2);
                step(a1, b3, a0, b2, s + 3);
            }
            // up to three steps left: their B fragments are in b0, b1, b2 and the first one's A fragments in a0
            const int left = nsteps - s;
            if (left >= 1) step(a0, b0, a1, b3, s);
            if (left >= 2) step(a1, b1, a0, b3, s + 1);
            if (left >= 3) step(a0, b2, a1, b3, s + 2);
            brow[0] += (size_t)nsteps * (64 * CPC);
            brow[1] += (size_t)nsteps * (64 * CPC);
        }
    }
    __syncthreads();  // every wave is done with the staged image: LDS becomes the epilogue's transposition space

    // ---- epilogue: round, bias, ReLU, transpose 32 channels x 128 positions through LDS, 16-byte stores ----
    if (wave_live) {
        unsigned char *region = lds + wave * 32 * kEpitch;
        const bool relu = p.act == AGH_ACT_RELU;
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) {
            const int o_lane = oc0 + nt * 32 + l32;
            float bq = 0.0f;
            if (p.has_bias) bq = Elem<T>::to_f32(bias[min(o_lane, p.oc - 1)]);
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
                    const int pl = mt * 32 + blk * 8 + kg * 4;  // position inside the wave's 128
                    if constexpr (ES == 2) {
                        // two packed conversions give the four rounded values as two dwords
                        uint32_t w[2] = {f32x2_to_bf16x2(acc[mt][nt][blk * 4 + 0], acc[mt][nt][blk * 4 + 1]),
                                         f32x2_to_bf16x2(acc[mt][nt][blk * 4 + 2], acc[mt][nt][blk * 4 + 3])};
                        if (p.has_bias) {  // wave-uniform: bias + rounded product, rounded again
#pragma unroll
                            for (int h = 0; h < 2; ++h)
                                w[h] = f32x2_to_bf16x2(bq + __uint_as_float(w[h] << 16), bq + __uint_as_float(w[h] & 0xFFFF0000u));
                        }
                        if (relu) {  // wave-uniform; keeps x when x >= 0 (so -0 stays, NaN goes to 0)
#pragma unroll
                            for (int h = 0; h < 2; ++h) {
                                const bool klo = __uint_as_float(w[h] << 16) >= 0.0f, khi = __uint_as_float(w[h] & 0xFFFF0000u) >= 0.0f;
                                w[h] = (klo ? (w[h] & 0xFFFFu) : 0u) | (khi ? (w[h] & 0xFFFF0000u) : 0u);
                            }
                        }
                        *(uint2 *)(region + l32 * kEpitch + pl * 2) = make_uint2(w[0], w[1]);
                    } else {
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = acc[mt][nt][blk * 4 + e];
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
            // same wave, LDS executes in order: the reads below see the writes above
            constexpr int CPRW = 128 * ES / 16, RPI = 64 / CPRW, NST = 32 / RPI;  // chunks per row, rows per instruction
#pragma unroll
            for (int r = 0; r < NST; ++r) {
                const int row = r * RPI + lane / CPRW, chunk = lane % CPRW;
                const uint4 v = *(const uint4 *)(region + row * kEpitch + chunk * 16);
                const int pos = p0 + wm * 128 + chunk * CPC, o = oc0 + nt * 32 + row;
                if (pos < p.npos && o < p.oc) *(uint4 *)(y + ((size_t)b * p.oc + o) * p.npos + pos) = v;
            }
        }
    }
}

}  // namespace

namespace agh {

// Returns 1 when the geometry is not one this kernel takes (the caller goes on to its other paths),
// otherwise a status code.  The API lock is held by the caller.
template <typename T>
int conv2_mfma_try(const char *name, const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic, int64_t ih,
                   int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t oh, int64_t ow, int act) {
    constexpr int ES = Geo<T>::ES, CPC = Geo<T>::CPC;
    const int64_t npos = oh * ow;
    if (ic < 2 * CPC || ic % (2 * CPC) != 0 || ic > 8192 || oc % 64 != 0 || iw % CPC != 0 || npos % CPC != 0 || fh * fw > 64) return 1;
    if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) != 0) return 1;
    // little work per output: the LDS-resident scalar kernels do better on small problems
    if (ic * fh * fw < 128 || npos < 256) return 1;
    const int64_t lcols = iw + 2 * pw;
    const int64_t rows_out = std::min<int64_t>(oh, (kTilePos - 1) / ow + 2);
    // two workgroups per CU (160 KB of LDS): the largest power-of-two channel count whose rows fit in half
    const int64_t lds_limit = 80 * 1024;
    int64_t icc = ic & -ic;  // channels per pass: a power of two that divides ic
    while (icc > 2 * CPC && (rows_out + fh - 1) * lcols * icc * ES > lds_limit) icc >>= 1;
    const int64_t tile_bytes = (rows_out + fh - 1) * lcols * icc * ES;
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
    p.nch_mask = icc / CPC - 1;
    const int64_t pix_bytes = icc * ES;  // pixels per 256 bytes = 256 / pix_bytes (at least 1)
    p.kshift = pix_bytes >= 256 ? 0 : (pix_bytes == 128 ? 1 : (pix_bytes == 64 ? 2 : 3));
    p.K = fh * fw * ic;
    p.per_xcd = blocks % 8 == 0 ? (int)(blocks / 8) : 0;
    p.div_ow = FastDiv((uint32_t)ow);
    p.div_tiles = FastDiv((uint32_t)tiles);
    p.div_octiles = FastDiv((uint32_t)octiles);
    p.div_vec = FastDiv((uint32_t)(iw / CPC));
    static bool attr_done = false;
    if (!attr_done) {
        AGH_HIP(hipFuncSetAttribute((const void *)conv2_mfma_kernel<T>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_limit));
        attr_done = true;
    }
    hipLaunchKernelGGL(conv2_mfma_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), (size_t)smem, stream(), (const T *)x,
                       (const T *)wperm, (const T *)bias, (T *)y, p);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template int conv2_mfma_try<uint16_t>(const char *, const void *, const void *, const void *, void *, int64_t, int64_t, int64_t, int64_t,
                                      int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int);
template int conv2_mfma_try<float>(const char *, const void *, const void *, const void *, void *, int64_t, int64_t, int64_t, int64_t,
                                   int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int64_t, int);

}  // namespace agh

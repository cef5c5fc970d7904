// Conv2 forward as an implicit GEMM on the matrix cores (bf16, unit stride and dilation): the patch
// matrix of im2col is never written.  A workgroup takes 256 consecutive output positions of one image
// and up to 128 output channels; it stages the input rows those positions touch ONCE in LDS, pixel
// major with the channels of a pixel contiguous, and then runs the k loop (filter tap, then 16
// channels per step) without a single barrier: the A operand of v_mfma_f32_32x32x16_bf16 (32
// positions x 16 channels of one tap) is a 16-byte LDS read per lane, the B operand (32 output
// channels x the same 16 k) comes straight from a fragment-ordered copy of the filter bank, which is
// small and stays in L2.  HBM traffic is the image in and the activation out, a tenth of
// what im2col + GEMM move; bias and ReLU are applied in the epilogue in the order the separate
// layers round.  Sums are f32 in k order (tap, channel), one rounding at the end, so results agree
// with the im2col chain within its bf16 tolerance, not bit for bit.
#include <type_traits>

#include "agh_internal.h"

using namespace agh;

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));

constexpr int kThreads = 256;
constexpr int kTilePos = 256;  // output positions per workgroup (8 MFMA tiles of 32)
constexpr int kTileOc = 128;   // output channels per workgroup (4 MFMA tiles of 32)
constexpr int kEpitch = 4 * 64 + 16;  // bytes per staged output-channel row in the epilogue (128 positions + pad)

struct ConvMfmaParams {
    int bs, ic, ih, iw, oc, oh, ow, fh, fw, ph, pw;
    int act, has_bias;
    int npos, tiles_per_img, oc_tiles;
    int lcols;     // staged columns: iw + 2*pw
    int nch_mask;  // ic/8 - 1 (16-byte chunks per pixel, a power of two)
    int kshift;    // log2(pixels per 256 bytes): the swizzle key of pixel q is (q >> kshift) & nch_mask
    int K;         // fh*fw*ic
    FastDiv div_ow, div_tiles, div_octiles, div_vec;
};

// Filter bank [oc][ic][fh][fw] -> MFMA B-fragment order: for every tile of 32 output channels and every
// k step s = tap * (ic/16) + c/16, one contiguous 1 KB block holding lane (kg, n)'s 8 values
// (channels 16*(c/16) + 8*kg .. +7 of output channel n) at position lane = 32*kg + n.  A wave then
// fetches a fragment with ONE fully coalesced 16-byte-per-lane load.
__global__ __launch_bounds__(kThreads) void pack_filter_kernel(const uint16_t *__restrict__ w, uint16_t *__restrict__ wp,
                                                                int ic, int ff, int nsteps, size_t total) {
    const size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;  // source index: [o][c][tap]
    if (e >= total) return;
    const size_t per_o = (size_t)ic * ff;
    const size_t o = e / per_o;
    const int r = (int)(e - o * per_o);
    const int c = r / ff, tap = r - c * ff;
    const int s = tap * (ic >> 4) + (c >> 4), kg = (c >> 3) & 1, i = c & 7;
    const size_t dst = ((((o >> 5) * nsteps + s) * 64) + kg * 32 + (o & 31)) * 8 + i;
    wp[dst] = w[e];
}

__global__ __launch_bounds__(kThreads, 2) void conv2_mfma_bf16_kernel(const uint16_t *__restrict__ x, const uint16_t *__restrict__ wp,
                                                                      const uint16_t *__restrict__ bias, uint16_t *__restrict__ y,
                                                                      ConvMfmaParams p) {
    extern __shared__ __align__(16) unsigned char lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave & 1, wn = wave >> 1;
    uint32_t t0, oct, b, tile;
    p.div_octiles.divmod(blockIdx.x, t0, oct);
    p.div_tiles.divmod(t0, b, tile);
    const int p0 = tile * kTilePos;
    const int plast = min(p0 + kTilePos, p.npos) - 1;
    const int ho_first = p.div_ow.div((uint32_t)p0), ho_last = p.div_ow.div((uint32_t)plast);
    const int lrows = ho_last - ho_first + p.fh;  // staged input rows
    const int pix_bytes = p.ic * 2;

    // ---- stage the input rows: items = (row, channel pair, 8-column vector) ----
    // The 16-byte channel chunks of pixel q are stored at chunk ^ key(q), key(q) = ((q >> kshift) + (q >> 4)) &
    // nch_mask.  The lanes of a ds_read_b128 of the k loop address 16 consecutive pixels and the same chunk:
    // the first term puts those 16 reads on 16 different 16-byte columns of the 256-byte LDS row.  The lanes
    // of a staging write address pixels 8 apart: the second term spreads those as well.
    {
        const int nvec = p.iw >> 3, npair = p.ic >> 1;
        const uint32_t items = (uint32_t)lrows * npair * nvec;
        // batches of SB items per thread: all 2*SB global loads are issued before the first LDS write
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
                    const uint16_t *src = x + (((size_t)b * p.ic + 2 * c2) * p.ih + hi) * (size_t)p.iw + v * 8;
                    r0[u] = *(const uint4 *)src;
                    r1[u] = *(const uint4 *)(src + (size_t)p.ih * p.iw);
                }
                const int c = 2 * (int)c2;
                pix0[u] = (int)lr * p.lcols + p.pw + (int)v * 8;
                base[u] = it < items ? pix0[u] * pix_bytes + (c & 7) * 2 : -1;
                cpart[u] = c >> 3;
            }
#pragma unroll
            for (int u = 0; u < SB; ++u) {
                if (base[u] < 0) continue;
                const uint32_t lo[4] = {r0[u].x, r0[u].y, r0[u].z, r0[u].w}, hi2[4] = {r1[u].x, r1[u].y, r1[u].z, r1[u].w};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const uint32_t a = (lo[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu, bb = (hi2[j >> 1] >> ((j & 1) * 16)) & 0xFFFFu;
                    const int addr = base[u] + j * pix_bytes + ((cpart[u] ^ ((((pix0[u] + j) >> p.kshift) + ((pix0[u] + j) >> 4)) & p.nch_mask)) << 4);
                    *(uint32_t *)(lds + addr) = a | (bb << 16);
                }
            }
        }
        // padding columns left and right of the image
        const int npadcol = p.lcols - p.iw, nch = p.nch_mask + 1;
        const uint32_t pads = (uint32_t)lrows * npadcol * nch;
        for (uint32_t it = tid; it < pads; it += kThreads) {
            const uint32_t ch = it % nch, rc = it / nch;
            const uint32_t k = rc % npadcol, lr = rc / npadcol;
            const int col = (int)k < p.pw ? (int)k : p.iw + (int)k;
            *(uint4 *)(lds + ((int)lr * p.lcols + col) * pix_bytes + (ch << 4)) = make_uint4(0, 0, 0, 0);
        }
    }

    // ---- per-lane operand addressing ----
    const int kg = lane >> 5, l32 = lane & 31;
    int apix[4], acol[4];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        const int pp = min(p0 + (wm * 4 + mt) * 32 + l32, p.npos - 1);  // clamped: a duplicate, never stored
        uint32_t ho, wo;
        p.div_ow.divmod((uint32_t)pp, ho, wo);
        apix[mt] = ((int)ho - ho_first) * p.lcols + (int)wo;
        acol[mt] = (int)wo;
    }
    const int nsteps = p.fh * p.fw * (p.ic >> 4);
    const int oc0 = oct * kTileOc + wn * 64;
    const bool wave_live = oc0 < p.oc;  // oc is a multiple of 64
    const uint16_t *brow[2];
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)  // fragment-ordered bank: block (tile of 32 channels, step), 8 elements per lane
        brow[nt] = wp + ((size_t)(min(oc0 + nt * 32, p.oc - 32) >> 5) * nsteps * 64 + lane) * 8;

    f32x16 acc[4][2];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int nt = 0; nt < 2; ++nt) acc[mt][nt] = (f32x16)(0.0f);

    __syncthreads();

    // ---- k loop: taps outer, 16 channels per step, operands of step s+1 requested before the MFMAs of step s ----
    const int ncc = p.ic >> 4;
    int fi = 0, fj = 0, cc = 0;  // position of the NEXT step to load
    int abase[4], akey[4];          // byte address of the lane's pixel for tap (0,0); swizzle key of the current tap, << 4
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        abase[mt] = apix[mt] * pix_bytes;
        akey[mt] = (((apix[mt] >> p.kshift) + (apix[mt] >> 4)) & p.nch_mask) << 4;
    }
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
    auto advance_a = [&]() {
        if (++cc == ncc) {
            cc = 0;
            if (++fj == p.fw) { fj = 0; ++fi; }
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const int q = apix[mt] + fi * p.lcols + fj;
                akey[mt] = (((q >> p.kshift) + (q >> 4)) & p.nch_mask) << 4;
            }
        }
    };
    auto load_b_part = [&](uint4(&bq)[2], int s, auto ntc) {
        constexpr int nt = decltype(ntc)::value;
        bq[nt] = *(const uint4 *)(brow[nt] + (size_t)min(s, nsteps - 1) * (64 * 8));
    };
    auto mma = [&](const uint4(&a)[4], const uint4(&bq)[2], auto nc) {
        constexpr int n = decltype(nc)::value, mt = n >> 1, nt = n & 1;
        acc[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a[mt]), __builtin_bit_cast(bf16x8_t, bq[nt]),
                                                              acc[mt][nt], 0, 0, 0);
    };
    using I0 = std::integral_constant<int, 0>;
    using I1 = std::integral_constant<int, 1>;
    using I2 = std::integral_constant<int, 2>;
    using I3 = std::integral_constant<int, 3>;
    using I4 = std::integral_constant<int, 4>;
    using I5 = std::integral_constant<int, 5>;
    using I6 = std::integral_constant<int, 6>;
    using I7 = std::integral_constant<int, 7>;
    // One step: the eight MFMAs of step s on (a, b), with the fetches of step s+1's A fragments (into an)
    // and of step s+3's B fragments (into bn) handed out between them, one per MFMA.  sched_barrier pins
    // the order, so the matrix pipe gets a new MFMA every 32 cycles while the other requests trickle out.
    // No branch surrounds a load: one that would run past the last step re-reads a valid location (with
    // conditional loads the compiler can no longer count outstanding loads and waits for all of them).
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
    if (wave_live) {
        uint4 a0[4], a1[4], b0[2], b1[2], b2[2], b3[2];
        load_b_part(b0, 0, I0{}); load_b_part(b0, 0, I1{});
        load_b_part(b1, 1, I0{}); load_b_part(b1, 1, I1{});
        load_b_part(b2, 2, I0{}); load_b_part(b2, 2, I1{});
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
            if (p.has_bias) bq = bf16_to_f32(bias[min(o_lane, p.oc - 1)]);
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int blk = 0; blk < 4; ++blk) {
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
                    const int pl = mt * 32 + blk * 8 + kg * 4;  // position inside the wave's 128
                    *(uint2 *)(region + l32 * kEpitch + pl * 2) = make_uint2(w[0], w[1]);
                }
            // same wave, LDS executes in order: the reads below see the writes above
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const int row = r * 4 + (lane >> 4), chunk = lane & 15;
                const uint4 v = *(const uint4 *)(region + row * kEpitch + chunk * 16);
                const int pos = p0 + wm * 128 + chunk * 8, o = oc0 + nt * 32 + row;
                if (pos < p.npos && o < p.oc) *(uint4 *)(y + ((size_t)b * p.oc + o) * p.npos + pos) = v;
            }
        }
    }
}

}  // namespace

namespace agh {

// Returns 1 when the geometry is not one this kernel takes (the caller goes on to its other paths),
// otherwise a status code.  The API lock is held by the caller.
int conv2_mfma_bf16_try(const char *name, const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic,
                        int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t oh,
                        int64_t ow, int act) {
    const bool pow2 = (ic & (ic - 1)) == 0;
    const int64_t npos = oh * ow;
    if (!pow2 || ic < 16 || ic > 256 || oc % 64 != 0 || iw % 8 != 0 || npos % 8 != 0 || fh * fw > 64) return 1;
    if ((((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) & 15) != 0) return 1;
    // little work per output: the LDS-resident scalar kernels do better on small problems
    if (ic * fh * fw < 128 || npos < 256) return 1;
    const int64_t lcols = iw + 2 * pw;
    const int64_t rows_out = std::min<int64_t>(oh, (kTilePos - 1) / ow + 2);
    const int64_t tile_bytes = (rows_out + fh - 1) * lcols * ic * 2;
    const int64_t smem = std::max<int64_t>(tile_bytes, 4 * 32 * kEpitch);
    if (smem > 64 * 1024) return 1;
    const int64_t tiles = (npos + kTilePos - 1) / kTilePos, octiles = (oc + kTileOc - 1) / kTileOc;
    const int64_t blocks = bs * tiles * octiles;
    if (blocks > 0x7FFFFFFFll || bs * ic * ih * iw > ((int64_t)1 << 40)) return 1;

    void *wperm = nullptr;
    const size_t wtotal = (size_t)(oc * ic * fh * fw);
    if (int rc = workspace(wtotal * 2, &wperm)) return rc;
    hipLaunchKernelGGL(pack_filter_kernel, dim3((unsigned)((wtotal + kThreads - 1) / kThreads)), dim3(kThreads), 0, stream(),
                       (const uint16_t *)w, (uint16_t *)wperm, (int)ic, (int)(fh * fw), (int)(fh * fw * (ic / 16)), wtotal);
    AGH_LAUNCH_CHECK(name);

    ConvMfmaParams p;
    p.bs = bs; p.ic = ic; p.ih = ih; p.iw = iw; p.oc = oc; p.oh = oh; p.ow = ow; p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw;
    p.act = act; p.has_bias = bias != nullptr;
    p.npos = npos; p.tiles_per_img = tiles; p.oc_tiles = octiles; p.lcols = lcols;
    p.nch_mask = ic / 8 - 1;
    p.kshift = ic >= 128 ? 0 : (ic == 64 ? 1 : (ic == 32 ? 2 : 3));
    p.K = fh * fw * ic;
    p.div_ow = FastDiv((uint32_t)ow);
    p.div_tiles = FastDiv((uint32_t)tiles);
    p.div_octiles = FastDiv((uint32_t)octiles);
    p.div_vec = FastDiv((uint32_t)(iw / 8));
    static bool attr_done = false;
    if (!attr_done) {
        AGH_HIP(hipFuncSetAttribute((const void *)conv2_mfma_bf16_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024));
        attr_done = true;
    }
    hipLaunchKernelGGL(conv2_mfma_bf16_kernel, dim3((unsigned)blocks), dim3(kThreads), (size_t)smem, stream(),
                       (const uint16_t *)x, (const uint16_t *)wperm, (const uint16_t *)bias, (uint16_t *)y, p);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

}  // namespace agh

// Direct 2-D convolution for small channel counts (the LeNet5-sized layers), with the
// ReLU and the 2x2/stride-2 MaxPool2 that follow such a layer optionally fused in.
//
// Conv2::forward in the reference goes im2col -> dot -> NHWC->NCHW copy on a device
// (src/learn/neural_network/layer.rs:950-1005) and through a register-tiled direct kernel on
// the host (layer/conv_direct.rs:23-83).  For layers whose whole input image and filter bank
// fit in LDS, materialising the patch matrix is pure overhead (conv1 of LeNet5 at batch 1000
// would write and re-read 57.6 MB to do 173 MFLOP), so this kernel convolves straight out of
// LDS:
//   - a workgroup stages `imgs` input images (converted to f32) and the filter bank,
//     transposed to [tap][oc] so that the OCT output channels of a work item are one vector
//     read at a wave-uniform address (an LDS broadcast);
//   - a work item owns one output pixel - or, with the pool fused, one 2x2 pool window - for
//     OCT output channels, and walks the taps (ci, fi, fj) accumulating in f32 registers;
//   - the epilogue applies, in the order the separate layers would: round to T, add bias in T,
//     ReLU (x >= 0 ? x : 0), first-strict-maximum over the window in row-major order, and
//     writes NCHW directly.
#include "agh_internal.h"

using namespace agh;

namespace {

struct ConvParams {
    int bs, ic, ih, iw, oc, oh, ow;
    int fh, fw, ph, pw, sh, sw, dh, dw;
    int act, has_bias;
    int imgs;      // images per workgroup
    int ngroups;   // ceil(oc / OCT)
    int ocpad;     // ngroups * OCT
    int yh, yw;    // output tensor spatial size (pooled or not)
    int items_per_img;
    FastDiv div_items, div_pix, div_yw;
};

template <typename T>
__device__ __forceinline__ T round_bias_relu(float acc, bool has_bias, T bias, int act) {
    T r = Elem<T>::from_f32(acc);
    const T rb = Elem<T>::from_f32(Elem<T>::to_f32(bias) + Elem<T>::to_f32(r));
    r = has_bias ? rb : r;
    const bool neg = !(Elem<T>::to_f32(r) >= 0.0f);
    return (act == AGH_ACT_RELU && neg) ? Elem<T>::zero() : r;
}

// Fills n LDS slots from global memory with U reads of a thread in flight at a time: `get(e)` reads (it is called
// with e < n only and must not fault), `put(e, v)` stores.  Written as two unrolled passes because a plain
// `for (e...) lds[e] = g[...]` loop compiles to one read, one wait and one store per trip, and a workgroup that stages
// a few thousand values that way spends most of its life in a dozen memory round trips one after another.
template <int U, typename V, typename Get, typename Put>
__device__ __forceinline__ void staged_fill(int n, Get get, Put put) {
    const int step = (int)blockDim.x;
    for (int base = (int)threadIdx.x; base < n; base += U * step) {
        V v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = get(min(base + u * step, n - 1));
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (base + u * step < n) put(base + u * step, v[u]);
    }
}

// The two halves of staged_fill for one batch of U slots starting at slot `first`, so that a kernel can put the
// reads of several regions (filter bank, images) in flight before it stores any of them.
template <int U, typename V, typename Get>
__device__ __forceinline__ void batch_read(V (&v)[U], int first, int n, Get get) {
    const int step = (int)blockDim.x, base = first + (int)threadIdx.x;
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = get(min(base + u * step, n - 1));
}
template <int U, typename V, typename Put>
__device__ __forceinline__ void batch_store(const V (&v)[U], int first, int n, Put put) {
    const int step = (int)blockDim.x, base = first + (int)threadIdx.x;
#pragma unroll
    for (int u = 0; u < U; ++u)
        if (base + u * step < n) put(base + u * step, v[u]);
}
// slots [first, n) by staged_fill
template <int U, typename V, typename Get, typename Put>
__device__ __forceinline__ void staged_fill_from(int first, int n, Get get, Put put) {
    const int step = (int)blockDim.x;
    for (int base = first + (int)threadIdx.x; base < n; base += U * step) {
        V v[U];
#pragma unroll
        for (int u = 0; u < U; ++u) v[u] = get(min(base + u * step, n - 1));
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (base + u * step < n) put(base + u * step, v[u]);
    }
}

template <typename T, int OCT, bool POOL>
__global__ __launch_bounds__(256) void conv2_direct_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                            const T *__restrict__ bias, T *__restrict__ y,
                                                            ConvParams p) {
    extern __shared__ __align__(16) float smem_f[];
    const int taps = p.ic * p.fh * p.fw;
    float *ws = smem_f;                         // [taps][ocpad]
    float *xs = smem_f + (size_t)taps * p.ocpad;  // [imgs][ic][ih][iw]
    const int img_sz = p.ic * p.ih * p.iw;
    const int b0 = blockIdx.x * p.imgs;
    const int nimg = min(p.imgs, p.bs - b0);

    staged_fill<8, T>(
        taps * p.ocpad,
        [&](int e) {
            const int tap = e / p.ocpad, o = min(e - tap * p.ocpad, p.oc - 1);
            return w[(size_t)o * taps + tap];
        },
        [&](int e, T v) { ws[e] = (e % p.ocpad) < p.oc ? Elem<T>::to_f32(v) : 0.0f; });
    const T *xb = x + (size_t)b0 * img_sz;
    staged_fill<8, T>(nimg * img_sz, [&](int e) { return xb[e]; }, [&](int e, T v) { xs[e] = Elem<T>::to_f32(v); });
    __syncthreads();

    constexpr int NPIX = POOL ? 4 : 1;
    const int total = nimg * p.items_per_img;
    for (int item = threadIdx.x; item < total; item += blockDim.x) {
        uint32_t img, r0, grp, pix, py, px;
        p.div_items.divmod((uint32_t)item, img, r0);
        p.div_pix.divmod(r0, grp, pix);  // pixel fastest: neighbouring lanes write neighbouring outputs
        p.div_yw.divmod(pix, py, px);
        const float *xi = xs + (size_t)img * img_sz;
        const float *wg = ws + grp * OCT;

        float acc[NPIX][OCT];
#pragma unroll
        for (int a = 0; a < NPIX; ++a)
#pragma unroll
            for (int o = 0; o < OCT; ++o) acc[a][o] = 0.0f;
        // top-left input coordinate of each of the NPIX output pixels
        int h0[NPIX], w0[NPIX];
#pragma unroll
        for (int a = 0; a < NPIX; ++a) {
            const int ho = POOL ? 2 * (int)py + (a >> 1) : (int)py;
            const int wo = POOL ? 2 * (int)px + (a & 1) : (int)px;
            h0[a] = -p.ph + p.sh * ho;
            w0[a] = -p.pw + p.sw * wo;
        }
        int tap = 0;
        for (int ci = 0; ci < p.ic; ++ci) {
            const float *xc = xi + ci * p.ih * p.iw;
            for (int fi = 0; fi < p.fh; ++fi)
                for (int fj = 0; fj < p.fw; ++fj, ++tap) {
                    float wv[OCT];
#pragma unroll
                    for (int o = 0; o < OCT; ++o) wv[o] = wg[tap * p.ocpad + o];
#pragma unroll
                    for (int a = 0; a < NPIX; ++a) {
                        const int hi = h0[a] + fi * p.dh, wi = w0[a] + fj * p.dw;
                        const bool ok = hi >= 0 && hi < p.ih && wi >= 0 && wi < p.iw;
                        const float v = ok ? xc[hi * p.iw + wi] : 0.0f;
#pragma unroll
                        for (int o = 0; o < OCT; ++o) acc[a][o] = __builtin_fmaf(v, wv[o], acc[a][o]);
                    }
                }
        }
#pragma unroll
        for (int o = 0; o < OCT; ++o) {
            const int oc = grp * OCT + o;
            const bool live = oc < p.oc;  // (no `continue`: the loop must unroll so acc stays in registers)
            const T bv = (p.has_bias && live) ? bias[oc] : Elem<T>::zero();
            T m = round_bias_relu<T>(acc[0][o], p.has_bias != 0, bv, p.act);
            if (POOL) {
                float mf = Elem<T>::to_f32(m);
#pragma unroll
                for (int a = 1; a < NPIX; ++a) {
                    const T v = round_bias_relu<T>(acc[a][o], p.has_bias != 0, bv, p.act);
                    const float vf = Elem<T>::to_f32(v);
                    if (vf > mf) { m = v; mf = vf; }
                }
            }
            if (live) y[(((size_t)(b0 + img) * p.oc + oc) * p.yh + py) * p.yw + px] = m;
        }
    }
}

// ---- row-tiled variant for stride 1, dilation 1 (any padding) ----
//
// A work item computes WT = 8 consecutive output pixels of one output row - or, with the pool
// fused, of a PAIR of rows, i.e. four whole pool windows - for OCT output channels.  The staged
// image is zero-padded in LDS, so the inner loop has no bounds checks: per (channel, input row)
// it reads WT + FW - 1 input values once (three 16-byte LDS reads) and the FW x OCT filter values
// of the filter row(s) that input row meets (uniform addresses, LDS broadcasts), then does up to
// 2 * FW * WT * OCT FMAs out of registers - about 12 FMAs per LDS read instead of 3.
struct RowTileParams {
    int bs, ic, ih, iw, oc, oh, ow, fh, ph, pw;
    int act, has_bias;
    int imgs, ngroups, ocpad;
    int ihp, pitch;       // padded rows staged per channel, LDS row pitch (floats, multiple of 4)
    int nwb;              // WT-wide blocks per output row
    int nrows;            // output rows (or row pairs with the pool) per image
    int yh, yw;
    int items_per_img;
    FastDiv div_items, div_rowsxwb, div_nwb, div_ocpad, div_pitch, div_ihp;
};

template <typename T, int FW, int OCT, bool POOL, int FHC>  // FHC: the filter height when it equals FW, else 0 (run time)
__global__ __launch_bounds__(256) void conv2_rowtile_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                             const T *__restrict__ bias, T *__restrict__ y,
                                                             RowTileParams p) {
    constexpr int WT = 8, NR = POOL ? 2 : 1, XW = WT + FW - 1, XV = (XW + 3) / 4;
    extern __shared__ __align__(16) float smem_f[];
    // a filter height known at compile time unrolls the row loop: which filter row an input row meets is then decided
    // at compile time, not by branches around every group of FMAs (LeNet5 conv1: 10.3 -> 9.0 us)
    constexpr int kUnrollRows = FHC ? FHC + (POOL ? 1 : 0) : 1;
    const int fh = FHC ? FHC : p.fh;
    const int taps = p.ic * fh * FW;
    float *ws = smem_f;                                         // [ic][fh][FW][ocpad]
    float *xs = smem_f + (((size_t)taps * p.ocpad + 3) & ~(size_t)3);  // [imgs][ic][ihp][pitch], zero padded
    const int ch_sz = p.ihp * p.pitch, img_sz = p.ic * ch_sz;
    const int b0 = blockIdx.x * p.imgs;
    const int nimg = min(p.imgs, p.bs - b0);

    staged_fill<8, T>(
        taps * p.ocpad,
        [&](int e) {
            uint32_t tap, o;
            p.div_ocpad.divmod((uint32_t)e, tap, o);
            return w[(size_t)min((int)o, p.oc - 1) * taps + tap];
        },
        [&](int e, T v) {
            uint32_t tap, o;
            p.div_ocpad.divmod((uint32_t)e, tap, o);
            ws[e] = (int)o < p.oc ? Elem<T>::to_f32(v) : 0.0f;
        });
    // the padding cells read the nearest cell of the image (a valid address) and store zero
    auto cell = [&](int e, int &hi, int &wi) -> size_t {
        uint32_t r1, col, r2, row;  // r2 = img * ic + channel
        p.div_pitch.divmod((uint32_t)e, r1, col);
        p.div_ihp.divmod(r1, r2, row);
        hi = (int)row - p.ph;
        wi = (int)col - p.pw;
        return ((size_t)b0 * p.ic + r2) * p.ih * p.iw;
    };
    staged_fill<8, T>(
        nimg * img_sz,
        [&](int e) {
            int hi, wi;
            const size_t plane = cell(e, hi, wi);
            return x[plane + (size_t)min(max(hi, 0), p.ih - 1) * p.iw + min(max(wi, 0), p.iw - 1)];
        },
        [&](int e, T v) {
            int hi, wi;
            cell(e, hi, wi);
            xs[e] = (hi >= 0 && hi < p.ih && wi >= 0 && wi < p.iw) ? Elem<T>::to_f32(v) : 0.0f;
        });
    __syncthreads();

    const int total = nimg * p.items_per_img;
    for (int item = threadIdx.x; item < total; item += blockDim.x) {
        uint32_t img, r0, grp, r1, row, wb;
        p.div_items.divmod((uint32_t)item, img, r0);
        p.div_rowsxwb.divmod(r0, grp, r1);
        p.div_nwb.divmod(r1, row, wb);
        const int ho0 = POOL ? 2 * (int)row : (int)row;  // first output row of this item
        const float *xi = xs + (size_t)img * img_sz + ho0 * p.pitch + wb * WT;
        const float *wg = ws + grp * OCT;

        float acc[NR][WT][OCT];
#pragma unroll
        for (int a = 0; a < NR; ++a)
#pragma unroll
            for (int t = 0; t < WT; ++t)
#pragma unroll
                for (int o = 0; o < OCT; ++o) acc[a][t][o] = 0.0f;

        for (int ci = 0; ci < p.ic; ++ci) {
            const float *xc = xi + ci * ch_sz;
            const float *wc = wg + (size_t)ci * fh * FW * p.ocpad;
            // input row r (relative to ho0) meets filter row r of output row 0 and r-1 of output row 1
#pragma unroll kUnrollRows
            for (int r = 0; r < fh + NR - 1; ++r) {
                float xin[XV * 4];
#pragma unroll
                for (int v = 0; v < XV; ++v) {
                    const float4 q = *(const float4 *)(xc + r * p.pitch + 4 * v);
                    xin[4 * v + 0] = q.x; xin[4 * v + 1] = q.y; xin[4 * v + 2] = q.z; xin[4 * v + 3] = q.w;
                }
#pragma unroll
                for (int a = 0; a < NR; ++a) {
                    const int fi = r - a;
                    if (fi >= 0 && fi < fh) {
                        const float *wr = wc + fi * FW * p.ocpad;
#pragma unroll
                        for (int fj = 0; fj < FW; ++fj) {
                            float wv[OCT];
#pragma unroll
                            for (int o = 0; o < OCT; ++o) wv[o] = wr[fj * p.ocpad + o];
#pragma unroll
                            for (int t = 0; t < WT; ++t)
#pragma unroll
                                for (int o = 0; o < OCT; ++o)
                                    acc[a][t][o] = __builtin_fmaf(xin[t + fj], wv[o], acc[a][t][o]);
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int o = 0; o < OCT; ++o) {
            const int oc = grp * OCT + o;
            const bool live = oc < p.oc;
            const T bv = (p.has_bias && live) ? bias[oc] : Elem<T>::zero();
            T *yp = y + (((size_t)(b0 + img) * p.oc + (live ? oc : 0)) * p.yh + row) * p.yw;
            if (POOL) {
#pragma unroll
                for (int j = 0; j < WT / 2; ++j) {
                    // window in row-major order: (0,2j) (0,2j+1) (1,2j) (1,2j+1); first strict maximum wins
                    T m = round_bias_relu<T>(acc[0][2 * j][o], p.has_bias != 0, bv, p.act);
                    float mf = Elem<T>::to_f32(m);
                    const T v1 = round_bias_relu<T>(acc[0][2 * j + 1][o], p.has_bias != 0, bv, p.act);
                    const T v2 = round_bias_relu<T>(acc[NR - 1][2 * j][o], p.has_bias != 0, bv, p.act);
                    const T v3 = round_bias_relu<T>(acc[NR - 1][2 * j + 1][o], p.has_bias != 0, bv, p.act);
                    float f = Elem<T>::to_f32(v1);
                    if (f > mf) { m = v1; mf = f; }
                    f = Elem<T>::to_f32(v2);
                    if (f > mf) { m = v2; mf = f; }
                    f = Elem<T>::to_f32(v3);
                    if (f > mf) { m = v3; mf = f; }
                    const int px = wb * (WT / 2) + j;
                    if (live && px < p.yw) yp[px] = m;
                }
            } else {
#pragma unroll
                for (int t = 0; t < WT; ++t) {
                    const int px = wb * WT + t;
                    if (live && px < p.yw) yp[px] = round_bias_relu<T>(acc[0][t][o], p.has_bias != 0, bv, p.act);
                }
            }
        }
    }
}

// ---- few channels, small images: implicit GEMM on v_mfma_f32_16x16x4_f32 ----
//
// The layers of small networks (LeNet5's conv2: 6 -> 16 channels on 12 x 12 images) have too few outputs per image to
// fill the chip with register tiles and too many multiply-adds per output (150) for one thread each: the row-tiled
// kernel spends 17 us on conv2 at batch 1000, three quarters of it a single wave per SIMD walking its 2400 FMAs.
// Here the same staged (zero-padded) images feed the matrix pipes: a 16 x 16 x 4 MFMA takes 16 output positions of one
// image (rows), up to 16 output channels (columns) and 4 taps.  The A operand is gathered straight from the staged
// image, one 4-byte LDS read per lane (position base + tap offset; the offsets of all taps sit in a small LDS table);
// the B operand is the filter bank as [tap][16] in LDS.  With the pool fused, the 16 rows of a tile are 4 whole 2 x 2
// windows, cell-minor: the accumulator layout (lane group g holds rows 4g .. 4g+3) then leaves each lane one complete
// window of one channel, and bias, ReLU and the first-strict-maximum pooling happen in registers.
// A wave takes (image, TG consecutive tiles) units; the k loop runs in chunks of 8 steps whose B values and tap
// offsets are fetched one chunk ahead.  f32 accumulation like every other kernel here; the summation order over the
// taps differs from the row-tiled kernel's (4 partial chains), which the f32 tolerance of the tests covers.
struct SmallMfmaParams {
    int bs, ic, ih, iw, oc, oh, ow, fh, fw, ph, pw;
    int act, has_bias;
    int imgs;           // images per workgroup
    int ihp, pitch;     // staged rows per channel and their pitch (floats)
    int ktot, ksteps;   // taps; k steps of 4 (a multiple of 8, the taps beyond ktot multiply zeros)
    int nout;           // results per image and channel: positions, or windows with the pool
    int mtiles;         // 16-row tiles per image
    int units_per_img;  // ceil(mtiles / TG)
    int yw;             // width of the result (pooled or not)
    FastDiv div_pitch, div_ihp, div_yw, div_fw, div_fhfw, div_upi;
};
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <typename T, bool POOL, int TG>
__global__ __launch_bounds__(256) void conv2_small_mfma_kernel(const T *__restrict__ x, const T *__restrict__ w,
                                                                const T *__restrict__ bias, T *__restrict__ y,
                                                                SmallMfmaParams p) {
    extern __shared__ __align__(16) float smem_f[];
    const int kpad = p.ksteps * 4;
    float *Bs = smem_f;                          // [kpad][16]
    int *tapoff = (int *)(smem_f + kpad * 16);   // [kpad], byte offsets into a staged image
    float *xs = smem_f + kpad * 17;              // [imgs][ic][ihp][pitch], zero padded
    const int ch_sz = p.ihp * p.pitch, img_sz = p.ic * ch_sz;
    const int b0 = blockIdx.x * p.imgs;
    const int nimg = min(p.imgs, p.bs - b0);

    for (int k = threadIdx.x; k < kpad; k += blockDim.x) {
        uint32_t ci, rem, fi, fj;
        p.div_fhfw.divmod((uint32_t)min(k, p.ktot - 1), ci, rem);
        p.div_fw.divmod(rem, fi, fj);
        tapoff[k] = (int)(ci * ch_sz + fi * p.pitch + fj) * 4;
    }
    // a padding cell reads the nearest cell of the image (a valid address) and stores zero
    auto cell = [&](int e, int &hi, int &wi) -> size_t {
        uint32_t r1, col, r2, row;  // r2 = img * ic + channel
        p.div_pitch.divmod((uint32_t)e, r1, col);
        p.div_ihp.divmod(r1, r2, row);
        hi = (int)row - p.ph;
        wi = (int)col - p.pw;
        return ((size_t)b0 * p.ic + r2) * p.ih * p.iw;
    };
    const int nw = kpad * 16, nx = nimg * img_sz;
    auto get_w = [&](int e) { return w[(size_t)min(e & 15, p.oc - 1) * p.ktot + min(e >> 4, p.ktot - 1)]; };
    auto put_w = [&](int e, T v) { Bs[e] = ((e & 15) < p.oc && (e >> 4) < p.ktot) ? Elem<T>::to_f32(v) : 0.0f; };
    constexpr int WU = 12, XU = 8;
    T wv[WU], xv[XU];
    batch_read<WU>(wv, 0, nw, get_w);
    if (p.ph == 0 && p.pw == 0) {  // nothing to pad: the staged images are a copy
        const T *xb = x + (size_t)b0 * img_sz;
        auto get_x = [&](int e) { return xb[e]; };
        auto put_x = [&](int e, T v) { xs[e] = Elem<T>::to_f32(v); };
        batch_read<XU>(xv, 0, nx, get_x);
        batch_store<WU>(wv, 0, nw, put_w);
        batch_store<XU>(xv, 0, nx, put_x);
        staged_fill_from<8, T>(XU * (int)blockDim.x, nx, get_x, put_x);
    } else {
        auto get_x = [&](int e) {
            int hi, wi;
            const size_t plane = cell(e, hi, wi);
            return x[plane + (size_t)min(max(hi, 0), p.ih - 1) * p.iw + min(max(wi, 0), p.iw - 1)];
        };
        auto put_x = [&](int e, T v) {
            int hi, wi;
            cell(e, hi, wi);
            xs[e] = (hi >= 0 && hi < p.ih && wi >= 0 && wi < p.iw) ? Elem<T>::to_f32(v) : 0.0f;
        };
        batch_read<XU>(xv, 0, nx, get_x);
        batch_store<WU>(wv, 0, nw, put_w);
        batch_store<XU>(xv, 0, nx, put_x);
        staged_fill_from<8, T>(XU * (int)blockDim.x, nx, get_x, put_x);
    }
    staged_fill_from<8, T>(WU * (int)blockDim.x, nw, get_w, put_w);
    __syncthreads();

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, i = lane & 15;
    const int nunits = nimg * p.units_per_img;
    const char *Bl = (const char *)(Bs + lane);
    const char *tl = (const char *)(tapoff + g);
    for (int u = wave; u < nunits; u += 4) {
        uint32_t img, ug;
        p.div_upi.divmod((uint32_t)u, img, ug);
        const int tile0 = (int)ug * TG;
        // this lane's A row of every tile: byte offset of the position's top-left input cell in LDS
        const char *abase[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) {
            const int tile = min(tile0 + t, p.mtiles - 1);
            uint32_t oy, ox;
            if (POOL) {
                uint32_t py, px;
                p.div_yw.divmod((uint32_t)min(tile * 4 + (i >> 2), p.nout - 1), py, px);
                oy = 2 * py + ((i >> 1) & 1);
                ox = 2 * px + (i & 1);
            } else {
                p.div_yw.divmod((uint32_t)min(tile * 16 + i, p.nout - 1), oy, ox);
            }
            abase[t] = (const char *)(xs + (size_t)img * img_sz + oy * p.pitch + ox);
        }
        f32x4_t acc[TG];
#pragma unroll
        for (int t = 0; t < TG; ++t) acc[t] = f32x4_t{0.0f, 0.0f, 0.0f, 0.0f};
        float bq[8];
        int tq[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            bq[q] = *(const float *)(Bl + q * 256);
            tq[q] = *(const int *)(tl + q * 16);
        }
        for (int s0 = 0; s0 < p.ksteps; s0 += 8) {
            float bc[8];
            int tc[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) { bc[q] = bq[q]; tc[q] = tq[q]; }
            if (s0 + 8 < p.ksteps) {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    bq[q] = *(const float *)(Bl + (s0 + 8 + q) * 256);
                    tq[q] = *(const int *)(tl + (s0 + 8 + q) * 16);
                }
            }
            // the taps behind ktot multiply zeros of the bank; their A values are zeroed too (0 * inf would poison the
            // sum), which only the last chunk has to look at
            const bool tail = s0 + 8 >= p.ksteps;
#pragma unroll
            for (int q = 0; q < 8; ++q)
#pragma unroll
                for (int t = 0; t < TG; ++t) {
                    float a = *(const float *)(abase[t] + tc[q]);
                    if (tail && 4 * (s0 + q) + g >= p.ktot) a = 0.0f;
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bc[q], acc[t], 0, 0, 0);
                }
        }
        // lane (g, i) holds rows 4g .. 4g+3 of column i: one window (pool) or 4 consecutive positions of channel i
        const bool live = i < p.oc;
        const T bv = (p.has_bias && live) ? bias[i] : Elem<T>::zero();
        T *yc = y + ((size_t)(b0 + img) * p.oc + (live ? i : 0)) * p.nout;
#pragma unroll
        for (int t = 0; t < TG; ++t) {
            const int tile = tile0 + t;
            if (tile >= p.mtiles) break;
            if (POOL) {
                T m = round_bias_relu<T>(acc[t][0], p.has_bias != 0, bv, p.act);
                float mf = Elem<T>::to_f32(m);
#pragma unroll
                for (int r = 1; r < 4; ++r) {
                    const T v = round_bias_relu<T>(acc[t][r], p.has_bias != 0, bv, p.act);
                    const float f = Elem<T>::to_f32(v);
                    if (f > mf) { m = v; mf = f; }
                }
                const int wi = tile * 4 + g;
                if (live && wi < p.nout) yc[wi] = m;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int pos = tile * 16 + 4 * g + r;
                    if (live && pos < p.nout) yc[pos] = round_bias_relu<T>(acc[t][r], p.has_bias != 0, bv, p.act);
                }
            }
        }
    }
}

// ---- LeNet5 inference in one launch ----
//
// The model of the reference's benchmark (benches/neural-network-benches/src/
// autograph_backend.rs:88-162): conv 1->6 5x5, relu, pool 2x2, conv 6->16 5x5, relu, pool 2x2,
// flatten, dense 256->128, relu, dense 128->84, relu, dense 84->10 + bias.  At batch 1000 the
// whole forward pass is 0.57 GFLOP; run layer by layer it is bound by launch latency and by
// round trips of tiny activations through HBM.  Here a workgroup takes IMGS images through all
// twelve layers with every activation in LDS: the two conv+relu+pool stages use the same
// row-tiled inner loop as conv2_rowtile_kernel, the Dense stages are LDS-broadcast dot products
// against weights read (coalesced) from L2.  Activations are rounded to T after every layer,
// exactly where the layer-by-layer path rounds, so both paths agree per layer up to f32
// summation order.
template <int FW, int OCT, int WT>
__device__ __forceinline__ void rowpair_conv(const float *xi, int ch_sz, int pitch, int ic, int fh, const float *wg,
                                             int ocpad, float (&acc)[2][WT][OCT]) {
    constexpr int XW = WT + FW - 1, XV = (XW + 3) / 4;
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int t = 0; t < WT; ++t)
#pragma unroll
            for (int o = 0; o < OCT; ++o) acc[a][t][o] = 0.0f;
    for (int ci = 0; ci < ic; ++ci) {
        const float *xc = xi + ci * ch_sz;
        const float *wc = wg + (size_t)ci * fh * FW * ocpad;
        for (int r = 0; r < fh + 1; ++r) {
            float xin[XV * 4];
#pragma unroll
            for (int v = 0; v < XV; ++v) {
                const float4 q = *(const float4 *)(xc + r * pitch + 4 * v);
                xin[4 * v + 0] = q.x; xin[4 * v + 1] = q.y; xin[4 * v + 2] = q.z; xin[4 * v + 3] = q.w;
            }
#pragma unroll
            for (int a = 0; a < 2; ++a) {
                const int fi = r - a;
                if (fi >= 0 && fi < fh) {
                    const float *wr = wc + fi * FW * ocpad;
#pragma unroll
                    for (int fj = 0; fj < FW; ++fj) {
                        float wv[OCT];
#pragma unroll
                        for (int o = 0; o < OCT; ++o) wv[o] = wr[fj * ocpad + o];
#pragma unroll
                        for (int t = 0; t < WT; ++t)
#pragma unroll
                            for (int o = 0; o < OCT; ++o) acc[a][t][o] = __builtin_fmaf(xin[t + fj], wv[o], acc[a][t][o]);
                    }
                }
            }
        }
    }
}

// relu + first-strict-maximum pooling of window j of a row pair, rounding to T first
template <typename T, int OCT, int WT>
__device__ __forceinline__ float relu_pool_window(const float (&acc)[2][WT][OCT], int j, int o) {
    const T zero = Elem<T>::zero();
    T m = round_bias_relu<T>(acc[0][2 * j][o], false, zero, AGH_ACT_RELU);
    float mf = Elem<T>::to_f32(m);
    const T v1 = round_bias_relu<T>(acc[0][2 * j + 1][o], false, zero, AGH_ACT_RELU);
    const T v2 = round_bias_relu<T>(acc[1][2 * j][o], false, zero, AGH_ACT_RELU);
    const T v3 = round_bias_relu<T>(acc[1][2 * j + 1][o], false, zero, AGH_ACT_RELU);
    float f = Elem<T>::to_f32(v1);
    if (f > mf) mf = f;
    f = Elem<T>::to_f32(v2);
    if (f > mf) mf = f;
    f = Elem<T>::to_f32(v3);
    if (f > mf) mf = f;
    return mf;  // activations stay in LDS as f32 copies of the T values
}

// What a training step needs from the forward pass besides the logits (all [bs, ...] in standard layout): the
// convolution outputs before the relu (c1 [6,24,24], c2 [16,8,8]), the pooled activations (p1 [6,12,12], p2 [16,4,4]),
// and the dense layers' outputs before (d1 [128], d2 [84]) and after (a1, a2) the relu.
template <typename T>
struct LenetSaves {
    T *c1, *p1, *c2, *p2, *d1, *a1, *d2, *a2;
};

// N consecutive activations (N * sizeof(T) a multiple of 4 bytes, destination aligned to that size) rounded to T and
// stored with the widest vector stores
template <typename T, int N>
__device__ __forceinline__ void store_rounded(T *dst, const float (&v)[N]) {
    if constexpr (sizeof(T) == 4) {
        if constexpr (N % 4 == 0) {
#pragma unroll
            for (int i = 0; i < N; i += 4) *(float4 *)((float *)dst + i) = make_float4(v[i], v[i + 1], v[i + 2], v[i + 3]);
        } else {
#pragma unroll
            for (int i = 0; i < N; i += 2) *(float2 *)((float *)dst + i) = make_float2(v[i], v[i + 1]);
        }
    } else {
        uint32_t w[N / 2];
#pragma unroll
        for (int i = 0; i < N / 2; ++i) w[i] = f32x2_to_bf16x2(v[2 * i], v[2 * i + 1]);
        if constexpr (N == 8) *(uint4 *)dst = make_uint4(w[0], w[1], w[2], w[3]);
        else if constexpr (N == 4) *(uint2 *)dst = make_uint2(w[0], w[1]);
        else *(uint32_t *)dst = w[0];
    }
}

// 16 bytes per lane from global memory straight into LDS: lane L's data lands at lds_base + 16 L (lds_base is
// wave-uniform and travels in M0).  Inline assembly, so the compiler's wait counting does not know it: whoever reads
// the destination waits with s_waitcnt vmcnt(0) and a barrier first.
__device__ __forceinline__ void lds_direct_load16(const void *gptr, uint32_t lds_base_uniform) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
                 :
                 : "v"(gptr), "s"(__builtin_amdgcn_readfirstlane((int)lds_base_uniform))
                 : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_address_of(const void *p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const unsigned char *)p;
}

// waves_per_eu(2, 2): eight waves per workgroup are two per SIMD whatever the register count; without the hint the
// compiler aimed the bf16 training instantiation at 128 registers and gave up the early weight loads for it (30 us
// instead of 20)
// IMGS images per workgroup.  4: a batch of a thousand is one round of 250 workgroups.  1 (batches up to 256, e.g. the
// training step's hundred): the same 512 threads share ONE image, every stage cut finer (conv1 in 2 x 4 register tiles,
// conv2's taps split between two waves per pooled row), so that a stage takes a quarter of the time: the launch is a
// chain of stage latencies, and with four images per workgroup a small batch would leave most of the chip idle while
// each busy CU walks four images' worth of every stage.
template <typename T, bool SAVE, int IMGS>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) void lenet5_forward_kernel(const T *__restrict__ x, const T *__restrict__ w1,
                                                              const T *__restrict__ w2, const T *__restrict__ wd1,
                                                              const T *__restrict__ wd2, const T *__restrict__ wd3,
                                                              const T *__restrict__ b3, T *__restrict__ out, int bs,
                                                              LenetSaves<T> sv, int w23_aligned) {
    static_assert(IMGS == 1 || IMGS == 4, "one image or four per workgroup");
    __shared__ __align__(16) float xs[IMGS * 28 * 28];     // input images, pitch 28
    __shared__ __align__(16) float w1s[25 * 6];            // [tap][oc]
    __shared__ __align__(16) float p1[IMGS * 6 * 12 * 12]; // after conv1 + relu + pool
    __shared__ __align__(16) float w2s[160 * 16];          // [ci][fi][fj][oc], ten rows of zeros behind the 150 taps
    __shared__ int tap2[160];                              // byte offset of tap k inside an image of p1 (0 behind the taps)
    __shared__ __align__(16) float p2[IMGS * 256];         // after conv2 + relu + pool, flattened [c][h][w]
    __shared__ __align__(16) float d1[IMGS * 128];
    __shared__ __align__(16) float d2[IMGS * 84];
    __shared__ __align__(16) float parts[16 * IMGS * 128];  // dense1 partial sums
    __shared__ __align__(16) T wd2s[128 * 84];              // dense2 / dense3 weights as they lie in memory
    __shared__ __align__(16) T wd3s[1024];                  // (84 * 10, rounded up to whole KB)
    constexpr int NT = 512;  // 8 waves: two per SIMD, so one can wait on LDS while the other multiplies
    constexpr int kD3Off = 4 * IMGS * 84;  // dense3's partial sums in `parts`, behind dense2's
    const int tid = threadIdx.x;
    const int b0 = blockIdx.x * IMGS;
    const int nimg = min(IMGS, bs - b0);

    // Everything staged is read first and stored afterwards, so that the reads are all in flight together: written as
    // `lds[e] = global[...]` loops they compile to one read, one wait and one store per trip (a dozen memory round trips
    // one after another, 3 of the launch's 16 us).  Addresses are clamped, what lies outside is stored as zero.
    {
        constexpr int XU = (IMGS * 784 + NT - 1) / NT;  // 7 image values a thread
        const int nx = nimg * 784;
        T w1v, w2v[5], xv[XU];
        {
            const int e = min(tid, 149), tap = e / 6, o = e - tap * 6;
            w1v = w1[o * 25 + tap];
        }
#pragma unroll
        for (int u = 0; u < 5; ++u) {
            const int e = tid + u * NT, tap = e >> 4, o = e & 15;
            w2v[u] = w2[o * 150 + min(tap, 149)];
        }
        const T *xb = x + (size_t)b0 * 784;
#pragma unroll
        for (int u = 0; u < XU; ++u) xv[u] = xb[min(tid + u * NT, nx - 1)];
        if (tid < 150) w1s[tid] = Elem<T>::to_f32(w1v);
#pragma unroll
        for (int u = 0; u < 5; ++u) {
            const int e = tid + u * NT;
            w2s[e] = (e >> 4) < 150 ? Elem<T>::to_f32(w2v[u]) : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < XU; ++u) {
            const int e = tid + u * NT;
            if (e < IMGS * 784) xs[e] = e < nx ? Elem<T>::to_f32(xv[u]) : 0.0f;
        }
    }
    if (tid < 160) {
        const int k = min(tid, 149), ci = k / 25, rem = k - ci * 25, fi = rem / 5, fj = rem - fi * 5;
        tap2[tid] = tid < 150 ? (ci * 144 + fi * 12 + fj) * 4 : 0;
    }
    // dense1 weights of this thread (see the dense1 stage below), requested now, used much later
    float4 wreg[16];
    {
        const int cg = tid & 31, kg = tid >> 5;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
            const T *src = wd1 + (size_t)(kg * 16 + kk) * 128 + cg * 4;
            if constexpr (sizeof(T) == 4) {
                wreg[kk] = *(const float4 *)src;
            } else {
                const uint2 raw = *(const uint2 *)src;
                wreg[kk] = make_float4(bf16_to_f32((uint16_t)(raw.x & 0xFFFF)), bf16_to_f32((uint16_t)(raw.x >> 16)),
                                       bf16_to_f32((uint16_t)(raw.y & 0xFFFF)), bf16_to_f32((uint16_t)(raw.y >> 16)));
            }
        }
    }
    // The weights of the last two dense layers travel into LDS behind everything requested so far, 1 KB per
    // instruction without passing through registers, while the convolution stages run: read where they are used
    // (130 loads per thread, each waiting on L2) they cost the launch 3 of its 16 us.
    {
        constexpr int kW2Bytes = 128 * 84 * (int)sizeof(T), kW3Bytes = 84 * 10 * (int)sizeof(T);
        static_assert(kW2Bytes % 1024 == 0 && kW3Bytes % 16 == 0, "whole direct loads");
        const int lane = tid & 63, wave = tid >> 6;
        if (w23_aligned) {
            for (int c = wave; c < kW2Bytes / 1024; c += NT / 64)
                lds_direct_load16((const char *)wd2 + c * 1024 + lane * 16, lds_address_of(wd2s) + c * 1024);
            for (int c = wave; c < (kW3Bytes + 1023) / 1024; c += NT / 64)
                lds_direct_load16((const char *)wd3 + min(c * 1024 + lane * 16, kW3Bytes - 16), lds_address_of(wd3s) + c * 1024);
        } else {  // views at odd offsets: element copies
            for (int e = tid; e < 128 * 84; e += NT) wd2s[e] = wd2[e];
            for (int e = tid; e < 840; e += NT) wd3s[e] = wd3[e];
        }
    }
    __syncthreads();

    // conv1 (1->6, 5x5) + relu + pool
    if constexpr (IMGS == 1) {
        // items = 6 channels x 12 row pairs x 6 column blocks of 4
        if (tid < 432) {
            const int oc = tid / 72, r1 = tid - oc * 72, row = r1 / 6, wb = r1 - row * 6;
            float acc[2][4][1];
            rowpair_conv<5, 1, 4>(xs + 2 * row * 28 + wb * 4, 784, 28, 1, 5, w1s + oc, 6, acc);
#pragma unroll
            for (int j = 0; j < 2; ++j) p1[(oc * 12 + row) * 12 + wb * 2 + j] = relu_pool_window<T, 1, 4>(acc, j, 0);
            if constexpr (SAVE) {
                const size_t plane = (size_t)b0 * 6 + oc;
#pragma unroll
                for (int a = 0; a < 2; ++a) {
                    float v[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[t] = acc[a][t][0];
                    store_rounded<T, 4>(sv.c1 + (plane * 24 + 2 * row + a) * 24 + wb * 4, v);
                }
                const float q[2] = {p1[(oc * 12 + row) * 12 + wb * 2], p1[(oc * 12 + row) * 12 + wb * 2 + 1]};
                store_rounded<T, 2>(sv.p1 + (plane * 12 + row) * 12 + wb * 2, q);
            }
        }
    } else if (tid < IMGS * 108) {  // items = img x 3 channel pairs x 12 row pairs x 3 column blocks of 8
        const int img = tid / 108, r0 = tid - img * 108;
        const int grp = r0 / 36, r1 = r0 - grp * 36;
        const int row = r1 / 3, wb = r1 - row * 3;
        float acc[2][8][2];
        rowpair_conv<5, 2, 8>(xs + img * 784 + 2 * row * 28 + wb * 8, 784, 28, 1, 5, w1s + grp * 2, 6, acc);
#pragma unroll
        for (int o = 0; o < 2; ++o)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                p1[((img * 6 + grp * 2 + o) * 12 + row) * 12 + wb * 4 + j] = relu_pool_window<T, 2, 8>(acc, j, o);
        if constexpr (SAVE) {
            if (img < nimg) {
#pragma unroll
                for (int o = 0; o < 2; ++o) {
                    const size_t plane = (size_t)(b0 + img) * 6 + grp * 2 + o;
#pragma unroll
                    for (int a = 0; a < 2; ++a) {
                        float v[8];
#pragma unroll
                        for (int t = 0; t < 8; ++t) v[t] = acc[a][t][o];
                        store_rounded<T, 8>(sv.c1 + (plane * 24 + 2 * row + a) * 24 + wb * 8, v);
                    }
                    float q[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) q[j] = p1[((img * 6 + grp * 2 + o) * 12 + row) * 12 + wb * 4 + j];
                    store_rounded<T, 4>(sv.p1 + (plane * 12 + row) * 12 + wb * 4, q);
                }
            }
        }
    }
    __syncthreads();

    // conv2 (6->16, 5x5) + relu + pool on v_mfma_f32_16x16x4_f32, as conv2_small_mfma_kernel does it: an MFMA takes the
    // 4 pool windows of one pooled row (16 positions, cell-minor) x 16 channels x 4 taps, the A operand gathered from
    // p1 through the tap table.  Wave w: image w / 2, pooled rows 2 (w % 2) and 2 (w % 2) + 1; 40 steps of 4 taps.
    if constexpr (IMGS == 1) {
        // one image: wave w takes pooled row w % 4 and half w / 4 of the 40 steps; the halves are added through LDS
        const int lane = tid & 63, wave = tid >> 6, g = lane >> 4, i = lane & 15;
        const int row = wave & 3, kh = wave >> 2;
        const char *abase = (const char *)(p1 + (2 * row + ((i >> 1) & 1)) * 12 + 2 * (i >> 2) + (i & 1));
        const char *Bl = (const char *)(w2s + lane) + kh * 20 * 256, *tl = (const char *)(tap2 + g) + kh * 20 * 16;
        f32x4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        float bq[20];
        int tq[20];
#pragma unroll
        for (int q = 0; q < 20; ++q) {
            bq[q] = *(const float *)(Bl + q * 256);
            tq[q] = *(const int *)(tl + q * 16);
        }
#pragma unroll
        for (int q = 0; q < 20; ++q) {
            float a = *(const float *)(abase + tq[q]);
            if (4 * (kh * 20 + q) + g >= 150) a = 0.0f;  // behind the taps: zero times zero, whatever p1 holds
            acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bq[q], acc, 0, 0, 0);
        }
        f32x4_t *xch = (f32x4_t *)parts;  // free until dense1
        if (kh == 1) xch[row * 64 + lane] = acc;
        __syncthreads();
        if (kh == 0) {
            acc += xch[row * 64 + lane];
            const T zero = Elem<T>::zero();
            float mf = Elem<T>::to_f32(round_bias_relu<T>(acc[0], false, zero, AGH_ACT_RELU));
#pragma unroll
            for (int r = 1; r < 4; ++r) {
                const float f = Elem<T>::to_f32(round_bias_relu<T>(acc[r], false, zero, AGH_ACT_RELU));
                if (f > mf) mf = f;
            }
            p2[(i * 4 + row) * 4 + g] = mf;
            if constexpr (SAVE) {
                const size_t plane = (size_t)b0 * 16 + i;
#pragma unroll
                for (int dy = 0; dy < 2; ++dy) {
                    const float v[2] = {acc[2 * dy], acc[2 * dy + 1]};
                    store_rounded<T, 2>(sv.c2 + (plane * 8 + 2 * row + dy) * 8 + 2 * g, v);
                }
                sv.p2[(plane * 4 + row) * 4 + g] = Elem<T>::from_f32(mf);
            }
        }
    } else
    {
        const int lane = tid & 63, wave = tid >> 6, g = lane >> 4, i = lane & 15;
        const int img = wave >> 1, tile0 = (wave & 1) * 2;
        const char *abase[2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
            abase[t] = (const char *)(p1 + img * 864 + (2 * (tile0 + t) + ((i >> 1) & 1)) * 12 + 2 * (i >> 2) + (i & 1));
        const char *Bl = (const char *)(w2s + lane), *tl = (const char *)(tap2 + g);
        f32x4_t acc[2] = {f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}, f32x4_t{0.0f, 0.0f, 0.0f, 0.0f}};
        float bq[8];
        int tq[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            bq[q] = *(const float *)(Bl + q * 256);
            tq[q] = *(const int *)(tl + q * 16);
        }
#pragma unroll
        for (int s0 = 0; s0 < 40; s0 += 8) {
            float bc[8];
            int tc[8];
#pragma unroll
            for (int q = 0; q < 8; ++q) { bc[q] = bq[q]; tc[q] = tq[q]; }
            if (s0 + 8 < 40) {
#pragma unroll
                for (int q = 0; q < 8; ++q) {
                    bq[q] = *(const float *)(Bl + (s0 + 8 + q) * 256);
                    tq[q] = *(const int *)(tl + (s0 + 8 + q) * 16);
                }
            }
#pragma unroll
            for (int q = 0; q < 8; ++q)
#pragma unroll
                for (int t = 0; t < 2; ++t) {
                    float a = *(const float *)(abase[t] + tc[q]);
                    if (4 * (s0 + q) + g >= 150) a = 0.0f;  // behind the taps: zero times zero, whatever p1 holds (s0, q constants)
                    acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, bc[q], acc[t], 0, 0, 0);
                }
        }
        // lane (g, i): channel i, pooled column g; acc[t][2 dy + dx] is cell (dy, dx) of the window in pooled row tile0 + t
        const T zero = Elem<T>::zero();
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const int row = tile0 + t;
            float mf = Elem<T>::to_f32(round_bias_relu<T>(acc[t][0], false, zero, AGH_ACT_RELU));
#pragma unroll
            for (int r = 1; r < 4; ++r) {
                const float f = Elem<T>::to_f32(round_bias_relu<T>(acc[t][r], false, zero, AGH_ACT_RELU));
                if (f > mf) mf = f;
            }
            p2[img * 256 + (i * 4 + row) * 4 + g] = mf;
            if constexpr (SAVE) {
                if (img < nimg) {
                    const size_t plane = (size_t)(b0 + img) * 16 + i;
#pragma unroll
                    for (int dy = 0; dy < 2; ++dy) {
                        const float v[2] = {acc[t][2 * dy], acc[t][2 * dy + 1]};
                        store_rounded<T, 2>(sv.c2 + (plane * 8 + 2 * row + dy) * 8 + 2 * g, v);
                    }
                    sv.p2[(plane * 4 + row) * 4 + g] = Elem<T>::from_f32(mf);
                }
            }
        }
    }
    __syncthreads();

    // dense1 256 -> 128 + relu.  Thread (cg, kg) owns the weights W1[16kg .. 16kg+15][4cg .. 4cg+3]; they
    // were fetched into registers at the top of the kernel (16 coalesced 16-byte loads per thread, in
    // flight during both convolution stages).  Each thread forms its 4 columns x 4 images partial sums
    // over its 16 k, the 16 k-groups are then added through LDS in a fixed order.
    {
        const int cg = tid & 31, kg = tid >> 5;
        float part[IMGS][4];
#pragma unroll
        for (int r = 0; r < IMGS; ++r)
#pragma unroll
            for (int c = 0; c < 4; ++c) part[r][c] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 16; kk += 4) {
            float4 xv[IMGS];
#pragma unroll
            for (int r = 0; r < IMGS; ++r) xv[r] = *(const float4 *)(p2 + r * 256 + kg * 16 + kk);
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const float4 wv = wreg[kk + u];
#pragma unroll
                for (int r = 0; r < IMGS; ++r) {
                    const float xk = u == 0 ? xv[r].x : u == 1 ? xv[r].y : u == 2 ? xv[r].z : xv[r].w;
                    part[r][0] = __builtin_fmaf(xk, wv.x, part[r][0]);
                    part[r][1] = __builtin_fmaf(xk, wv.y, part[r][1]);
                    part[r][2] = __builtin_fmaf(xk, wv.z, part[r][2]);
                    part[r][3] = __builtin_fmaf(xk, wv.w, part[r][3]);
                }
            }
        }
        // xs and p1 are free by now: the [kg][img][128] partials (16*4*128 floats = 32 KB) do not fit xs
        // alone, so they go to a buffer of their own
#pragma unroll
        for (int r = 0; r < IMGS; ++r)
            *(float4 *)(parts + (kg * IMGS + r) * 128 + cg * 4) = make_float4(part[r][0], part[r][1], part[r][2], part[r][3]);
    }
    __syncthreads();
    if (tid < IMGS * 128) {
        const int o = tid;
        float a = 0.0f;
#pragma unroll
        for (int kg = 0; kg < 16; ++kg) a += parts[kg * IMGS * 128 + o];
        const T act = round_bias_relu<T>(a, false, Elem<T>::zero(), AGH_ACT_RELU);
        d1[o] = Elem<T>::to_f32(act);
        if constexpr (SAVE) {
            if ((o >> 7) < nimg) {
                sv.d1[(size_t)b0 * 128 + o] = Elem<T>::from_f32(a);
                sv.a1[(size_t)b0 * 128 + o] = act;
            }
        }
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the direct loads of wd2s / wd3s (not known to the compiler)
    __syncthreads();
    // dense2 128 -> 84 + relu, weights from LDS.  Thread (c, kq) forms the partial sums of output c over a quarter of k
    // for all four images (four independent chains of 32, each weight read once); the quarters are then added in order
    // through LDS (`parts` is free again).  One thread per output over all of k is a chain of 128 dependent FMAs behind
    // 256 LDS reads: 1.6 us of the launch.
    if (tid < 4 * 84) {
        const int kq = tid / 84, c = tid - kq * 84;
        float part[IMGS];
#pragma unroll
        for (int r = 0; r < IMGS; ++r) part[r] = 0.0f;
#pragma unroll
        for (int kk = 0; kk < 32; kk += 4) {
            const int k = kq * 32 + kk;
            float4 xk[IMGS];
#pragma unroll
            for (int r = 0; r < IMGS; ++r) xk[r] = *(const float4 *)(d1 + r * 128 + k);
            const float w0 = Elem<T>::to_f32(wd2s[k * 84 + c]), w1v = Elem<T>::to_f32(wd2s[(k + 1) * 84 + c]);
            const float w2v = Elem<T>::to_f32(wd2s[(k + 2) * 84 + c]), w3v = Elem<T>::to_f32(wd2s[(k + 3) * 84 + c]);
#pragma unroll
            for (int r = 0; r < IMGS; ++r) {
                part[r] = __builtin_fmaf(xk[r].x, w0, part[r]);
                part[r] = __builtin_fmaf(xk[r].y, w1v, part[r]);
                part[r] = __builtin_fmaf(xk[r].z, w2v, part[r]);
                part[r] = __builtin_fmaf(xk[r].w, w3v, part[r]);
            }
        }
#pragma unroll
        for (int r = 0; r < IMGS; ++r) parts[(kq * IMGS + r) * 84 + c] = part[r];
    }
    __syncthreads();
    if (tid < IMGS * 84) {
        const int r = tid / 84;
        float a = parts[tid];
#pragma unroll
        for (int kq = 1; kq < 4; ++kq) a += parts[kq * IMGS * 84 + tid];
        const T act = round_bias_relu<T>(a, false, Elem<T>::zero(), AGH_ACT_RELU);
        d2[tid] = Elem<T>::to_f32(act);
        if constexpr (SAVE) {
            if (r < nimg) {
                sv.d2[(size_t)b0 * 84 + tid] = Elem<T>::from_f32(a);
                sv.a2[(size_t)b0 * 84 + tid] = act;
            }
        }
    }
    __syncthreads();
    // dense3 84 -> 10 + bias: thread (kp, r, c) sums 12 of the 84 products, the seven parts are added in order
    if (tid < 7 * IMGS * 10) {
        const int kp = tid / (IMGS * 10), rc = tid - kp * (IMGS * 10), r = rc / 10, c = rc - r * 10;
        float a = 0.0f;
        const float *xr = d2 + r * 84 + kp * 12;
#pragma unroll
        for (int kk = 0; kk < 12; kk += 4) {
            const float4 xk = *(const float4 *)(xr + kk);
            const int k = kp * 12 + kk;
            a = __builtin_fmaf(xk.x, Elem<T>::to_f32(wd3s[k * 10 + c]), a);
            a = __builtin_fmaf(xk.y, Elem<T>::to_f32(wd3s[(k + 1) * 10 + c]), a);
            a = __builtin_fmaf(xk.z, Elem<T>::to_f32(wd3s[(k + 2) * 10 + c]), a);
            a = __builtin_fmaf(xk.w, Elem<T>::to_f32(wd3s[(k + 3) * 10 + c]), a);
        }
        parts[kD3Off + tid] = a;  // behind the dense2 partials, which other waves may still be reading
    }
    __syncthreads();
    if (tid < IMGS * 10) {
        const int r = tid / 10, c = tid - r * 10;
        float a = parts[kD3Off + tid];
#pragma unroll
        for (int kp = 1; kp < 7; ++kp) a += parts[kD3Off + kp * IMGS * 10 + tid];
        if (r < nimg) out[(size_t)(b0 + r) * 10 + c] = round_bias_relu<T>(a, true, b3[c], AGH_ACT_NONE);
    }
}

// The input-gradient chain of a LeNet5 training step in one launch, one workgroup per image: cross-entropy backward,
// the three dense layers' input gradients with their relu backward, pooling + relu backward of conv2's output written as
// the [64, 16] matrix its weight gradient multiplies, conv2's input gradient (dot with the filter bank, then col2im),
// pooling + relu backward of conv1's output as the [576, 6] matrix.  Every value is rounded to T where the separate
// launches round it, and every T-typed running sum adds in their order (col2im: filter rows and columns descending,
// the dot over the output channels ascending), so the results differ from theirs only through the order of the f32
// adds inside the dense dot products.
template <typename T>
struct LenetBackward {
    const T *logits;            // [bs, 10]
    const uint8_t *target;      // [bs]
    const T *c1, *c2, *d1, *d2; // conv outputs before relu [bs,6,24,24], [bs,16,8,8]; dense outputs before relu [bs,128], [bs,84]
    const T *w2, *wd1, *wd2, *wd3;
    T *g_logits, *g_d2, *g_d1;  // [bs,10], [bs,84], [bs,128]
    T *gm2, *gm1;               // [bs*64, 16], [bs*576, 6]
    float dy;                   // upstream gradient of the summed loss divided by the batch size
};

// pooling (2x2, stride 2) backward through a relu, one window: g lands on the first maximum of relu(x) and passes where
// x >= 0 (the rule of max_pool2_relu_backward_2x2_kernel); cell k = 2 * row + column
template <typename T>
__device__ __forceinline__ void pool_relu_window_backward(const T (&xv)[4], float gy, T (&cell)[4]) {
    auto relu_of = [](T v) { return Elem<T>::raw(v) >= 0.0f ? v : Elem<T>::zero(); };
    float mf = Elem<T>::raw(relu_of(xv[0]));
    int am = 0;
#pragma unroll
    for (int k = 1; k < 4; ++k) {
        const float vf = Elem<T>::raw(relu_of(xv[k]));
        if (vf > mf) { mf = vf; am = k; }
    }
    const T g = Elem<T>::from_f32(0.0f + gy);
#pragma unroll
    for (int k = 0; k < 4; ++k) cell[k] = (am == k && Elem<T>::raw(xv[k]) >= 0.0f) ? g : Elem<T>::zero();
}

template <typename T>
__global__ __launch_bounds__(256) void lenet5_backward_kernel(LenetBackward<T> a) {
    __shared__ __align__(16) float wl[150 * 16];   // conv2's filter bank, [ci*25 + fi*5 + fj][oc]
    __shared__ __align__(16) float gm2s[64 * 16];  // gradient of conv2's output, [y*8 + x][oc]
    __shared__ float gls[16], gd2s[84], gd1s[128], gfs[256], gp1s[864];
    constexpr int kPmPitch = 151;                  // odd: the col2im reads of neighbouring pixels fall into different banks
    __shared__ float pm[64 * kPmPitch];            // gm2 . W, every entry rounded to T
    constexpr int NT = 256;
    constexpr int EPV = 16 / (int)sizeof(T);  // elements per 16-byte load
    const int tid = threadIdx.x;
    const size_t b = blockIdx.x;
    // Everything this workgroup reads from memory has an address known now, so all of it is requested here, before the
    // first use: the stages below are a chain of seven short steps, and a load issued inside a step would add its L2
    // latency to that chain.  (About 100 registers per thread; the launch is 100 workgroups, occupancy is no concern.)
    T w2v[10];  // the filter bank, coalesced: element tid + u * 256 of w2[oc][ci*25 + tap]
#pragma unroll
    for (int u = 0; u < 10; ++u) w2v[u] = a.w2[min(tid + u * NT, 2399)];
    T lrow[10];  // the image's logits (used by the ten threads of the first stage)
#pragma unroll
    for (int j = 0; j < 10; ++j) lrow[j] = a.logits[b * 10 + j];
    const int label = a.target[b];
    T w3v[10];   // row min(tid, 83) of wd3
#pragma unroll
    for (int c = 0; c < 10; ++c) w3v[c] = a.wd3[min(tid, 83) * 10 + c];
    const T d2v = a.d2[b * 84 + min(tid, 83)], d1v = a.d1[b * 128 + (tid & 127)];
    uint2 w2r[84 * (int)sizeof(T) / 8];  // row tid & 127 of wd2 (84 elements: 8-byte aligned)
    {
        const uint2 *src = (const uint2 *)(a.wd2 + (tid & 127) * 84);
#pragma unroll
        for (int c = 0; c < 84 * (int)sizeof(T) / 8; ++c) w2r[c] = src[c];
    }
    uint4 w1r[128 / EPV];  // row tid of wd1
    {
        const uint4 *src = (const uint4 *)(a.wd1 + tid * 128);
#pragma unroll
        for (int c = 0; c < 128 / EPV; ++c) w1r[c] = src[c];
    }
    T x2[4];  // the thread's pooling window of conv2's output
    {
        const int oc = tid >> 4, ho = (tid >> 2) & 3, wo = tid & 3;
        const T *xp = a.c2 + ((b * 16 + oc) * 8 + 2 * ho) * 8 + 2 * wo;
        x2[0] = xp[0]; x2[1] = xp[1]; x2[2] = xp[8]; x2[3] = xp[9];
    }
    T x1[4][4];  // its (up to four) pooling windows of conv1's output
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int e = min(tid + u * NT, 863);
        const int ci = e / 144, r = e - ci * 144, ho = r / 12, wo = r - ho * 12;
        const T *xp = a.c1 + ((b * 6 + ci) * 24 + 2 * ho) * 24 + 2 * wo;
        x1[u][0] = xp[0]; x1[u][1] = xp[1]; x1[u][2] = xp[24]; x1[u][3] = xp[25];
    }
    auto elem = [](const auto &packed, int c) -> float {  // element c of a row held as 8- or 16-byte words
        if constexpr (sizeof(T) == 4) return __uint_as_float(((const uint32_t *)&packed)[c]);
        else {
            const uint32_t w = ((const uint32_t *)&packed)[c >> 1];
            return __uint_as_float((c & 1) ? (w & 0xFFFF0000u) : (w << 16));
        }
    };

    // cross-entropy backward (softmax - one-hot, times dy), rounded to T
    if (tid < 10) {
        float m = Elem<T>::to_f32(lrow[0]);
#pragma unroll
        for (int j = 0; j < 10; ++j) m = fmaxf(m, Elem<T>::to_f32(lrow[j]));
        float s = 0.0f;
#pragma unroll
        for (int j = 0; j < 10; ++j) s += expf(Elem<T>::to_f32(lrow[j]) - m);
        float mine = 0.0f;
#pragma unroll
        for (int j = 0; j < 10; ++j) mine = j == tid ? Elem<T>::to_f32(lrow[j]) : mine;
        const float pr = expf(mine - m) / s;
        const T g = Elem<T>::from_f32(a.dy * (pr - (tid == label ? 1.0f : 0.0f)));
        a.g_logits[b * 10 + tid] = g;
        gls[tid] = Elem<T>::to_f32(g);
    }
#pragma unroll
    for (int u = 0; u < 10; ++u) {
        const int i = tid + u * NT;
        const int o = i / 150, k = i - o * 150;
        if (i < 2400) wl[k * 16 + o] = Elem<T>::to_f32(w2v[u]);
    }
    __syncthreads();
    // dense3: g_a2 = g_logits . wd3^T (wd3 [84, 10]), then relu backward on dense2's pre-activation
    if (tid < 84) {
        float d = 0.0f;
#pragma unroll
        for (int c = 0; c < 10; ++c) d = __builtin_fmaf(gls[c], Elem<T>::to_f32(w3v[c]), d);
        const T ga = Elem<T>::from_f32(d);
        const T gd = Elem<T>::raw(d2v) >= 0.0f ? ga : Elem<T>::zero();
        a.g_d2[b * 84 + tid] = gd;
        gd2s[tid] = Elem<T>::to_f32(gd);
    }
    __syncthreads();
    // dense2: g_a1 = g_d2 . wd2^T (wd2 [128, 84]), relu backward on dense1's pre-activation
    if (tid < 128) {
        float d = 0.0f;
#pragma unroll
        for (int c = 0; c < 84; ++c) d = __builtin_fmaf(gd2s[c], elem(w2r, c), d);
        const T ga = Elem<T>::from_f32(d);
        const T gd = Elem<T>::raw(d1v) >= 0.0f ? ga : Elem<T>::zero();
        a.g_d1[b * 128 + tid] = gd;
        gd1s[tid] = Elem<T>::to_f32(gd);
    }
    __syncthreads();
    // dense1: g_f = g_d1 . wd1^T (wd1 [256, 128])
    {
        float d = 0.0f;
#pragma unroll
        for (int c = 0; c < 128; ++c) d = __builtin_fmaf(gd1s[c], elem(w1r, c), d);
        gfs[tid] = Elem<T>::to_f32(Elem<T>::from_f32(d));
    }
    __syncthreads();
    // pooling + relu backward of conv2's output: one window per thread (16 channels x 4 x 4 windows)
    {
        const int oc = tid >> 4, ho = (tid >> 2) & 3, wo = tid & 3;
        T cell[4];
        pool_relu_window_backward<T>(x2, gfs[tid], cell);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int pos = (2 * ho + (k >> 1)) * 8 + 2 * wo + (k & 1);
            gm2s[pos * 16 + oc] = Elem<T>::to_f32(cell[k]);
            a.gm2[(b * 64 + pos) * 16 + oc] = cell[k];
        }
    }
    __syncthreads();
    // conv2's input gradient in two steps, as the host does it.  First the product gm2 . W, a [64, 150] matrix whose
    // entries are f32 dots over the 16 output channels (ascending) rounded to T: a thread owns 4 positions x 10 taps and
    // keeps its four gradient rows in registers, so an entry costs a fraction of the LDS reads a per-pixel walk would need.
    if (tid < 240) {
        const int pg = tid / 15, kg = tid - pg * 15;
        float4 g[4][4];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
            for (int q = 0; q < 4; ++q) g[r][q] = *(const float4 *)(gm2s + (pg * 4 + r) * 16 + q * 4);
#pragma unroll 2
        for (int kk = 0; kk < 10; ++kk) {
            const int k = kg * 10 + kk;
            float4 w[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) w[q] = *(const float4 *)(wl + k * 16 + q * 4);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float d = 0.0f;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    d = __builtin_fmaf(g[r][q].x, w[q].x, d);
                    d = __builtin_fmaf(g[r][q].y, w[q].y, d);
                    d = __builtin_fmaf(g[r][q].z, w[q].z, d);
                    d = __builtin_fmaf(g[r][q].w, w[q].w, d);
                }
                pm[(pg * 4 + r) * kPmPitch + k] = Elem<T>::to_f32(Elem<T>::from_f32(d));
            }
        }
    }
    __syncthreads();
    // then col2im: per pixel of the [6, 12, 12] map the patch entries that land on it, added in T in the host's order
    // (filter rows and columns descending)
    for (int e = tid; e < 864; e += NT) {
        const int ci = e / 144, r = e - ci * 144, hy = r / 12, wy = r - hy * 12;
        T acc = Elem<T>::zero();
#pragma unroll
        for (int fi = 4; fi >= 0; --fi) {
            const int th = hy - fi;
            const bool hok = th >= 0 && th < 8;
            const int thc = min(max(th, 0), 7);
#pragma unroll
            for (int fj = 4; fj >= 0; --fj) {
                const int tw = wy - fj;
                const bool ok = hok && tw >= 0 && tw < 8;
                const float v = pm[(thc * 8 + min(max(tw, 0), 7)) * kPmPitch + ci * 25 + fi * 5 + fj];
                acc = Elem<T>::from_f32(Elem<T>::raw(acc) + (ok ? v : 0.0f));
            }
        }
        gp1s[e] = Elem<T>::to_f32(acc);
    }
    __syncthreads();
    // pooling + relu backward of conv1's output (6 channels x 12 x 12 windows), written as the [576, 6] matrix
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        const int e = tid + u * NT;
        if (e < 864) {
            const int ci = e / 144, r = e - ci * 144, ho = r / 12, wo = r - ho * 12;
            T cell[4];
            pool_relu_window_backward<T>(x1[u], gp1s[e], cell);
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int pos = (2 * ho + (k >> 1)) * 24 + 2 * wo + (k & 1);
                a.gm1[(b * 576 + pos) * 6 + ci] = cell[k];
            }
        }
    }
}

template <typename T>
int lenet5_backward_entry(const char *name, const void *logits, const void *target, float dy, const void *c1, const void *c2,
                          const void *d1, const void *d2, const void *w2, const void *wd1, const void *wd2, const void *wd3,
                          void *g_logits, void *g_d2, void *g_d1, void *gm2, void *gm1, int64_t bs) {
    AGH_API_ENTER();
    if (bs < 0) return fail(AGH_EINVAL, "%s: negative batch size", name);
    if (bs == 0) return AGH_OK;
    if (bs > ((int64_t)1 << 24)) return fail(AGH_ERANGE, "%s: batch too large", name);
    if (!logits || !target || !c1 || !c2 || !d1 || !d2 || !w2 || !wd1 || !wd2 || !wd3 || !g_logits || !g_d2 || !g_d1 || !gm2 || !gm1)
        return fail(AGH_ENULL, "%s: null buffer", name);
    if (((uintptr_t)wd1 & 15) != 0 || ((uintptr_t)wd2 & 7) != 0)
        return fail(AGH_EINVAL, "%s: wd1 must be 16-byte and wd2 8-byte aligned", name);
    LenetBackward<T> a;
    a.logits = (const T *)logits; a.target = (const uint8_t *)target;
    a.c1 = (const T *)c1; a.c2 = (const T *)c2; a.d1 = (const T *)d1; a.d2 = (const T *)d2;
    a.w2 = (const T *)w2; a.wd1 = (const T *)wd1; a.wd2 = (const T *)wd2; a.wd3 = (const T *)wd3;
    a.g_logits = (T *)g_logits; a.g_d2 = (T *)g_d2; a.g_d1 = (T *)g_d1; a.gm2 = (T *)gm2; a.gm1 = (T *)gm1;
    a.dy = dy / (float)bs;  // `dy /= batch_size` first, in f32, as the host does
    hipLaunchKernelGGL(lenet5_backward_kernel<T>, dim3((unsigned)bs), dim3(256), 0, stream(), a);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// The weight gradients of the three dense layers, the bias gradient and the loss of a LeNet5 training step in one
// launch: dwd3 = a2^T . g_logits [84, 10], dwd2 = a1^T . g_d2 [128, 84], dwd1 = f^T . g_d1 [256, 128] (each an f32 dot over
// the batch, rounded once to T, as the GEMM rounds it), db3 = the rows of g_logits added one at a time in T (the axis-0
// sum of the host), loss = the row losses added in row order (one workgroup, as cross_entropy_loss_kernel).  A
// workgroup owns a 16 x 16 tile of one product and stages the two 16-column strips it multiplies in LDS.
template <typename T>
struct LenetDenseGrads {
    const T *a2, *a1, *f;               // [bs, 84], [bs, 128], [bs, 256]
    const T *g_logits, *g_d2, *g_d1;    // [bs, 10], [bs, 84], [bs, 128]
    T *dwd3, *dwd2, *dwd1, *db3;        // [84, 10], [128, 84], [256, 128], [10]
    const T *logits;                    // [bs, 10]
    const uint8_t *target;              // [bs]
    float *loss;                        // one f32 (device or pinned host memory); may be null
    int bs;
};

template <typename T>
__global__ __launch_bounds__(256) void lenet5_dense_grads_kernel(LenetDenseGrads<T> q) {
    constexpr int RCH = 128;  // batch rows per pass
    __shared__ float as[RCH * 16], gs[RCH * 16];
    __shared__ float part[256];
    const int tid = threadIdx.x;
    int wg = blockIdx.x;
    // tiles: dwd1 16 x 8, dwd2 8 x 6, dwd3 6 x 1, then the bias gradient, then the loss
    const T *A, *G;
    T *D;
    int K, N, tk, tn;
    if (wg < 128) { A = q.f; G = q.g_d1; D = q.dwd1; K = 256; N = 128; tk = wg / 8; tn = wg % 8; }
    else if (wg < 176) { wg -= 128; A = q.a1; G = q.g_d2; D = q.dwd2; K = 128; N = 84; tk = wg / 6; tn = wg % 6; }
    else if (wg < 182) { wg -= 176; A = q.a2; G = q.g_logits; D = q.dwd3; K = 84; N = 10; tk = wg; tn = 0; }
    else if (wg == 182) {
        // the rows go through LDS, 200 at a time: read straight from memory the hundred dependent additions of a column
        // would each wait for their own load
        T acc = Elem<T>::zero();
        for (int r0 = 0; r0 < q.bs; r0 += 200) {
            const int cnt = min(200, q.bs - r0) * 10;
            __syncthreads();
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = q.g_logits[(size_t)r0 * 10 + min(tid + u * 256, cnt - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (tid + u * 256 < cnt) as[tid + u * 256] = Elem<T>::to_f32(v[u]);
            __syncthreads();
            if (tid < 10)
                for (int r = 0; r < cnt / 10; ++r) acc = Elem<T>::from_f32(Elem<T>::raw(acc) + as[r * 10 + tid]);
        }
        if (tid < 10) q.db3[tid] = acc;
        return;
    } else {
        if (!q.loss) return;
        float total = 0.0f;
        for (int base = 0; base < q.bs; base += 256) {
            const int r = base + tid;
            float l = 0.0f;
            if (r < q.bs) {
                const T *row = q.logits + (size_t)r * 10;
                float m = Elem<T>::to_f32(row[0]);
                for (int j = 0; j < 10; ++j) m = fmaxf(m, Elem<T>::to_f32(row[j]));
                float sum = 0.0f;
                for (int j = 0; j < 10; ++j) sum += expf(Elem<T>::to_f32(row[j]) - m);
                l = logf(sum) - (Elem<T>::to_f32(row[q.target[r]]) - m);
            }
            part[tid] = l;
            __syncthreads();
            if (tid == 0) {
                const int cnt = min(256, q.bs - base);
                for (int i = 0; i < cnt; ++i) total += part[i];
            }
            __syncthreads();
        }
        if (tid == 0) *q.loss = total;
        return;
    }
    const int k0 = tk * 16, n0 = tn * 16;
    const int i = tid >> 4, j = tid & 15;
    float acc = 0.0f;
    for (int r0 = 0; r0 < q.bs; r0 += RCH) {
        const int rows = min(RCH, q.bs - r0);
        __syncthreads();
        // all 16 elements of a thread are requested before the first is stored: one at a time the staging alone would
        // be a chain of eight memory latencies
        T av[RCH * 16 / 256], gv[RCH * 16 / 256];
#pragma unroll
        for (int u = 0; u < RCH * 16 / 256; ++u) {
            const int e = tid + u * 256, r = min(e >> 4, rows - 1), c = e & 15;
            av[u] = A[(size_t)(r0 + r) * K + min(k0 + c, K - 1)];
            gv[u] = G[(size_t)(r0 + r) * N + min(n0 + c, N - 1)];
        }
#pragma unroll
        for (int u = 0; u < RCH * 16 / 256; ++u) {
            const int e = tid + u * 256, r = e >> 4, c = e & 15;
            const bool rok = r < rows;
            as[e] = rok && k0 + c < K ? Elem<T>::to_f32(av[u]) : 0.0f;
            gs[e] = rok && n0 + c < N ? Elem<T>::to_f32(gv[u]) : 0.0f;
        }
        __syncthreads();
#pragma unroll 8
        for (int r = 0; r < rows; ++r) acc = __builtin_fmaf(as[r * 16 + i], gs[r * 16 + j], acc);
    }
    if (k0 + i < K && n0 + j < N) D[(size_t)(k0 + i) * N + n0 + j] = Elem<T>::from_f32(acc);
}

template <typename T>
int lenet5_dense_grads_entry(const char *name, const void *a2, const void *a1, const void *f, const void *g_logits,
                             const void *g_d2, const void *g_d1, void *dwd3, void *dwd2, void *dwd1, void *db3,
                             const void *logits, const void *target, void *loss, int64_t bs) {
    AGH_API_ENTER();
    if (bs < 0) return fail(AGH_EINVAL, "%s: negative batch size", name);
    if (bs == 0) return AGH_OK;
    if (bs > ((int64_t)1 << 24)) return fail(AGH_ERANGE, "%s: batch too large", name);
    if (!a2 || !a1 || !f || !g_logits || !g_d2 || !g_d1 || !dwd3 || !dwd2 || !dwd1 || !db3)
        return fail(AGH_ENULL, "%s: null buffer", name);
    if (loss && (!logits || !target)) return fail(AGH_ENULL, "%s: the loss needs the logits and the labels", name);
    LenetDenseGrads<T> q;
    q.a2 = (const T *)a2; q.a1 = (const T *)a1; q.f = (const T *)f;
    q.g_logits = (const T *)g_logits; q.g_d2 = (const T *)g_d2; q.g_d1 = (const T *)g_d1;
    q.dwd3 = (T *)dwd3; q.dwd2 = (T *)dwd2; q.dwd1 = (T *)dwd1; q.db3 = (T *)db3;
    q.logits = (const T *)logits; q.target = (const uint8_t *)target; q.loss = (float *)loss; q.bs = (int)bs;
    hipLaunchKernelGGL(lenet5_dense_grads_kernel<T>, dim3(184), dim3(256), 0, stream(), q);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// The weight gradients of the two convolutions of a LeNet5 training step without their patch matrices:
// dw2[oc][ci][fi][fj] = sum over images and output positions of gm2[(y, x)][oc] * p1[ci][y + fi][x + fj] (the product
// gm2^T . im2col(p1) of layer.rs:990-1003), dw1 likewise from gm1 and x.  One workgroup per image forms the image's f32
// partial sums from operands staged in LDS; a second launch adds the partials in image order and rounds once to T, as
// the split-K GEMM does.
constexpr int kLenetPartPitch = 2560;  // per image: 2400 entries of dw2, 150 of dw1
template <typename T>
__global__ __launch_bounds__(512) void lenet5_conv_grads_kernel(const T *__restrict__ x, const T *__restrict__ p1,
                                                                  const T *__restrict__ gm1, const T *__restrict__ gm2,
                                                                  float *__restrict__ part) {
    __shared__ __align__(16) float g2[64 * 16];   // [y*8 + x][oc]
    __shared__ __align__(8) float g1[576 * 6];    // [y*24 + x][oc]
    __shared__ float p1s[864], xs[784];
    __shared__ float q2[16 * 150], q1[8 * 150];   // partial sums: conv2 second half of the positions; conv1 by row group
    constexpr int NT = 512;
    const int tid = threadIdx.x;
    const size_t b = blockIdx.x;
    {
        // every element is requested before the first is stored
        T v2[2], vp[2], vx[2], v1[7];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            v2[u] = gm2[b * 1024 + tid + u * NT];
            vp[u] = p1[b * 864 + min(tid + u * NT, 863)];
            vx[u] = x[b * 784 + min(tid + u * NT, 783)];
        }
#pragma unroll
        for (int u = 0; u < 7; ++u) v1[u] = gm1[b * 3456 + min(tid + u * NT, 3455)];
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            const int i = tid + u * NT;
            g2[i] = Elem<T>::to_f32(v2[u]);
            if (i < 864) p1s[i] = Elem<T>::to_f32(vp[u]);
            if (i < 784) xs[i] = Elem<T>::to_f32(vx[u]);
        }
#pragma unroll
        for (int u = 0; u < 7; ++u)
            if (tid + u * NT < 3456) g1[tid + u * NT] = Elem<T>::to_f32(v1[u]);
    }
    __syncthreads();
    float *out = part + b * kLenetPartPitch;
    float acc2[16];
    if (tid < 300) {
        // conv2: one tap (ci, fi, fj) x 16 output channels over half of the 64 positions (ascending); the gradient row is
        // a broadcast read
        const int half = tid / 150, k = tid - half * 150;
        const int ci = k / 25, t = k - ci * 25, fi = t / 5, fj = t - fi * 5;
#pragma unroll
        for (int o = 0; o < 16; ++o) acc2[o] = 0.0f;
#pragma unroll
        for (int yy = 0; yy < 4; ++yy) {
            const int y = half * 4 + yy;
#pragma unroll
            for (int xx = 0; xx < 8; ++xx) {
                const float v = p1s[ci * 144 + (y + fi) * 12 + xx + fj];
                const float4 *g = (const float4 *)(g2 + (y * 8 + xx) * 16);
#pragma unroll
                for (int qd = 0; qd < 4; ++qd) {
                    const float4 gv = g[qd];
                    acc2[4 * qd + 0] = __builtin_fmaf(gv.x, v, acc2[4 * qd + 0]);
                    acc2[4 * qd + 1] = __builtin_fmaf(gv.y, v, acc2[4 * qd + 1]);
                    acc2[4 * qd + 2] = __builtin_fmaf(gv.z, v, acc2[4 * qd + 2]);
                    acc2[4 * qd + 3] = __builtin_fmaf(gv.w, v, acc2[4 * qd + 3]);
                }
            }
        }
        if (half == 1) {
#pragma unroll
            for (int o = 0; o < 16; ++o) q2[o * 150 + k] = acc2[o];
        }
    } else if (tid < 500) {
        // conv1: one tap x 6 output channels over three of the 24 output rows
        const int t = tid - 300, rg = t / 25, tap = t - rg * 25, fi = tap / 5, fj = tap - fi * 5;
        float acc[6];
#pragma unroll
        for (int o = 0; o < 6; ++o) acc[o] = 0.0f;
#pragma unroll
        for (int yy = 0; yy < 3; ++yy) {
            const int y = 3 * rg + yy;
#pragma unroll 12
            for (int xx = 0; xx < 24; ++xx) {
                const float v = xs[(y + fi) * 28 + xx + fj];
                const float2 *g = (const float2 *)(g1 + (y * 24 + xx) * 6);
                const float2 ga = g[0], gb = g[1], gc = g[2];
                acc[0] = __builtin_fmaf(ga.x, v, acc[0]);
                acc[1] = __builtin_fmaf(ga.y, v, acc[1]);
                acc[2] = __builtin_fmaf(gb.x, v, acc[2]);
                acc[3] = __builtin_fmaf(gb.y, v, acc[3]);
                acc[4] = __builtin_fmaf(gc.x, v, acc[4]);
                acc[5] = __builtin_fmaf(gc.y, v, acc[5]);
            }
        }
#pragma unroll
        for (int o = 0; o < 6; ++o) q1[rg * 150 + o * 25 + tap] = acc[o];
    }
    __syncthreads();
    if (tid < 150) {
#pragma unroll
        for (int o = 0; o < 16; ++o) out[o * 150 + tid] = acc2[o] + q2[o * 150 + tid];
    } else if (tid >= 300 && tid < 450) {
        const int k = tid - 300;
        float s = q1[k];
#pragma unroll
        for (int rg = 1; rg < 8; ++rg) s += q1[rg * 150 + k];
        out[2400 + k] = s;
    }
}

// 64 outputs per workgroup; wave j adds the images of the j-th quarter of the batch (its loads all in flight together),
// the four sums are then added in a fixed order
template <typename T>
__global__ __launch_bounds__(256) void lenet5_conv_grads_reduce_kernel(const float *__restrict__ part, T *__restrict__ dw1,
                                                                         T *__restrict__ dw2, int bs) {
    __shared__ float sums[4][64];
    const int lane = threadIdx.x & 63, j = threadIdx.x >> 6;
    const int k = min((int)blockIdx.x * 64 + lane, 2549);
    const int per = (bs + 3) / 4, b0 = j * per, b1 = min(bs, b0 + per);
    float s = 0.0f;
    int b = b0;
    for (; b + 8 <= b1; b += 8) {
        float v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = part[(size_t)(b + u) * kLenetPartPitch + k];
#pragma unroll
        for (int u = 0; u < 8; ++u) s += v[u];
    }
    for (; b < b1; ++b) s += part[(size_t)b * kLenetPartPitch + k];
    sums[j][lane] = s;
    __syncthreads();
    if (j == 0 && (int)blockIdx.x * 64 + lane < 2550) {
        const float tot = (sums[0][lane] + sums[1][lane]) + (sums[2][lane] + sums[3][lane]);
        if (k < 2400) dw2[k] = Elem<T>::from_f32(tot);
        else dw1[k - 2400] = Elem<T>::from_f32(tot);
    }
}

template <typename T>
int lenet5_conv_grads_entry(const char *name, const void *x, const void *p1, const void *gm1, const void *gm2, void *dw1,
                            void *dw2, int64_t bs) {
    AGH_API_ENTER();
    if (bs < 0) return fail(AGH_EINVAL, "%s: negative batch size", name);
    if (bs == 0) return AGH_OK;
    if (bs > ((int64_t)1 << 20)) return fail(AGH_ERANGE, "%s: batch too large", name);
    if (!x || !p1 || !gm1 || !gm2 || !dw1 || !dw2) return fail(AGH_ENULL, "%s: null buffer", name);
    void *ws = nullptr;
    if (int rc = workspace((size_t)bs * kLenetPartPitch * sizeof(float), &ws)) return rc;
    hipLaunchKernelGGL(lenet5_conv_grads_kernel<T>, dim3((unsigned)bs), dim3(512), 0, stream(), (const T *)x, (const T *)p1,
                       (const T *)gm1, (const T *)gm2, (float *)ws);
    AGH_LAUNCH_CHECK(name);
    hipLaunchKernelGGL(lenet5_conv_grads_reduce_kernel<T>, dim3(40), dim3(256), 0, stream(), (const float *)ws, (T *)dw1,
                       (T *)dw2, (int)bs);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T, bool POOL>
int launch_oct(int oct, dim3 grid, dim3 block, size_t smem, const T *x, const T *w, const T *bias, T *y,
               const ConvParams &p) {
    switch (oct) {
        case 1: hipLaunchKernelGGL((conv2_direct_kernel<T, 1, POOL>), grid, block, smem, stream(), x, w, bias, y, p); break;
        case 2: hipLaunchKernelGGL((conv2_direct_kernel<T, 2, POOL>), grid, block, smem, stream(), x, w, bias, y, p); break;
        case 4: hipLaunchKernelGGL((conv2_direct_kernel<T, 4, POOL>), grid, block, smem, stream(), x, w, bias, y, p); break;
        case 6: hipLaunchKernelGGL((conv2_direct_kernel<T, 6, POOL>), grid, block, smem, stream(), x, w, bias, y, p); break;
        default: hipLaunchKernelGGL((conv2_direct_kernel<T, 8, POOL>), grid, block, smem, stream(), x, w, bias, y, p); break;
    }
    return AGH_OK;
}

template <typename T>
int conv2_direct_entry(const char *name, const void *x, const void *w, const void *bias, void *y, int64_t bs,
                       int64_t ic, int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                       int64_t sh, int64_t sw, int64_t dh, int64_t dw, int act, int pool2x2) {
    AGH_API_ENTER();
    if (bs < 0 || ic < 1 || ih < 1 || iw < 1 || oc < 1 || fh < 1 || fw < 1 || ph < 0 || pw < 0 || sh < 1 || sw < 1 ||
        dh < 1 || dw < 1)
        return fail(AGH_EINVAL, "%s: invalid shape/options", name);
    if (act != AGH_ACT_NONE && act != AGH_ACT_RELU) return fail(AGH_EINVAL, "%s: unknown activation %d", name, act);
    if (ih + 2 * ph < dh * (fh - 1) + 1 || iw + 2 * pw < dw * (fw - 1) + 1)
        return fail(AGH_EINVAL, "%s: filter (with dilation) larger than the padded input", name);
    const int64_t lim = 1 << 20;
    if (bs > ((int64_t)1 << 30) || ic > lim || ih > lim || iw > lim || oc > lim || fh > lim || fw > lim || ph > lim ||
        pw > lim || sh > lim || sw > lim || dh > lim || dw > lim)
        return fail(AGH_ERANGE, "%s: dimension too large", name);
    const int64_t oh = (ih + 2 * ph - dh * (fh - 1) - 1) / sh + 1, ow = (iw + 2 * pw - dw * (fw - 1) - 1) / sw + 1;
    if (pool2x2 && (oh < 2 || ow < 2)) return fail(AGH_EINVAL, "%s: output smaller than the 2x2 pool window", name);
    if (bs == 0) return AGH_OK;
    if (!x || !w || !y) return fail(AGH_ENULL, "%s: null buffer", name);

    // enough channels: implicit GEMM on the matrix cores (returns 1 when the geometry is not its own)
    if (sh == 1 && sw == 1 && dh == 1 && dw == 1 && !pool2x2) {
        const int rc = conv2_mfma_try<T>(name, x, w, bias, y, bs, ic, ih, iw, oc, fh, fw, ph, pw, oh, ow, act);
        if (rc != 1) return rc;
    }

    // up to 16 output channels over enough taps on small images: matrix cores fed from the staged image
    if (sh == 1 && sw == 1 && dh == 1 && dw == 1 && oc <= 16) {
        const char *env = getenv("AGH_CONV_SMALL");  // 0 / 1 forces the choice (measurements)
        const int64_t taps = ic * fh * fw;
        const bool want = env ? atoi(env) != 0 : (oc >= 8 && taps >= 32);
        SmallMfmaParams q;
        q.bs = (int)bs; q.ic = (int)ic; q.ih = (int)ih; q.iw = (int)iw; q.oc = (int)oc; q.oh = (int)oh; q.ow = (int)ow;
        q.fh = (int)fh; q.fw = (int)fw; q.ph = (int)ph; q.pw = (int)pw;
        q.act = act; q.has_bias = bias != nullptr;
        q.ihp = (int)(ih + 2 * ph);
        q.pitch = (int)(iw + 2 * pw);
        q.ktot = (int)taps;
        q.ksteps = (int)((taps + 31) / 32 * 8);
        const int64_t yh = pool2x2 ? oh / 2 : oh, yw = pool2x2 ? ow / 2 : ow;
        q.nout = (int)(yh * yw);
        q.yw = (int)yw;
        q.mtiles = (int)(pool2x2 ? (yh * yw + 3) / 4 : (yh * yw + 15) / 16);
        const int tg = q.mtiles >= 8 ? 4 : 2;
        q.units_per_img = (q.mtiles + tg - 1) / tg;
        const int64_t kpad = (int64_t)q.ksteps * 4;
        const int64_t fixed_bytes = kpad * 17 * 4, img_bytes = ic * (int64_t)q.ihp * q.pitch * 4;
        constexpr int64_t kLds = 64 * 1024;
        if (want && taps <= 2048 && fixed_bytes + img_bytes <= kLds && yh * yw <= ((int64_t)1 << 20)) {
            const int64_t cus = compute_units() > 0 ? compute_units() : 256;
            // a workgroup's four waves want a unit each; more images per workgroup only while the grid still
            // covers the chip twice
            int64_t imgs = std::max<int64_t>(1, 4 / q.units_per_img);
            while (fixed_bytes + (imgs + 1) * img_bytes <= kLds && (imgs + 1) * q.units_per_img <= 8 &&
                   (bs + imgs) / (imgs + 1) >= 2 * cus)
                ++imgs;
            while (imgs > 1 && fixed_bytes + imgs * img_bytes > kLds) --imgs;
            if (imgs > bs) imgs = bs;
            q.imgs = (int)imgs;
            q.div_pitch = FastDiv((uint32_t)q.pitch);
            q.div_ihp = FastDiv((uint32_t)q.ihp);
            q.div_yw = FastDiv((uint32_t)yw);
            q.div_fw = FastDiv((uint32_t)fw);
            q.div_fhfw = FastDiv((uint32_t)(fh * fw));
            q.div_upi = FastDiv((uint32_t)q.units_per_img);
            const int64_t blocks = (bs + imgs - 1) / imgs;
            if (blocks > 0x7FFFFFFF) return fail(AGH_ERANGE, "%s: too many workgroups", name);
            const size_t smem = (size_t)(fixed_bytes + imgs * img_bytes);
            const dim3 grid((unsigned)blocks), block(256);
            const T *xp = (const T *)x, *wp = (const T *)w, *bp = (const T *)bias;
            T *yp = (T *)y;
#define AGH_SM(POOLV, TGV) \
    hipLaunchKernelGGL((conv2_small_mfma_kernel<T, POOLV, TGV>), grid, block, smem, stream(), xp, wp, bp, yp, q)
            if (pool2x2) { if (tg == 4) AGH_SM(true, 4); else AGH_SM(true, 2); }
            else { if (tg == 4) AGH_SM(false, 4); else AGH_SM(false, 2); }
#undef AGH_SM
            AGH_LAUNCH_CHECK(name);
            return AGH_OK;
        }
    }

    // stride 1, dilation 1, filter width 3 or 5: row-tiled kernel
    if (sh == 1 && sw == 1 && dh == 1 && dw == 1 && (fw == 3 || fw == 5)) {
        RowTileParams q;
        q.bs = bs; q.ic = ic; q.ih = ih; q.iw = iw; q.oc = oc; q.oh = oh; q.ow = ow; q.fh = fh; q.ph = ph; q.pw = pw;
        q.act = act; q.has_bias = bias != nullptr;
        // two output channels per work item unless that leaves fewer than ~4 waves per CU in flight
        const int64_t cus0 = compute_units() > 0 ? compute_units() : 256;
        const int64_t rows0 = pool2x2 ? oh / 2 : oh, wbs0 = (ow + 7) / 8;
        const int oct = (oc <= 1 || bs * rows0 * wbs0 * ((oc + 1) / 2) < cus0 * 4 * 64) ? 1 : 2;
        q.ngroups = (oc + oct - 1) / oct;
        q.ocpad = q.ngroups * oct;
        q.nwb = (ow + 7) / 8;
        q.ihp = ih + 2 * ph;
        int64_t pitch = iw + 2 * pw;
        if (pitch < q.nwb * 8 + fw - 1) pitch = q.nwb * 8 + fw - 1;
        // whole 16-byte reads of WT + FW - 1 floats starting at a multiple of 8
        const int64_t xw4 = ((8 + fw - 1 + 3) / 4) * 4;
        if (pitch < (q.nwb - 1) * 8 + xw4) pitch = (q.nwb - 1) * 8 + xw4;
        q.pitch = (int)((pitch + 3) & ~(int64_t)3);
        q.yh = pool2x2 ? oh / 2 : oh;
        q.yw = pool2x2 ? ow / 2 : ow;
        q.nrows = q.yh;
        const int64_t items = (int64_t)q.nrows * q.nwb * q.ngroups;
        const int64_t taps = ic * fh * fw;
        const int64_t w_bytes = ((taps * q.ocpad + 3) & ~(int64_t)3) * 4, img_bytes = (int64_t)ic * q.ihp * q.pitch * 4;
        constexpr int64_t kLds = 64 * 1024;
        if (w_bytes + img_bytes <= kLds && items <= ((int64_t)1 << 24)) {
            const int64_t cus = compute_units() > 0 ? compute_units() : 256;
            int64_t imgs = items >= 256 ? 1 : 256 / items;
            while (imgs > 1 && w_bytes + imgs * img_bytes > kLds) --imgs;
            while (imgs > 1 && (bs + imgs - 1) / imgs < cus) --imgs;
            if (imgs > bs) imgs = bs;
            q.imgs = (int)imgs;
            q.items_per_img = (int)items;
            q.div_items = FastDiv((uint32_t)items);
            q.div_rowsxwb = FastDiv((uint32_t)(q.nrows * q.nwb));
            q.div_nwb = FastDiv((uint32_t)q.nwb);
            q.div_ocpad = FastDiv((uint32_t)q.ocpad);
            q.div_pitch = FastDiv((uint32_t)q.pitch);
            q.div_ihp = FastDiv((uint32_t)q.ihp);
            const int64_t work = imgs * items;
            const int threads = work >= 256 ? 256 : (int)((work + 63) / 64 * 64);
            const int64_t blocks = (bs + imgs - 1) / imgs;
            if (blocks > 0x7FFFFFFF) return fail(AGH_ERANGE, "%s: too many workgroups", name);
            const size_t smem = (size_t)(w_bytes + imgs * img_bytes);
            const dim3 grid((unsigned)blocks), block(threads);
            const T *xp = (const T *)x, *wp = (const T *)w, *bp = (const T *)bias;
            T *yp = (T *)y;
#define AGH_RT(FWV, OCTV, POOLV) \
    do { \
        if (fh == FWV) hipLaunchKernelGGL((conv2_rowtile_kernel<T, FWV, OCTV, POOLV, FWV>), grid, block, smem, stream(), xp, wp, bp, yp, q); \
        else hipLaunchKernelGGL((conv2_rowtile_kernel<T, FWV, OCTV, POOLV, 0>), grid, block, smem, stream(), xp, wp, bp, yp, q); \
    } while (0)
            if (fw == 3) {
                if (oct == 1) { if (pool2x2) AGH_RT(3, 1, true); else AGH_RT(3, 1, false); }
                else { if (pool2x2) AGH_RT(3, 2, true); else AGH_RT(3, 2, false); }
            } else {
                if (oct == 1) { if (pool2x2) AGH_RT(5, 1, true); else AGH_RT(5, 1, false); }
                else { if (pool2x2) AGH_RT(5, 2, true); else AGH_RT(5, 2, false); }
            }
#undef AGH_RT
            AGH_LAUNCH_CHECK(name);
            return AGH_OK;
        }
    }

    ConvParams p;
    p.bs = bs; p.ic = ic; p.ih = ih; p.iw = iw; p.oc = oc; p.oh = oh; p.ow = ow;
    p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
    p.act = act; p.has_bias = bias != nullptr;
    p.yh = pool2x2 ? oh / 2 : oh;
    p.yw = pool2x2 ? ow / 2 : ow;
    // output channels per work item: the whole bank when it is small, else groups of 8
    int oct = 8;
    for (int c : {1, 2, 4, 6, 8})
        if (oc <= c) { oct = c; break; }
    p.ngroups = (oc + oct - 1) / oct;
    p.ocpad = p.ngroups * oct;
    const int64_t pix = (int64_t)p.yh * p.yw;
    const int64_t items = pix * p.ngroups;
    const int64_t taps = ic * fh * fw;
    const int64_t img_bytes = ic * ih * iw * 4, w_bytes = taps * p.ocpad * 4;
    constexpr int64_t kLds = 64 * 1024;
    if (w_bytes + img_bytes > kLds || items > ((int64_t)1 << 24))
        return fail(AGH_ERANGE, "%s: image + filter bank (%lld bytes) do not fit in LDS; use im2col + gemm", name,
                    (long long)(w_bytes + img_bytes));
    // images per workgroup: aim at ~256 work items, stay inside LDS, keep >= 2 workgroups per CU
    int64_t imgs = items >= 256 ? 1 : 256 / items;
    while (imgs > 1 && w_bytes + imgs * img_bytes > kLds) --imgs;
    const int64_t cus = compute_units() > 0 ? compute_units() : 256;
    while (imgs > 1 && (bs + imgs - 1) / imgs < 2 * cus) --imgs;
    if (imgs > bs) imgs = bs;
    p.imgs = (int)imgs;
    p.items_per_img = (int)items;
    p.div_items = FastDiv((uint32_t)items);
    p.div_pix = FastDiv((uint32_t)pix);
    p.div_yw = FastDiv((uint32_t)p.yw);
    int64_t work = imgs * items;
    int threads = work >= 256 ? 256 : (int)((work + 63) / 64 * 64);
    const int64_t blocks = (bs + imgs - 1) / imgs;
    if (blocks > 0x7FFFFFFF) return fail(AGH_ERANGE, "%s: too many workgroups", name);
    const size_t smem = (size_t)(w_bytes + imgs * img_bytes);
    if (pool2x2)
        launch_oct<T, true>(oct, dim3((unsigned)blocks), dim3(threads), smem, (const T *)x, (const T *)w, (const T *)bias,
                            (T *)y, p);
    else
        launch_oct<T, false>(oct, dim3((unsigned)blocks), dim3(threads), smem, (const T *)x, (const T *)w,
                             (const T *)bias, (T *)y, p);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

}  // namespace

template <typename T>
int lenet5_forward_entry(const char *name, const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                         const void *wd3, const void *b3, void *logits, int64_t bs, void *const *saves) {
    AGH_API_ENTER();
    if (bs < 0 || bs > ((int64_t)1 << 30)) return fail(AGH_EINVAL, "%s: bad batch size", name);
    if (bs == 0) return AGH_OK;
    if (!x || !w1 || !w2 || !wd1 || !wd2 || !wd3 || !b3 || !logits) return fail(AGH_ENULL, "%s: null buffer", name);
    LenetSaves<T> sv = {};
    const int w23_aligned = (((uintptr_t)wd2 | (uintptr_t)wd3) & 15) == 0;
    if (saves) {
        for (int i = 0; i < 8; ++i)
            if (!saves[i]) return fail(AGH_ENULL, "%s: null buffer for a saved activation", name);
        sv = {(T *)saves[0], (T *)saves[1], (T *)saves[2], (T *)saves[3], (T *)saves[4], (T *)saves[5], (T *)saves[6], (T *)saves[7]};
    }
    // one image per workgroup while that still fits the chip in one round
    const bool single = bs <= 256;  // measured: 7.0 against 11.2 us up to 256 images, 13.1 against 11.3 us at 384
#define AGH_LENET(SAVEV, IMGSV) \
    hipLaunchKernelGGL((lenet5_forward_kernel<T, SAVEV, IMGSV>), dim3((unsigned)((bs + IMGSV - 1) / IMGSV)), dim3(512), 0, stream(), \
                       (const T *)x, (const T *)w1, (const T *)w2, (const T *)wd1, (const T *)wd2, (const T *)wd3, (const T *)b3, \
                       (T *)logits, (int)bs, sv, w23_aligned)
    if (saves) {
        if (single) AGH_LENET(true, 1); else AGH_LENET(true, 4);
    } else {
        if (single) AGH_LENET(false, 1); else AGH_LENET(false, 4);
    }
#undef AGH_LENET
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

extern "C" {

int agh_conv2_direct_f32(const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic, int64_t ih,
                         int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t sh,
                         int64_t sw, int64_t dh, int64_t dw, int act, int pool2x2) {
    return conv2_direct_entry<float>("agh_conv2_direct_f32", x, w, bias, y, bs, ic, ih, iw, oc, fh, fw, ph, pw, sh, sw,
                                     dh, dw, act, pool2x2);
}
int agh_conv2_direct_bf16(const void *x, const void *w, const void *bias, void *y, int64_t bs, int64_t ic, int64_t ih,
                          int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t sh,
                          int64_t sw, int64_t dh, int64_t dw, int act, int pool2x2) {
    return conv2_direct_entry<uint16_t>("agh_conv2_direct_bf16", x, w, bias, y, bs, ic, ih, iw, oc, fh, fw, ph, pw, sh,
                                        sw, dh, dw, act, pool2x2);
}

int agh_lenet5_forward_f32(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                           const void *wd3, const void *b3, void *logits, int64_t bs) {
    return lenet5_forward_entry<float>("agh_lenet5_forward_f32", x, w1, w2, wd1, wd2, wd3, b3, logits, bs, nullptr);
}
int agh_lenet5_forward_bf16(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                            const void *wd3, const void *b3, void *logits, int64_t bs) {
    return lenet5_forward_entry<uint16_t>("agh_lenet5_forward_bf16", x, w1, w2, wd1, wd2, wd3, b3, logits, bs, nullptr);
}
int agh_lenet5_forward_train_f32(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                                 const void *wd3, const void *b3, void *c1, void *p1, void *c2, void *p2, void *d1,
                                 void *a1, void *d2, void *a2, void *logits, int64_t bs) {
    void *saves[8] = {c1, p1, c2, p2, d1, a1, d2, a2};
    return lenet5_forward_entry<float>("agh_lenet5_forward_train_f32", x, w1, w2, wd1, wd2, wd3, b3, logits, bs, saves);
}
int agh_lenet5_forward_train_bf16(const void *x, const void *w1, const void *w2, const void *wd1, const void *wd2,
                                  const void *wd3, const void *b3, void *c1, void *p1, void *c2, void *p2, void *d1,
                                  void *a1, void *d2, void *a2, void *logits, int64_t bs) {
    void *saves[8] = {c1, p1, c2, p2, d1, a1, d2, a2};
    return lenet5_forward_entry<uint16_t>("agh_lenet5_forward_train_bf16", x, w1, w2, wd1, wd2, wd3, b3, logits, bs, saves);
}

#define AGH_LENET_BWD_ARGS                                                                                             \
    const void *logits, const void *target, float dy, const void *c1, const void *c2, const void *d1, const void *d2, \
        const void *w2, const void *wd1, const void *wd2, const void *wd3, void *g_logits, void *g_d2, void *g_d1,    \
        void *gm2, void *gm1, int64_t bs
int agh_lenet5_backward_f32(AGH_LENET_BWD_ARGS) {
    return lenet5_backward_entry<float>("agh_lenet5_backward_f32", logits, target, dy, c1, c2, d1, d2, w2, wd1, wd2, wd3,
                                        g_logits, g_d2, g_d1, gm2, gm1, bs);
}
int agh_lenet5_backward_bf16(AGH_LENET_BWD_ARGS) {
    return lenet5_backward_entry<uint16_t>("agh_lenet5_backward_bf16", logits, target, dy, c1, c2, d1, d2, w2, wd1, wd2, wd3,
                                           g_logits, g_d2, g_d1, gm2, gm1, bs);
}

#define AGH_LENET_DG_ARGS                                                                                            \
    const void *a2, const void *a1, const void *f, const void *g_logits, const void *g_d2, const void *g_d1, void *dwd3, \
        void *dwd2, void *dwd1, void *db3, const void *logits, const void *target, void *loss, int64_t bs
int agh_lenet5_dense_weight_grads_f32(AGH_LENET_DG_ARGS) {
    return lenet5_dense_grads_entry<float>("agh_lenet5_dense_weight_grads_f32", a2, a1, f, g_logits, g_d2, g_d1, dwd3, dwd2,
                                           dwd1, db3, logits, target, loss, bs);
}
int agh_lenet5_dense_weight_grads_bf16(AGH_LENET_DG_ARGS) {
    return lenet5_dense_grads_entry<uint16_t>("agh_lenet5_dense_weight_grads_bf16", a2, a1, f, g_logits, g_d2, g_d1, dwd3,
                                              dwd2, dwd1, db3, logits, target, loss, bs);
}

int agh_lenet5_conv_weight_grads_f32(const void *x, const void *p1, const void *gm1, const void *gm2, void *dw1, void *dw2,
                                     int64_t bs) {
    return lenet5_conv_grads_entry<float>("agh_lenet5_conv_weight_grads_f32", x, p1, gm1, gm2, dw1, dw2, bs);
}
int agh_lenet5_conv_weight_grads_bf16(const void *x, const void *p1, const void *gm1, const void *gm2, void *dw1, void *dw2,
                                      int64_t bs) {
    return lenet5_conv_grads_entry<uint16_t>("agh_lenet5_conv_weight_grads_bf16", x, p1, gm1, gm2, dw1, dw2, bs);
}

}  // extern "C"

// Memory-bound kernels of the hot path: im2col / col2im for Conv2, MaxPool2 forward and
// backward, ReLU, byte fill.  All of them are bounded by HBM traffic, so the work is laid
// out for coalesced 16-byte stores and single-pass reads; index arithmetic is kept off
// the critical path with launch-constant multiply-high division.
#include <type_traits>

#include "agh_internal.h"

using namespace agh;

namespace {

constexpr int kThreads = 256;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

inline int64_t conv_out(int64_t i, int64_t f, int64_t p, int64_t s, int64_t d) {
    return (i + 2 * p - d * (f - 1) - 1) / s + 1;
}
inline int64_t col2im_out(int64_t i, int64_t f, int64_t p, int64_t s, int64_t d) {
    return (i - 1) * s + d * (f - 1) + 1 - 2 * p;
}

// ------------------------------------------------------------------- fill ----
__global__ __launch_bounds__(kThreads) void fill_bytes_kernel(uint8_t *dst, uint32_t pattern, size_t bytes) {
    // head/tail bytes individually, the aligned middle as 16-byte stores
    size_t addr = (size_t)dst;
    size_t head = (16 - (addr & 15)) & 15;
    if (head > bytes) head = bytes;
    size_t body = (bytes - head) / 16;
    size_t tail = bytes - head - body * 16;
    size_t tid = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    size_t stride = (size_t)gridDim.x * blockDim.x;
    const u32x4 v = {pattern, pattern, pattern, pattern};
    uint8_t *mid = dst + head;
    for (size_t i = tid; i < body; i += stride) __builtin_nontemporal_store(v, (u32x4 *)mid + i);
    if (tid < head) dst[tid] = (uint8_t)pattern;
    if (tid < tail) dst[head + body * 16 + tid] = (uint8_t)pattern;
}

// ----------------------------------------------------------------- im2col ----
//
// One workgroup produces the patch rows of one (image b, output row ho) for a chunk of
// CC channels: it stages the fh input rows those patches touch, for every channel of the
// chunk, in LDS (zero-filled where the window hangs over the border), then streams the
// patch matrix out.  For a fixed ho the rows (b, ho, wo = 0..ow-1) are adjacent in y, so
// when the chunk is all channels the workgroup writes ONE contiguous block of
// ow * c*fh*fw elements with 16-byte stores; the input is read once per (ho, fi) pair and
// re-reads across neighbouring ho hit L2.
struct Im2colParams {
    int bs, c, ih, iw, oh, ow;
    int fh, fw, ph, pw, sh, sw, dh, dw;
    int cc;        // channels per workgroup
    int nchunk;    // ceil(c / cc)
    int span;      // input columns a row of patches touches: (ow-1)*sw + (fw-1)*dw + 1
    int span_pad;  // LDS row pitch (elements)
    int nslot;     // 16-byte pieces per image row (vector staging)
    int npad;      // padding cells per staged row: pw on the left, the rest right of the image
    int nblocks;   // workgroups with work
    int per_xcd;   // ceil(nblocks / 8)
    int ktot;      // c*fh*fw
    FastDiv div_l, div_ff, div_fw, div_nchunk, div_oh, div_span, div_fh, div_nslot, div_npad;
};

template <typename T, int VEC, bool VSTAGE>
__global__ __launch_bounds__(kThreads) void im2col_lds_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                               Im2colParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    // layout: int tab[L rounded to 4] | T tile[cc*fh*span_pad]
    // Workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its own.  Neighbouring
    // output rows of an image stage the same input rows, so every XCD is given a contiguous run of
    // (image, output row) pairs: the re-reads then hit its L2 instead of going out to memory again.
    const uint32_t bid = (blockIdx.x & 7) * p.per_xcd + (blockIdx.x >> 3);
    if (bid >= (uint32_t)p.nblocks) return;
    uint32_t t0, chunk, b, ho;
    p.div_nchunk.divmod(bid, t0, chunk);
    p.div_oh.divmod(t0, b, ho);
    const int c0 = chunk * p.cc;
    const int ff = p.fh * p.fw;
    const int L = p.cc * ff;  // columns this workgroup writes per patch row (cc divides c)
    int *tab = (int *)smem_raw;
    T *tile = (T *)(smem_raw + (size_t)((L + 3) & ~3) * sizeof(int));

    // Column j = (cl, fi, fj) -> LDS offset of its element for wo = 0.  With vector stores, lane l of a
    // wave later reads the VEC offsets of its 16-byte group jv with one table read and fetches the VEC
    // elements one per LDS instruction; were every lane to fetch element u of its group in instruction u,
    // the lanes of a half-wave would hit every fourth LDS bank only.  So the group's entries are kept
    // rotated by (l / 8) % 4 dwords: in instruction u the four 8-lane blocks of a half-wave fetch
    // elements u, u+1, u+2, u+3 (dwords) of their groups, which covers all 32 banks when the row pitch
    // makes consecutive columns fall in consecutive banks.  The rotation is undone in registers.
    for (int j = threadIdx.x; j < L; j += kThreads) {
        uint32_t cl, r, fi, fj;
        p.div_ff.divmod(j, cl, r);
        p.div_fw.divmod(r, fi, fj);
        int slot = j;
        if constexpr (VEC > 1) {
            const int jv = j / VEC, u = j % VEC;
            const int rot = ((jv >> 3) & 3) * (VEC / 4);
            slot = jv * VEC + ((u - rot + VEC) % VEC);
        }
        tab[slot] = (cl * p.fh + fi) * p.span_pad + fj * p.dw;
    }
    // Stage rows.  The staged space is flattened over the workgroup and walked in batches of SU items
    // per thread: all SU global loads are issued before the first LDS store, so a thread pays the
    // memory latency once per batch and not once per item.
    const uint32_t nrows = (uint32_t)(p.cc * p.fh);
    if constexpr (VSTAGE) {
        // Items are 16-byte pieces of the image rows (iw is a whole number of them); the padding cells
        // left and right of the image are zeroed separately.
        constexpr int SV = 16 / (int)sizeof(T), SU = 4;
        const uint32_t nitem = nrows * (uint32_t)p.nslot;
        for (uint32_t s0 = threadIdx.x; s0 < nitem; s0 += kThreads * SU) {
            union { u32x4 q; T e[SV]; } v[SU];
            uint32_t dsto[SU];
#pragma unroll
            for (int u = 0; u < SU; ++u) {
                const uint32_t s = s0 + u * kThreads;
                uint32_t r, sl, cl, fi;
                p.div_nslot.divmod(s, r, sl);
                p.div_fh.divmod(r, cl, fi);
                const int hidx = -p.ph + (int)fi * p.dh + p.sh * (int)ho;
                const bool ok = s < nitem && hidx >= 0 && hidx < p.ih;
                v[u].q = u32x4{0, 0, 0, 0};
                if (ok) v[u].q = *(const u32x4 *)(x + (((size_t)b * p.c + c0 + cl) * p.ih + hidx) * (size_t)p.iw + sl * SV);
                dsto[u] = s < nitem ? r * p.span_pad + p.pw + sl * SV : 0xFFFFFFFFu;
            }
#pragma unroll
            for (int u = 0; u < SU; ++u)
                if (dsto[u] != 0xFFFFFFFFu) {
#pragma unroll
                    for (int k = 0; k < SV; ++k) tile[dsto[u] + k] = v[u].e[k];
                }
        }
        const uint32_t npad = nrows * (uint32_t)p.npad;
        for (uint32_t s = threadIdx.x; s < npad; s += kThreads) {
            uint32_t r, k;
            p.div_npad.divmod(s, r, k);
            tile[r * p.span_pad + ((int)k < p.pw ? k : p.iw + k)] = 0;
        }
    } else {
        const uint32_t nstage = nrows * (uint32_t)p.span;
        constexpr int SU = 8;
        for (uint32_t s0 = threadIdx.x; s0 < nstage; s0 += kThreads * SU) {
            T v[SU];
            uint32_t dsto[SU];
#pragma unroll
            for (int u = 0; u < SU; ++u) {
                const uint32_t s = s0 + u * kThreads;
                uint32_t r, j, cl, fi;
                p.div_span.divmod(s, r, j);
                p.div_fh.divmod(r, cl, fi);
                const int hidx = -p.ph + (int)fi * p.dh + p.sh * (int)ho;
                const int widx = (int)j - p.pw;
                const bool ok = s < nstage && hidx >= 0 && hidx < p.ih && widx >= 0 && widx < p.iw;
                v[u] = 0;
                if (ok) v[u] = x[(((size_t)b * p.c + c0 + cl) * p.ih + hidx) * (size_t)p.iw + widx];
                dsto[u] = s < nstage ? r * p.span_pad + j : 0xFFFFFFFFu;
            }
#pragma unroll
            for (int u = 0; u < SU; ++u)
                if (dsto[u] != 0xFFFFFFFFu) tile[dsto[u]] = v[u];
        }
    }
    __syncthreads();

    const size_t row0 = ((size_t)b * p.oh + ho) * p.ow;  // first patch row of this workgroup
    T *ybase = y + row0 * p.ktot + (size_t)c0 * ff;
    if constexpr (VEC > 1) {
        // Every patch-row segment starts 16-byte aligned and holds a multiple of VEC elements.  A wave
        // takes WO_U patch rows at a time (wave-uniform, so the row base lives in scalar registers) and
        // its lanes walk the 16-byte groups of the segment: one table read serves WO_U stores, and the
        // per-lane arithmetic is the add of the patch's column base to each table offset plus the
        // un-rotation of the four dwords.
        constexpr int WO_U = 2, nwave = kThreads >> 6;
        const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63;
        const bool rot1 = (lane & 8) != 0, rot2 = (lane & 16) != 0;
        const int LV = L / VEC;
        for (int wg = wave * WO_U; wg < p.ow; wg += nwave * WO_U) {
            for (int jv = lane; jv < LV; jv += 64) {
                int4 offs[VEC / 4];
#pragma unroll
                for (int u = 0; u < VEC / 4; ++u) offs[u] = *(const int4 *)(tab + jv * VEC + 4 * u);
                uint32_t d[WO_U][4];
#pragma unroll
                for (int w = 0; w < WO_U; ++w) {
                    const int base = min(wg + w, p.ow - 1) * p.sw;  // clamped: a duplicate row, not stored
                    T t[VEC];
#pragma unroll
                    for (int u = 0; u < VEC / 4; ++u) {
                        t[4 * u + 0] = tile[offs[u].x + base];
                        t[4 * u + 1] = tile[offs[u].y + base];
                        t[4 * u + 2] = tile[offs[u].z + base];
                        t[4 * u + 3] = tile[offs[u].w + base];
                    }
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        if constexpr (sizeof(T) == 4) d[w][k] = (uint32_t)t[k];
                        else d[w][k] = (uint32_t)t[2 * k] | ((uint32_t)t[2 * k + 1] << 16);
                    }
                }
#pragma unroll
                for (int w = 0; w < WO_U; ++w) {
                    uint32_t r[4];
#pragma unroll
                    for (int m = 0; m < 4; ++m) r[m] = rot1 ? d[w][(m + 3) & 3] : d[w][m];
                    u32x4 o;
                    o.x = rot2 ? r[2] : r[0];
                    o.y = rot2 ? r[3] : r[1];
                    o.z = rot2 ? r[0] : r[2];
                    o.w = rot2 ? r[1] : r[3];
                    if (wg + w < p.ow)
                        __builtin_nontemporal_store(o, (u32x4 *)(ybase + (size_t)(wg + w) * p.ktot + jv * VEC));
                }
            }
        }
    } else {
        const uint32_t total = (uint32_t)p.ow * L;
        for (uint32_t e = threadIdx.x; e < total; e += kThreads) {
            uint32_t wo, j;
            p.div_l.divmod(e, wo, j);
            ybase[(size_t)wo * p.ktot + j] = tile[tab[j] + wo * p.sw];
        }
    }
}

// Fallback for geometries whose staged rows do not fit in LDS: one thread per output
// element, consecutive threads along a patch row.
template <typename T>
__global__ __launch_bounds__(kThreads) void im2col_direct_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                  Im2colParams p, size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    size_t row = e / p.ktot;
    int j = (int)(e - row * p.ktot);
    int wo = (int)(row % p.ow);
    size_t t = row / p.ow;
    int ho = (int)(t % p.oh);
    size_t b = t / p.oh;
    int ff = p.fh * p.fw;
    int ci = j / ff, r = j - ci * ff;
    int fi = r / p.fw, fj = r - fi * p.fw;
    int hidx = -p.ph + fi * p.dh + p.sh * ho;
    int widx = -p.pw + fj * p.dw + p.sw * wo;
    T v = 0;
    if (hidx >= 0 && hidx < p.ih && widx >= 0 && widx < p.iw)
        v = x[((b * p.c + ci) * p.ih + hidx) * (size_t)p.iw + widx];
    y[e] = v;
}

template <typename T>
int im2col_launch(const char *name, const void *x, void *y, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                  int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t sh, int64_t sw, int64_t dh, int64_t dw) {
    AGH_API_ENTER();
    if (bs < 0 || c < 0 || ih < 0 || iw < 0 || fh < 1 || fw < 1 || ph < 0 || pw < 0 || sh < 1 || sw < 1 || dh < 1 || dw < 1)
        return fail(AGH_EINVAL, "%s: invalid shape/options", name);
    if (ih + 2 * ph < dh * (fh - 1) + 1 || iw + 2 * pw < dw * (fw - 1) + 1)
        return fail(AGH_EINVAL, "%s: filter (with dilation) larger than the padded input", name);
    const int64_t oh = conv_out(ih, fh, ph, sh, dh), ow = conv_out(iw, fw, pw, sw, dw);
    const int64_t lim = (int64_t)1 << 30;
    if (bs > lim || c > lim || ih > lim || iw > lim || fh > lim || fw > lim || ph > lim || pw > lim || sh > lim ||
        sw > lim || dh > lim || dw > lim || c * fh * fw > lim || bs * oh > lim)
        return fail(AGH_ERANGE, "%s: dimension too large", name);
    const size_t total = (size_t)bs * oh * ow * c * fh * fw;
    if (total == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);

    Im2colParams p;
    p.bs = bs; p.c = c; p.ih = ih; p.iw = iw; p.oh = oh; p.ow = ow;
    p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
    p.ktot = c * fh * fw;
    const int64_t span = (ow - 1) * sw + (fw - 1) * dw + 1;
    const int ff = fh * fw;
    constexpr int VEC = 16 / sizeof(T);
    // Vector staging copies whole 16-byte pieces of the image rows: needs rows that are a whole number
    // of pieces and start on 16 bytes.
    const bool vstage = iw % VEC == 0 && ((uintptr_t)x & 15) == 0;
    // LDS row pitch: at least the columns a patch row touches (and the whole padded image row for
    // vector staging), and congruent to fw modulo the 32 LDS banks (128 bytes), so that column
    // (cl, fi, fj) of a patch sits fw*(cl*fh+fi)+fj banks after column 0: consecutive patch columns
    // fall in consecutive banks, which the rotated table of the kernel relies on.
    constexpr int64_t kBankElems = 128 / sizeof(T);
    int64_t span_pad = std::max<int64_t>(span, vstage ? pw + iw : 0);
    span_pad += ((fw - span_pad) % kBankElems + kBankElems) % kBankElems;
    constexpr int64_t kLdsBudget = 48 * 1024;
    auto lds_bytes = [&](int64_t cc) {
        return (int64_t)((cc * ff + 3) & ~3) * 4 + cc * fh * span_pad * (int64_t)sizeof(T);
    };
    // Channels per workgroup: the largest divisor of c whose staged rows fit the LDS budget.
    // Vector stores need every patch-row segment to start 16-byte aligned and to hold a
    // multiple of VEC elements, i.e. ktot and cc*ff multiples of VEC.
    auto pick = [&](bool vec) -> int64_t {
        for (int64_t d = c; d >= 1; --d) {
            if (c % d != 0) continue;
            if (vec && (d * ff) % VEC != 0) continue;
            if (lds_bytes(d) <= kLdsBudget && ow * d * ff < ((int64_t)1 << 31)) return d;
        }
        return 0;
    };
    bool vec = (p.ktot % VEC == 0);
    int64_t cc = vec ? pick(true) : 0;
    if (cc == 0) { vec = false; cc = pick(false); }
    if (cc == 0) {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
        hipLaunchKernelGGL(im2col_direct_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(),
                           (const T *)x, (T *)y, p, total);
        AGH_LAUNCH_CHECK(name);
        return AGH_OK;
    }
    p.cc = cc;
    p.nchunk = c / cc;
    p.span = span;
    p.span_pad = span_pad;
    p.nslot = iw / VEC;
    p.npad = pw + std::max<int64_t>(0, span - pw - iw);
    p.div_l = FastDiv((uint32_t)(cc * ff));
    p.div_ff = FastDiv((uint32_t)ff);
    p.div_fw = FastDiv((uint32_t)fw);
    p.div_nchunk = FastDiv((uint32_t)p.nchunk);
    p.div_oh = FastDiv((uint32_t)oh);
    p.div_fh = FastDiv((uint32_t)fh);
    p.div_span = FastDiv((uint32_t)span);
    p.div_nslot = FastDiv((uint32_t)std::max(1, p.nslot));
    p.div_npad = FastDiv((uint32_t)std::max(1, p.npad));
    const int64_t nblocks = bs * oh * p.nchunk;
    if (nblocks > 0x7FFFFFF0ll) return fail(AGH_ERANGE, "%s: too many workgroups", name);
    const size_t smem = (size_t)lds_bytes(cc);
    p.nblocks = (int)nblocks;
    p.per_xcd = (int)((nblocks + 7) / 8);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)(p.per_xcd * 8)), dim3(kThreads), smem, stream(), (const T *)x, (T *)y, p);
    };
    if (vec && vstage) launch(im2col_lds_kernel<T, VEC, true>);
    else if (vec) launch(im2col_lds_kernel<T, VEC, false>);
    else if (vstage) launch(im2col_lds_kernel<T, 1, true>);
    else launch(im2col_lds_kernel<T, 1, false>);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// ----------------------------------------------------------------- col2im ----
//
// Gather form: one thread owns one output pixel y[b,ci,hy,wy] and adds the patch entries
// that map onto it in the order the host loop meets them: patch row hi ascending, then
// patch column wi ascending (filter taps fi, fj therefore DEscending).  The accumulator has
// the element type, so a bf16 sum is rounded after every add, exactly like the host.
struct Col2imParams {
    int bs, c, ih, iw, oh, ow;  // ih, iw: patch grid; oh, ow: image
    int fh, fw, ph, pw, sh, sw, dh, dw;
    int ktot;
    FastDiv div_ow, div_oh, div_c, div_sh, div_sw;
};

template <typename T>
__global__ __launch_bounds__(kThreads) void col2im_gather_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                  Col2imParams p, size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    // e = ((b*c + ci)*oh + hy)*ow + wy ; planes < 2^31 checked on the host
    const size_t plane_sz = (size_t)p.oh * p.ow;
    const uint32_t plane = (uint32_t)(e / plane_sz);
    const uint32_t rem = (uint32_t)(e - (size_t)plane * plane_sz);
    uint32_t hy, wy, b, ci;
    p.div_ow.divmod(rem, hy, wy);
    p.div_c.divmod(plane, b, ci);
    const int ff = p.fh * p.fw;
    const T *xb = x + (size_t)b * p.ih * p.iw * p.ktot + (size_t)ci * ff;
    // Host order: fi descending (patch row ascending), then fj descending.  Every tap is LOADED, from a clamped
    // address, and an entry that does not exist contributes +0: the accumulator starts at +0 and a sum that
    // started at +0 is never -0, so adding +0 changes nothing, exactly like the host's skipped iteration, and
    // the loads no longer wait for one another behind branches.
    T acc = Elem<T>::zero();
    for (int fi = p.fh - 1; fi >= 0; --fi) {
        const int th = (int)hy + p.ph - fi * p.dh;
        uint32_t hid, rh;
        p.div_sh.divmod((uint32_t)max(th, 0), hid, rh);
        const bool hok = th >= 0 && rh == 0 && hid < (uint32_t)p.ih;
        const uint32_t hc = min(hid, (uint32_t)p.ih - 1);
        constexpr int G = 8;  // taps requested together
        for (int fj0 = p.fw - 1; fj0 >= 0; fj0 -= G) {
            T v[G];
            bool ok[G];
#pragma unroll
            for (int u = 0; u < G; ++u) {
                const int fj = fj0 - u;
                const int fjc = max(fj, 0);
                const int tw = (int)wy + p.pw - fjc * p.dw;
                uint32_t wid, rw;
                p.div_sw.divmod((uint32_t)max(tw, 0), wid, rw);
                ok[u] = hok && fj >= 0 && tw >= 0 && rw == 0 && wid < (uint32_t)p.iw;
                const uint32_t wc = min(wid, (uint32_t)p.iw - 1);
                v[u] = xb[((size_t)hc * p.iw + wc) * p.ktot + fi * p.fw + fjc];
            }
#pragma unroll
            for (int u = 0; u < G; ++u) {
                const T add = ok[u] ? v[u] : Elem<T>::zero();
                acc = Elem<T>::from_f32(Elem<T>::raw(acc) + Elem<T>::raw(add));
            }
        }
    }
    y[e] = acc;
}

// Streaming form, used whenever its tiles fit in LDS.  One workgroup owns a band of image rows of
// one image and a chunk of cc channels and walks the patch rows hi that touch the band in ascending
// order.  Per step it copies the cc*fh*fw-wide segments of the gw patches of that patch row into LDS
// with coalesced 4-byte loads (requested one step ahead, held in registers meanwhile), then every
// thread adds, for the pixel columns (channel, wy) it owns, the entries that fall on them: taps fj
// descending = patch column wi ascending.  Sums live in an LDS ring of (fh-1)*dh+1 image rows per
// column; a row is final once the walk has passed its last patch row, and is then written out and
// its ring slot cleared.  Each patch entry is read from HBM exactly once (plus the fh-1 patch rows
// that two neighbouring bands both need), and the order of the adds per pixel is the host's.
struct Col2imRingParams {
    int c, gh, gw, ih, iw;  // patch grid gh x gw, image ih x iw
    int fh, fw, ph, pw, sh, sw, dh, dw;
    int ktot, cc, nchunk, nband, band_rows;
    int ngroup;  // images * bands
    int rows;    // patch rows per step (unit-stride kernel)
    int lw;     // 32-bit words per patch segment (cc*fh*fw elements)
    int pitch;  // LDS pitch of a staged segment (elements); an odd number of words
    int rh;     // ring rows
    FastDiv div_nchunk, div_nband, div_iw, div_lw, div_sw, div_rh;
};

constexpr int kCol2imPrefetch = 32;  // 32-bit words a thread holds for the next step

template <typename T>
__global__ __launch_bounds__(kThreads) void col2im_ring_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                Col2imRingParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int PF = kCol2imPrefetch;
    constexpr int EPW = 4 / (int)sizeof(T);  // elements per 32-bit word
    const int tid = threadIdx.x;
    const int ncol = p.cc * p.iw;
    uint32_t *ring = (uint32_t *)smem_raw;  // [rh][ncol], one 32-bit slot per running sum
    T *stage = (T *)(ring + p.rh * ncol);   // [gw][pitch]
    uint32_t *stage32 = (uint32_t *)stage;
    uint32_t t0, band, chunk, b;
    p.div_nband.divmod(blockIdx.x, t0, band);
    p.div_nchunk.divmod(t0, b, chunk);
    const int c0 = chunk * p.cc, ff = p.fh * p.fw;
    const int hy0 = band * p.band_rows, hy1 = min(p.ih, hy0 + p.band_rows);
    // patch rows whose window [hi*sh - ph, hi*sh - ph + (fh-1)*dh] meets [hy0, hy1)
    const int lo_num = hy0 + p.ph - (p.fh - 1) * p.dh;
    const int hi_lo = lo_num <= 0 ? 0 : (lo_num + p.sh - 1) / p.sh;
    const int hi_hi = min(p.gh - 1, (hy1 - 1 + p.ph) / p.sh);

    for (int i = tid; i < p.rh * ncol; i += kThreads) ring[i] = 0;

    const uint32_t nwords = (uint32_t)p.gw * p.lw;
    const int ktotw = p.ktot / EPW, pitchw = p.pitch / EPW;
    uint32_t reg[PF];
    auto prefetch = [&](int hi) {
        const uint32_t *src = (const uint32_t *)(x + ((size_t)b * p.gh + hi) * p.gw * p.ktot + (size_t)c0 * ff);
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            const uint32_t e = tid + i * kThreads;
            uint32_t wi, k;
            p.div_lw.divmod(e, wi, k);
            reg[i] = 0;
            if (e < nwords) reg[i] = src[(size_t)wi * ktotw + k];
        }
    };
    auto slot_to = [](uint32_t v) -> T {
        if constexpr (sizeof(T) == 4) return __uint_as_float(v);
        else return (T)v;
    };
    auto to_slot = [](T v) -> uint32_t {
        if constexpr (sizeof(T) == 4) return __float_as_uint(v);
        else return (uint32_t)v;
    };

    if (hi_lo <= hi_hi) prefetch(hi_lo);
    int next_flush = hy0;
    for (int hi = hi_lo; hi <= hi_hi; ++hi) {
        __syncthreads();  // the previous step's reads of the stage (and the clearing of the ring) are done
#pragma unroll
        for (int i = 0; i < PF; ++i) {
            const uint32_t e = tid + i * kThreads;
            uint32_t wi, k;
            p.div_lw.divmod(e, wi, k);
            if (e < nwords) stage32[wi * pitchw + k] = reg[i];
        }
        __syncthreads();
        if (hi < hi_hi) prefetch(hi + 1);
        const int start = hi * p.sh - p.ph;
        const int fend = hi == hi_hi ? hy1 : min(hy1, start + p.sh);
        for (int col = tid; col < ncol; col += kThreads) {
            uint32_t cl, wy;
            p.div_iw.divmod((uint32_t)col, cl, wy);
            const T *sc = stage + cl * ff;
            for (int fi = 0; fi < p.fh; ++fi) {
                const int hy = start + fi * p.dh;
                if (hy < hy0 || hy >= hy1) continue;
                const int slot = (int)(hy - p.div_rh.div((uint32_t)hy) * p.rh) * ncol + col;
                T acc = slot_to(ring[slot]);
                for (int fj = p.fw - 1; fj >= 0; --fj) {
                    const int tw = (int)wy + p.pw - fj * p.dw;
                    if (tw < 0) continue;
                    uint32_t wi, rw;
                    p.div_sw.divmod((uint32_t)tw, wi, rw);
                    if (rw != 0 || wi >= (uint32_t)p.gw) continue;
                    const T v = sc[wi * p.pitch + fi * p.fw + fj];
                    acc = Elem<T>::from_f32(Elem<T>::raw(acc) + Elem<T>::raw(v));
                }
                ring[slot] = to_slot(acc);
            }
            // rows no later patch row reaches: write them out; rows outside the window got nothing
            T *yc = y + (((size_t)b * p.c + c0 + cl) * p.ih) * (size_t)p.iw + wy;
            for (int hy = next_flush; hy < fend; ++hy) {
                T val = Elem<T>::zero();
                if (hy >= start && hy < start + p.rh) {
                    const int slot = (int)(hy - p.div_rh.div((uint32_t)hy) * p.rh) * ncol + col;
                    val = slot_to(ring[slot]);
                    ring[slot] = 0;
                }
                yc[(size_t)hy * p.iw] = val;
            }
        }
        next_flush = max(next_flush, fend);
    }
    // band rows no patch row touches at all
    for (int col = tid; col < ncol; col += kThreads) {
        uint32_t cl, wy;
        p.div_iw.divmod((uint32_t)col, cl, wy);
        T *yc = y + (((size_t)b * p.c + c0 + cl) * p.ih) * (size_t)p.iw + wy;
        for (int hy = next_flush; hy < hy1; ++hy) yc[(size_t)hy * p.iw] = Elem<T>::zero();
    }
}

// Unit stride and dilation, square filter known at compile time: the streaming form with everything
// the general kernel computes per tap hoisted or folded.  The stage carries FW-1-pw all-zero segments
// on either side, so a tap never has to ask whether its patch column exists (adding +0 to a running
// sum changes nothing: a sum that starts at +0 can never be -0).  The F running sums of a pixel
// column sit in registers and move down one place per step, the finished one leaving for memory.
// Per thread and step: eight 16-byte loads, the stage write, and per owned pixel column F*F LDS
// reads and adds.
// Workgroup ids are dealt round-robin to the 8 XCDs, each with an L2 of its own; the chunks of one
// (image, band) share cache lines where their segments meet, so they are given ids 8 apart: same
// XCD, dispatched together.
template <typename T, int F>
__global__ __launch_bounds__(kThreads) void col2im_ring_unit_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                     Col2imRingParams p) {
    extern __shared__ __align__(16) unsigned char smem_raw[];
    constexpr int PFV = kCol2imPrefetch / 4;  // 16-byte vectors a thread holds for the next step
    constexpr int EPW = 4 / (int)sizeof(T);
    constexpr int NCOL = 4;                   // pixel columns per thread (cc*iw <= NCOL*kThreads)
    const int tid = threadIdx.x;
    const int ncol = p.cc * p.iw;
    const int padl = max(0, F - 1 - p.pw);
    T *stage = (T *)smem_raw;                 // [gw + 2*padl][pitch]
    uint32_t *stage32 = (uint32_t *)stage;
    uint32_t slot8, chunk, b, band;
    p.div_nchunk.divmod(blockIdx.x >> 3, slot8, chunk);
    const uint32_t group = slot8 * 8 + (blockIdx.x & 7);  // (image, band) pair
    if (group >= (uint32_t)p.ngroup) return;
    p.div_nband.divmod(group, b, band);
    constexpr int ff = F * F;
    const int c0 = chunk * p.cc;
    const int hy0 = band * p.band_rows, hy1 = min(p.ih, hy0 + p.band_rows);
    const int hi_lo = max(0, hy0 + p.ph - (F - 1));
    const int hi_hi = min(p.gh - 1, hy1 - 1 + p.ph);
    const int ktotw = p.ktot / EPW, pitchw = p.pitch / EPW;

    for (int r = 0; r < p.rows; ++r)
        for (int i = tid; i < padl * pitchw; i += kThreads) {
            stage32[r * (p.gw + 2 * padl) * pitchw + i] = 0;
            stage32[(r * (p.gw + 2 * padl) + p.gw + padl) * pitchw + i] = 0;
        }

    // launch-constant per-thread offsets.  A step takes `rows` patch rows; vector slot i of a thread
    // belongs to patch row i / per_row of the step (wave-uniform), so its base pointer is a scalar.
    const int lv = p.lw / 4;
    const uint32_t nvec = (uint32_t)p.gw * lv;
    const int per_row = (nvec + kThreads - 1) / kThreads, rows = p.rows;
    const int nseg = p.gw + 2 * padl;
    uint32_t src_off[PFV], dst_off[PFV];
#pragma unroll
    for (int i = 0; i < PFV; ++i) {
        const int r = i / per_row;
        const uint32_t e = tid + (i - r * per_row) * kThreads;
        uint32_t wi, kv;
        p.div_lw.divmod(e, wi, kv);  // divides by lv for this kernel
        src_off[i] = (e < nvec && r < rows) ? wi * ktotw + kv * 4 : 0xFFFFFFFFu;
        dst_off[i] = (r * nseg + wi + padl) * pitchw + kv * 4;
    }
    int tap_base[NCOL];
    T *ycol[NCOL];
    T acc[NCOL][F];
#pragma unroll
    for (int j = 0; j < NCOL; ++j) {
        const int col = tid + j * kThreads;
        uint32_t cl, wy;
        p.div_iw.divmod((uint32_t)min(col, ncol - 1), cl, wy);
        // element offset of tap fj = 0 of filter row 0; tap (fi, fj) is at + fi*F - fj*(pitch-1)
        tap_base[j] = ((int)wy + p.pw + padl) * p.pitch + (int)cl * ff;
        ycol[j] = y + (((size_t)b * p.c + c0 + cl) * p.ih) * (size_t)p.iw + wy;
#pragma unroll
        for (int fi = 0; fi < F; ++fi) acc[j][fi] = Elem<T>::zero();
    }
    const int tap_step = p.pitch - 1;

    u32x4 reg[PFV];
    auto prefetch = [&](int hi) {
#pragma unroll
        for (int i = 0; i < PFV; ++i) {
            const int r = i / per_row;
            // rows past the last one re-read it (never used): keeps the loads unconditional per row
            const int hr = min(hi + r, hi_hi);
            const uint32_t *src = (const uint32_t *)(x + ((size_t)b * p.gh + hr) * p.gw * p.ktot + (size_t)c0 * ff);
            if (src_off[i] != 0xFFFFFFFFu) reg[i] = *(const u32x4 *)(src + src_off[i]);
        }
    };

    if (hi_lo <= hi_hi) prefetch(hi_lo);
    for (int hi0 = hi_lo; hi0 <= hi_hi; hi0 += rows) {
        __syncthreads();  // the previous step's reads of the stage are done
#pragma unroll
        for (int i = 0; i < PFV; ++i)
            if (src_off[i] != 0xFFFFFFFFu) {
                stage32[dst_off[i] + 0] = reg[i].x;
                stage32[dst_off[i] + 1] = reg[i].y;
                stage32[dst_off[i] + 2] = reg[i].z;
                stage32[dst_off[i] + 3] = reg[i].w;
            }
        __syncthreads();
        if (hi0 + rows <= hi_hi) prefetch(hi0 + rows);
        for (int r = 0; r < rows && hi0 + r <= hi_hi; ++r) {
            // acc[j][fi] is the running sum of image row start + fi
            const int hi = hi0 + r;
            const int start = hi - p.ph;
            const bool last = hi == hi_hi;
            const T *st = stage + r * nseg * p.pitch;
#pragma unroll
            for (int j = 0; j < NCOL; ++j) {
                const int col = tid + j * kThreads;
                if (col < ncol) {
#pragma unroll
                    for (int fi = 0; fi < F; ++fi) {
                        const int hy = start + fi;
                        if (hy >= hy0 && hy < hy1) {  // wave-uniform
#pragma unroll
                            for (int fj = F - 1; fj >= 0; --fj) {
                                const T v = st[tap_base[j] - fj * tap_step + fi * F];
                                acc[j][fi] = Elem<T>::from_f32(Elem<T>::raw(acc[j][fi]) + Elem<T>::raw(v));
                            }
                        }
                    }
                    // row `start` gets nothing from later patch rows; after the last patch row all rows are final
                    if (start >= hy0 && start < hy1) ycol[j][(size_t)start * p.iw] = acc[j][0];
                    if (last) {
#pragma unroll
                        for (int fi = 1; fi < F; ++fi)
                            if (start + fi >= hy0 && start + fi < hy1) ycol[j][(size_t)(start + fi) * p.iw] = acc[j][fi];
                    }
#pragma unroll
                    for (int fi = 0; fi + 1 < F; ++fi) acc[j][fi] = acc[j][fi + 1];
                    acc[j][F - 1] = Elem<T>::zero();
                }
            }
        }
    }
}

// Picks the chunk/band split of the streaming kernel; false when the geometry does not fit.
template <typename T>
bool col2im_ring_plan(Col2imRingParams &p, size_t &smem, int64_t &nblocks, bool unit, const void *x, int64_t bs, int64_t c,
                      int64_t gh, int64_t gw, int64_t ih, int64_t iw, int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                      int64_t sh, int64_t sw, int64_t dh, int64_t dw) {
    constexpr int64_t es = sizeof(T), epw = 4 / es;
    const int64_t ff = fh * fw, ktot = c * ff;
    if (((uintptr_t)x & 3) != 0 || ktot % epw != 0) return false;
    // the unit-stride kernel loads 16-byte vectors and carries zero segments around the stage
    if (unit && (((uintptr_t)x & 15) != 0 || (ktot * es) % 16 != 0)) return false;
    const int64_t segs = unit ? gw + 2 * std::max<int64_t>(0, fw - 1 - pw) : gw;
    const int64_t rh = (fh - 1) * dh + 1;
    constexpr int64_t kLdsBudget = 48 * 1024;
    int64_t cc = 0, lds = 0, pitch = 0, nrows = 1;
    for (int64_t d = c; d >= 1; --d) {
        if (c % d != 0 || (d * ff) % epw != 0) continue;
        if (unit && ((d * ff * es) % 16 != 0 || d * iw > 4 * kThreads)) continue;
        const int64_t lw = d * ff / epw;
        if (gw * lw > (int64_t)kThreads * kCol2imPrefetch) continue;
        const int64_t pitchw = lw | 1;  // odd: threads of a wave walk patches, i.e. whole pitches
        int64_t need = rh * d * iw * 4 + segs * pitchw * 4;
        if (unit) {
            // as many patch rows per step as the prefetch registers and 40 KB of LDS hold
            const int64_t per_row = (gw * (lw / 4) + kThreads - 1) / kThreads;
            nrows = std::max<int64_t>(1, std::min<int64_t>({(int64_t)(kCol2imPrefetch / 4) / per_row, gh,
                                                             (40 * 1024) / (segs * pitchw * 4)}));
            need = nrows * segs * pitchw * 4;
        }
        if (need > kLdsBudget) continue;
        cc = d; lds = need; pitch = pitchw * epw;
        break;
    }
    if (cc == 0) return false;
    const int64_t nchunk = c / cc;
    const int64_t cus = compute_units() > 0 ? compute_units() : 256;
    const int64_t resident = cus * std::min<int64_t>(unit ? 4 : 2, (160 * 1024) / lds);  // registers allow 4 / 2
    // bands: more of them fill the chip, fewer of them re-read fewer boundary patch rows
    int64_t best_nb = 1, best_cost = -1;
    for (int64_t nb = 1; nb <= std::min<int64_t>(ih, 32); ++nb) {
        const int64_t rows = (ih + nb - 1) / nb;
        if ((ih + rows - 1) / rows != nb) continue;  // would leave an empty band
        const int64_t steps = ((rows + (fh - 1) * dh) / sh + nrows) / nrows;
        const int64_t waves = (bs * nchunk * nb + resident - 1) / resident;
        const int64_t cost = waves * (steps + 2);
        if (best_cost < 0 || cost < best_cost) { best_cost = cost; best_nb = nb; }
    }
    nblocks = unit ? ((bs * best_nb + 7) / 8) * 8 * nchunk : bs * nchunk * best_nb;
    p.ngroup = bs * best_nb;
    p.rows = nrows;
    if (nblocks > 0x7FFFFFFFll) return false;
    p.c = c; p.gh = gh; p.gw = gw; p.ih = ih; p.iw = iw;
    p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
    p.ktot = ktot; p.cc = cc; p.nchunk = nchunk; p.nband = best_nb; p.band_rows = (ih + best_nb - 1) / best_nb;
    p.lw = cc * ff / epw; p.pitch = pitch; p.rh = rh;
    p.div_nchunk = FastDiv((uint32_t)nchunk);
    p.div_nband = FastDiv((uint32_t)best_nb);
    p.div_iw = FastDiv((uint32_t)iw);
    p.div_lw = FastDiv((uint32_t)(unit ? p.lw / 4 : p.lw));
    p.div_sw = FastDiv((uint32_t)sw);
    p.div_rh = FastDiv((uint32_t)rh);
    smem = (size_t)lds;
    return true;
}

template <typename T>
int col2im_launch(const char *name, const void *x, void *y, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                  int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t sh, int64_t sw, int64_t dh, int64_t dw) {
    AGH_API_ENTER();
    if (bs < 0 || c < 0 || ih < 0 || iw < 0 || fh < 1 || fw < 1 || ph < 0 || pw < 0 || sh < 1 || sw < 1 || dh < 1 || dw < 1)
        return fail(AGH_EINVAL, "%s: invalid shape/options", name);
    if (bs == 0 || c == 0 || ih == 0 || iw == 0) return AGH_OK;
    const int64_t oh = col2im_out(ih, fh, ph, sh, dh), ow = col2im_out(iw, fw, pw, sw, dw);
    if (oh < 1 || ow < 1) return fail(AGH_EINVAL, "%s: padding larger than the reconstructed image", name);
    const int64_t lim = (int64_t)1 << 30;
    if (bs > lim || c > lim || ih > lim || iw > lim || oh > lim || ow > lim || fh > lim || fw > lim || ph > lim ||
        pw > lim || sh > lim || sw > lim || dh > lim || dw > lim || c * fh * fw > lim || bs * c > lim ||
        oh * ow > lim || oh + ph > lim || ow + pw > lim)
        return fail(AGH_ERANGE, "%s: dimension too large", name);
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    Col2imParams p;
    p.bs = bs; p.c = c; p.ih = ih; p.iw = iw; p.oh = oh; p.ow = ow;
    p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
    // The streaming (ring) kernels pay off when there is a patch matrix to stream; below a few megabytes one
    // gathering thread per image pixel finishes sooner.  AGH_COL2IM_RING=1 / 0 forces / forbids the ring form.
    const int64_t patch_bytes = bs * ih * iw * c * fh * fw * (int64_t)sizeof(T);
    const char *ring_env = getenv("AGH_COL2IM_RING");
    const bool use_ring = ring_env ? atoi(ring_env) != 0 : patch_bytes > ((int64_t)4 << 20);
    if (use_ring) {
        Col2imRingParams rp;
        size_t smem = 0;
        int64_t nblocks = 0;
        const bool unit_geom = sh == 1 && sw == 1 && dh == 1 && dw == 1 && fh == fw &&
                               (fh == 1 || fh == 2 || fh == 3 || fh == 5 || fh == 7);
        auto launch = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3((unsigned)nblocks), dim3(kThreads), smem, stream(), (const T *)x, (T *)y, rp);
        };
        if (unit_geom && col2im_ring_plan<T>(rp, smem, nblocks, true, x, bs, c, ih, iw, oh, ow, fh, fw, ph, pw, sh, sw, dh, dw)) {
            switch (fh) {
                case 1: launch(col2im_ring_unit_kernel<T, 1>); break;
                case 2: launch(col2im_ring_unit_kernel<T, 2>); break;
                case 3: launch(col2im_ring_unit_kernel<T, 3>); break;
                case 5: launch(col2im_ring_unit_kernel<T, 5>); break;
                default: launch(col2im_ring_unit_kernel<T, 7>); break;
            }
            AGH_LAUNCH_CHECK(name);
            return AGH_OK;
        }
        if (col2im_ring_plan<T>(rp, smem, nblocks, false, x, bs, c, ih, iw, oh, ow, fh, fw, ph, pw, sh, sw, dh, dw)) {
            launch(col2im_ring_kernel<T>);
            AGH_LAUNCH_CHECK(name);
            return AGH_OK;
        }
    }
    p.ktot = c * fh * fw;
    p.div_ow = FastDiv((uint32_t)ow);
    p.div_oh = FastDiv((uint32_t)oh);
    p.div_c = FastDiv((uint32_t)c);
    p.div_sh = FastDiv((uint32_t)sh);
    p.div_sw = FastDiv((uint32_t)sw);
    const size_t total = (size_t)bs * c * oh * ow;
    size_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
    hipLaunchKernelGGL(col2im_gather_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(), (const T *)x,
                       (T *)y, p, total);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// ------------------------------------------- conv2 backward w.r.t. the input ----
// dx = col2im(dy_matrix * W) in one launch, for convolutions whose filter bank fits in LDS (as f32).  One thread
// owns one image pixel, walks the patch entries that land on it in the host's order like col2im_gather_kernel, and
// computes each entry where the separate GEMM would have: an f32 dot over the output channels, rounded once to T.
// The running sum then adds that rounded value in T, so the only difference from GEMM + col2im is the order of
// the f32 adds inside one dot product.
template <typename T, bool VEC, bool UNIT, int FW, int OCU, bool LDSG = false>
__global__ __launch_bounds__(kThreads) void conv2_backward_input_kernel(const T *__restrict__ dy, const T *__restrict__ w,
                                                                         T *__restrict__ y, Col2imParams p, int oc,
                                                                         size_t total) {
    static_assert(!LDSG || (FW > 0 && VEC && UNIT), "the LDS-staged gradient exists for the row-at-a-time form only");
    extern __shared__ __align__(16) unsigned char smem_raw[];
    float *wl = (float *)smem_raw;  // [ktot][oc]: the output channels of one tap are contiguous
    // eight elements of w are requested before the first is used: one at a time the staging alone would be
    // a chain of oc*ktot/256 memory latencies
    const int nw = oc * p.ktot;
    for (int i0 = threadIdx.x; i0 < nw; i0 += 8 * kThreads) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = w[min(i0 + u * kThreads, nw - 1)];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            const int i = i0 + u * kThreads;
            const int o = i / p.ktot, k = i - o * p.ktot;  // coalesced read of w[o][k]
            if (i < nw) wl[k * oc + o] = Elem<T>::to_f32(v[u]);
        }
    }
    const size_t plane_sz = (size_t)p.oh * p.ow;
    // LDSG: an image is at least a workgroup's worth of pixels, so the workgroup's pixels lie in at most two
    // images, whose gradient matrices [ih*iw][oc] are staged as f32 with a row pitch of oc + 4 (16-byte reads of
    // neighbouring rows then fall into different banks).  Each row is needed by up to fh*fw pixels: they now
    // read it from LDS instead of through L1.
    using S = std::conditional_t<LDSG, float, T>;  // element type the dot products read
    const int pitch = LDSG ? oc + 4 : oc;
    float *gl = wl + nw;
    uint32_t b0 = 0;
    if constexpr (LDSG) {
        const size_t e0 = (size_t)blockIdx.x * kThreads, e1 = min(e0 + kThreads, total) - 1;
        uint32_t c0, c1, b1;
        p.div_c.divmod((uint32_t)(e0 / plane_sz), b0, c0);
        p.div_c.divmod((uint32_t)(e1 / plane_sz), b1, c1);
        const int rows = (int)(b1 - b0 + 1) * p.ih * p.iw, ng = rows * oc;
        const T *src = dy + (size_t)b0 * p.ih * p.iw * oc;
        for (int i0 = threadIdx.x; i0 < ng; i0 += 8 * kThreads) {
            T v[8];
#pragma unroll
            for (int u = 0; u < 8; ++u) v[u] = src[min(i0 + u * kThreads, ng - 1)];
#pragma unroll
            for (int u = 0; u < 8; ++u) {
                const int i = i0 + u * kThreads;
                const int r = i / oc, o = i - r * oc;
                if (i < ng) gl[r * pitch + o] = Elem<T>::to_f32(v[u]);
            }
        }
    }
    __syncthreads();
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    const uint32_t plane = (uint32_t)(e / plane_sz);
    const uint32_t rem = (uint32_t)(e - (size_t)plane * plane_sz);
    uint32_t hy, wy, b, ci;
    p.div_ow.divmod(rem, hy, wy);
    p.div_c.divmod(plane, b, ci);
    const int ff = p.fh * p.fw;
    constexpr int EPC = 16 / (int)sizeof(S);
    const S *gb;
    if constexpr (LDSG) gb = gl + (size_t)(b - b0) * p.ih * p.iw * pitch;
    else gb = dy + (size_t)b * p.ih * p.iw * oc;
    T acc = Elem<T>::zero();
    for (int fi = p.fh - 1; fi >= 0; --fi) {
        // UNIT: stride 1 in both directions, so every image row / column is a patch row / column (no division)
        const int th = (int)hy + p.ph - fi * p.dh;
        uint32_t hid = (uint32_t)max(th, 0), rh = 0;
        if constexpr (!UNIT) p.div_sh.divmod((uint32_t)max(th, 0), hid, rh);
        const bool hok = th >= 0 && rh == 0 && hid < (uint32_t)p.ih;
        const S *grow = gb + (size_t)min(hid, (uint32_t)p.ih - 1) * p.iw * pitch;
        const float *wrow = wl + (size_t)(ci * ff + fi * p.fw) * oc;
        if constexpr (FW > 0 && VEC && UNIT) {
            // a whole filter row at a time (fw == FW): the FW row vectors of one channel chunk are requested
            // together, so a pixel waits for fh * oc/EPC loads in a row instead of fh * fw * oc/EPC
            const S *gp[FW];
            bool okj[FW];
            float d[FW];
#pragma unroll
            for (int fj = 0; fj < FW; ++fj) {
                const int tw = (int)wy + p.pw - fj * p.dw;
                okj[fj] = hok && tw >= 0 && tw < p.iw;
                gp[fj] = grow + (size_t)min(max(tw, 0), p.iw - 1) * pitch;
                d[fj] = 0.0f;
            }
            // OCU channel chunks per trip (oc is a multiple of OCU * EPC): FW * OCU loads in flight
            for (int o0 = 0; o0 < oc; o0 += OCU * EPC) {
                u32x4 v[OCU][FW];
#pragma unroll
                for (int c = 0; c < OCU; ++c)
#pragma unroll
                    for (int fj = 0; fj < FW; ++fj) v[c][fj] = *(const u32x4 *)(gp[fj] + o0 + c * EPC);
#pragma unroll
                for (int c = 0; c < OCU; ++c)  // channels ascending inside every dot product
#pragma unroll
                    for (int fj = 0; fj < FW; ++fj) {
                        const float *wt = wrow + fj * oc + o0 + c * EPC;
                        const float4 w0 = *(const float4 *)wt;
                        const u32x4 q = v[c][fj];
                        if constexpr (sizeof(S) == 4) {
                            d[fj] = fmaf(__uint_as_float(q.x), w0.x, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.y), w0.y, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.z), w0.z, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.w), w0.w, d[fj]);
                        } else {
                            const float4 w1 = *(const float4 *)(wt + 4);
                            d[fj] = fmaf(__uint_as_float(q.x << 16), w0.x, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.x & 0xFFFF0000u), w0.y, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.y << 16), w0.z, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.y & 0xFFFF0000u), w0.w, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.z << 16), w1.x, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.z & 0xFFFF0000u), w1.y, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.w << 16), w1.z, d[fj]);
                            d[fj] = fmaf(__uint_as_float(q.w & 0xFFFF0000u), w1.w, d[fj]);
                        }
                    }
            }
#pragma unroll
            for (int fj = FW - 1; fj >= 0; --fj) {
                const T add = okj[fj] ? Elem<T>::from_f32(d[fj]) : Elem<T>::zero();
                acc = Elem<T>::from_f32(Elem<T>::raw(acc) + Elem<T>::raw(add));
            }
            continue;
        }
        for (int fj = p.fw - 1; fj >= 0; --fj) {
            const int tw = (int)wy + p.pw - fj * p.dw;
            uint32_t wid = (uint32_t)max(tw, 0), rw = 0;
            if constexpr (!UNIT) p.div_sw.divmod((uint32_t)max(tw, 0), wid, rw);
            const bool ok = hok && tw >= 0 && rw == 0 && wid < (uint32_t)p.iw;
            // the row is read from a clamped address whether or not the entry exists (it then adds +0)
            const T *g = (const T *)(const void *)grow + (size_t)min(wid, (uint32_t)p.iw - 1) * oc;  // not with LDSG
            const float *wt = wrow + fj * oc;
            float d = 0.0f;
            if constexpr (VEC) {
                for (int o = 0; o < oc; o += EPC) {
                    const u32x4 v = *(const u32x4 *)(g + o);
                    const float4 w0 = *(const float4 *)(wt + o);
                    if constexpr (sizeof(T) == 4) {
                        d = fmaf(__uint_as_float(v.x), w0.x, d);
                        d = fmaf(__uint_as_float(v.y), w0.y, d);
                        d = fmaf(__uint_as_float(v.z), w0.z, d);
                        d = fmaf(__uint_as_float(v.w), w0.w, d);
                    } else {
                        const float4 w1 = *(const float4 *)(wt + o + 4);
                        d = fmaf(__uint_as_float(v.x << 16), w0.x, d);
                        d = fmaf(__uint_as_float(v.x & 0xFFFF0000u), w0.y, d);
                        d = fmaf(__uint_as_float(v.y << 16), w0.z, d);
                        d = fmaf(__uint_as_float(v.y & 0xFFFF0000u), w0.w, d);
                        d = fmaf(__uint_as_float(v.z << 16), w1.x, d);
                        d = fmaf(__uint_as_float(v.z & 0xFFFF0000u), w1.y, d);
                        d = fmaf(__uint_as_float(v.w << 16), w1.z, d);
                        d = fmaf(__uint_as_float(v.w & 0xFFFF0000u), w1.w, d);
                    }
                }
            } else {
                for (int o = 0; o < oc; ++o) d = fmaf(Elem<T>::to_f32(g[o]), wt[o], d);
            }
            const T add = ok ? Elem<T>::from_f32(d) : Elem<T>::zero();
            acc = Elem<T>::from_f32(Elem<T>::raw(acc) + Elem<T>::raw(add));
        }
    }
    y[e] = acc;
}

template <typename T>
int conv2_backward_input_launch(const char *name, const void *dy, const void *w, void *dx, int64_t bs, int64_t c,
                                int64_t ih, int64_t iw, int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw,
                                int64_t sh, int64_t sw, int64_t dh, int64_t dw) {
    AGH_API_ENTER();
    if (bs < 0 || c < 0 || ih < 0 || iw < 0 || oc < 0 || fh < 1 || fw < 1 || ph < 0 || pw < 0 || sh < 1 || sw < 1 ||
        dh < 1 || dw < 1)
        return fail(AGH_EINVAL, "%s: invalid shape/options", name);
    if (bs == 0 || c == 0 || ih == 0 || iw == 0) return AGH_OK;
    const int64_t oh = col2im_out(ih, fh, ph, sh, dh), ow = col2im_out(iw, fw, pw, sw, dw);
    if (oh < 1 || ow < 1) return fail(AGH_EINVAL, "%s: padding larger than the reconstructed image", name);
    const int64_t lim = (int64_t)1 << 30;
    if (bs > lim || c > lim || ih > lim || iw > lim || oh > lim || ow > lim || fh > lim || fw > lim || ph > lim ||
        pw > lim || sh > lim || sw > lim || dh > lim || dw > lim || oc > lim || c * fh * fw > lim || bs * c > lim ||
        oh * ow > lim || oh + ph > lim || ow + pw > lim)
        return fail(AGH_ERANGE, "%s: dimension too large", name);
    const int64_t ktot = c * fh * fw;
    if (oc * ktot * 4 > 64 * 1024)
        return fail(AGH_ERANGE, "%s: filter bank of %lld x %lld does not fit in LDS; use gemm + col2im", name,
                    (long long)oc, (long long)ktot);
    if (!dy || !w || !dx) return fail(AGH_ENULL, "%s: null buffer", name);
    Col2imParams p;
    p.bs = bs; p.c = c; p.ih = ih; p.iw = iw; p.oh = oh; p.ow = ow;
    p.fh = fh; p.fw = fw; p.ph = ph; p.pw = pw; p.sh = sh; p.sw = sw; p.dh = dh; p.dw = dw;
    p.ktot = (int)ktot;
    p.div_ow = FastDiv((uint32_t)ow);
    p.div_oh = FastDiv((uint32_t)oh);
    p.div_c = FastDiv((uint32_t)c);
    p.div_sh = FastDiv((uint32_t)sh);
    p.div_sw = FastDiv((uint32_t)sw);
    const size_t total = (size_t)bs * c * oh * ow;
    size_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
    const size_t smem = (size_t)(oc * ktot * 4);
    constexpr int EPC = 16 / (int)sizeof(T);
    const bool vec = oc > 0 && oc % EPC == 0 && ((uintptr_t)dy & 15) == 0;
    const bool unit = sh == 1 && sw == 1;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kThreads), smem, stream(), (const T *)dy, (const T *)w,
                           (T *)dx, p, (int)oc, total);
    };
    // f32: the gradient matrices of two images next to the filter bank in LDS, when an image holds at least a
    // workgroup's worth of pixels (a workgroup then touches at most two images).  Measured at conv2 of LeNet5,
    // batch 100: 12.3 -> 8.8 us; the bf16 rows are half as long and gain nothing (8.6 -> 9.4 us), so they stay
    // on the path through L1.
    const size_t smem_g = smem + (size_t)2 * ih * iw * (oc + 4) * 4;
    const bool ldsg = sizeof(T) == 4 && vec && unit && (fw == 5 || fw == 3) && c * oh * ow >= kThreads &&
                      smem_g <= 64 * 1024;
    if constexpr (sizeof(T) == 4) if (ldsg) {
        const int ch = (int)(oc / 4);
        const int u = ch % 4 == 0 ? 4 : ch % 2 == 0 ? 2 : 1;
        auto launch_g = [&](auto kernel) {
            hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(kThreads), smem_g, stream(), (const T *)dy,
                               (const T *)w, (T *)dx, p, (int)oc, total);
        };
        if (fw == 5) {
            if (u == 4) launch_g(conv2_backward_input_kernel<T, true, true, 5, 4, true>);
            else if (u == 2) launch_g(conv2_backward_input_kernel<T, true, true, 5, 2, true>);
            else launch_g(conv2_backward_input_kernel<T, true, true, 5, 1, true>);
        } else {
            if (u == 4) launch_g(conv2_backward_input_kernel<T, true, true, 3, 4, true>);
            else if (u == 2) launch_g(conv2_backward_input_kernel<T, true, true, 3, 2, true>);
            else launch_g(conv2_backward_input_kernel<T, true, true, 3, 1, true>);
        }
        AGH_LAUNCH_CHECK(name);
        return AGH_OK;
    }
    const int chunks = vec ? (int)(oc / EPC) : 0;
    const int ocu = chunks % 4 == 0 ? 4 : chunks % 2 == 0 ? 2 : 1;
    if (vec && unit && fw == 5) {
        if (ocu == 4) launch(conv2_backward_input_kernel<T, true, true, 5, 4>);
        else if (ocu == 2) launch(conv2_backward_input_kernel<T, true, true, 5, 2>);
        else launch(conv2_backward_input_kernel<T, true, true, 5, 1>);
    } else if (vec && unit && fw == 3) {
        if (ocu == 4) launch(conv2_backward_input_kernel<T, true, true, 3, 4>);
        else if (ocu == 2) launch(conv2_backward_input_kernel<T, true, true, 3, 2>);
        else launch(conv2_backward_input_kernel<T, true, true, 3, 1>);
    } else if (vec && unit) launch(conv2_backward_input_kernel<T, true, true, 0, 1>);
    else if (vec) launch(conv2_backward_input_kernel<T, true, false, 0, 1>);
    else if (unit) launch(conv2_backward_input_kernel<T, false, true, 0, 1>);
    else launch(conv2_backward_input_kernel<T, false, false, 0, 1>);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// --------------------------------------------------------------- max pool ----
struct PoolParams {
    int ih, iw, oh, ow, h, w, sh, sw;
    FastDiv div_ow, div_oh;
    FastDiv div_gpr;  // 2x2 vector kernels: 16-byte groups per input row
};

template <typename T>
__global__ __launch_bounds__(kThreads) void max_pool2_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                              PoolParams p, size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    const size_t osz = (size_t)p.oh * p.ow;
    const size_t plane = e / osz;
    const uint32_t rem = (uint32_t)(e - plane * osz);
    uint32_t ho, wo;
    p.div_ow.divmod(rem, ho, wo);
    const T *src = x + (plane * p.ih + (size_t)ho * p.sh) * p.iw + (size_t)wo * p.sw;
    T m = src[0];
    float mf = Elem<T>::raw(m);
    for (int fi = 0; fi < p.h; ++fi)
        for (int fj = 0; fj < p.w; ++fj) {
            T v = src[(size_t)fi * p.iw + fj];
            float vf = Elem<T>::raw(v);
            if (vf > mf) { m = v; mf = vf; }
        }
    y[e] = m;
}

// Disjoint windows (sh >= h and sw >= w): one thread per window, in place.
template <typename T>
__global__ __launch_bounds__(kThreads) void max_pool2_backward_kernel(T *__restrict__ dx, const T *__restrict__ dy,
                                                                       PoolParams p, size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    const size_t osz = (size_t)p.oh * p.ow;
    const size_t plane = e / osz;
    const uint32_t rem = (uint32_t)(e - plane * osz);
    uint32_t ho, wo;
    p.div_ow.divmod(rem, ho, wo);
    T *win = dx + (plane * p.ih + (size_t)ho * p.sh) * p.iw + (size_t)wo * p.sw;
    float mf = Elem<T>::raw(win[0]);
    int am = 0;
    for (int fi = 0; fi < p.h; ++fi)
        for (int fj = 0; fj < p.w; ++fj) {
            int off = fi * p.iw + fj;
            float vf = Elem<T>::raw(win[off]);
            if (vf > mf) { mf = vf; am = off; }
        }
    // `0 + dy` in T, as the host's `+=` on the zeroed cell computes it
    const T g = Elem<T>::from_f32(0.0f + Elem<T>::raw(dy[e]));
    for (int fi = 0; fi < p.h; ++fi)
        for (int fj = 0; fj < p.w; ++fj) {
            int off = fi * p.iw + fj;
            win[off] = (off == am) ? g : Elem<T>::zero();
        }
}

// 2x2 windows, stride 2, rows of whole 16-byte vectors: a work item is one 16-byte vector from each of the two
// rows of a row pair (4 f32 / 8 bf16 elements: 2 / 4 neighbouring windows), so every load instruction of a wave
// covers 1 KB of the row pair's memory, and the 8 bytes of results leave as one store.  The grid is sized to
// the chip and strides over the items two at a time: both items' loads are in flight before the first compare.
// Loads and stores carry no streaming hint: a pooling layer sits between a producer and a consumer, and activations
// of this size (a few hundred MB at most) are served from, and left in, the last-level cache.
// Same visiting order inside a window as the general kernel: (0,0), (0,1), (1,0), (1,1), strictly-greater wins.
//
// The windows are worked on as f32 values throughout: a bf16 cell is its 16 bits in the high half of a dword (the low
// half of a loaded dword shifted up, the high half masked), the winner's bits are the high half of the winning f32.
// The launch streams 1.25 bytes per input byte and has nothing else to hide behind, so the instruction count per
// window matters: with EVEN (ih == 2 * oh, no row left over at the bottom of a plane) row pairs follow one another
// through the whole tensor and an item's place needs one division, not two.
template <typename T>
struct PoolVec {
    static constexpr int VEC = 16 / (int)sizeof(T), NW = VEC / 2;
};
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

struct Pool2x2Item {
    size_t in_off, out_off;  // element offsets of the row pair's vector and of its outputs
};
template <bool EVEN>
__device__ __forceinline__ Pool2x2Item pool2x2_item(const PoolParams &p, uint32_t g, int vec) {
    Pool2x2Item it;
    if constexpr (EVEN) {
        const uint32_t orow = p.div_gpr.div(g);  // row pair, counted through all planes
        it.in_off = (size_t)(g + orow * p.div_gpr.d) * (size_t)vec;  // vectors before it: 2 * orow * gpr + gi
        it.out_off = (size_t)g * (size_t)(vec / 2);
    } else {
        uint32_t orow, gi, plane, ho;
        p.div_gpr.divmod(g, orow, gi);     // orow = plane * oh + ho
        p.div_oh.divmod(orow, plane, ho);
        it.in_off = ((size_t)plane * p.ih + (size_t)ho * 2) * p.iw + (size_t)gi * vec;
        it.out_off = (size_t)orow * p.ow + (size_t)gi * (vec / 2);
    }
    return it;
}

// window k of an item as four f32 values in visiting order, from the two rows' vectors
template <typename T>
__device__ __forceinline__ void pool2x2_window(const u32x4 &r0, const u32x4 &r1, int k, float (&f)[4]) {
    if constexpr (sizeof(T) == 4) {
        f[0] = __uint_as_float(r0[2 * k]); f[1] = __uint_as_float(r0[2 * k + 1]);
        f[2] = __uint_as_float(r1[2 * k]); f[3] = __uint_as_float(r1[2 * k + 1]);
    } else {
        f[0] = __uint_as_float(r0[k] << 16); f[1] = __uint_as_float(r0[k] & 0xFFFF0000u);
        f[2] = __uint_as_float(r1[k] << 16); f[3] = __uint_as_float(r1[k] & 0xFFFF0000u);
    }
}
// two bf16 values, each the high half of an f32, as one dword (lo in the low half)
__device__ __forceinline__ uint32_t pack_high_halves(float lo, float hi) {
    return __builtin_amdgcn_perm(__float_as_uint(hi), __float_as_uint(lo), 0x07060302u);
}

template <typename T, bool EVEN>
__global__ __launch_bounds__(kThreads) void max_pool2_2x2_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                  PoolParams p, uint32_t groups) {
    constexpr int VEC = PoolVec<T>::VEC, NW = PoolVec<T>::NW;
    const uint32_t stride = gridDim.x * kThreads;
    for (uint32_t g0 = blockIdx.x * kThreads + threadIdx.x; g0 < groups; g0 += 2 * stride) {
        const uint32_t g1 = g0 + stride;
        const bool two = g1 < groups;
        const Pool2x2Item it0 = pool2x2_item<EVEN>(p, g0, VEC), it1 = pool2x2_item<EVEN>(p, two ? g1 : g0, VEC);
        u32x4 r[2][2];
        r[0][0] = *(const u32x4 *)(x + it0.in_off);
        r[0][1] = *(const u32x4 *)(x + it0.in_off + p.iw);
        r[1][0] = *(const u32x4 *)(x + it1.in_off);
        r[1][1] = *(const u32x4 *)(x + it1.in_off + p.iw);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (u == 1 && !two) break;
            float mf[NW];
#pragma unroll
            for (int k = 0; k < NW; ++k) {
                float f[4];
                pool2x2_window<T>(r[u][0], r[u][1], k, f);
                mf[k] = f[0];
#pragma unroll
                for (int q = 1; q < 4; ++q)
                    if (f[q] > mf[k]) mf[k] = f[q];
            }
            u32x2 out;
            if constexpr (sizeof(T) == 4) {
                out[0] = __float_as_uint(mf[0]); out[1] = __float_as_uint(mf[1]);
            } else {
                out[0] = pack_high_halves(mf[0], mf[1]); out[1] = pack_high_halves(mf[2], mf[3]);
            }
            *(u32x2 *)(y + (u ? it1.out_off : it0.out_off)) = out;
        }
    }
}

template <typename T, bool EVEN>
__global__ __launch_bounds__(kThreads) void max_pool2_backward_2x2_kernel(T *__restrict__ dx, const T *__restrict__ dy,
                                                                           PoolParams p, uint32_t groups) {
    constexpr int VEC = PoolVec<T>::VEC, NW = PoolVec<T>::NW;
    const uint32_t stride = gridDim.x * kThreads;
    for (uint32_t g0 = blockIdx.x * kThreads + threadIdx.x; g0 < groups; g0 += 2 * stride) {
        const uint32_t g1 = g0 + stride;
        const bool two = g1 < groups;
        const Pool2x2Item it0 = pool2x2_item<EVEN>(p, g0, VEC), it1 = pool2x2_item<EVEN>(p, two ? g1 : g0, VEC);
        u32x4 r[2][2];
        u32x2 gy[2];
        r[0][0] = *(const u32x4 *)(dx + it0.in_off);
        r[0][1] = *(const u32x4 *)(dx + it0.in_off + p.iw);
        gy[0] = *(const u32x2 *)(dy + it0.out_off);
        r[1][0] = *(const u32x4 *)(dx + it1.in_off);
        r[1][1] = *(const u32x4 *)(dx + it1.in_off + p.iw);
        gy[1] = *(const u32x2 *)(dy + it1.out_off);
#pragma unroll
        for (int u = 0; u < 2; ++u) {
            if (u == 1 && !two) break;
            u32x4 o0, o1;
#pragma unroll
            for (int k = 0; k < NW; ++k) {
                float f[4];
                pool2x2_window<T>(r[u][0], r[u][1], k, f);
                // `0 + dy` in T, as the host's `+=` on the zeroed cell computes it.  c[q]: what the window's dwords
                // hold if cell q wins (f32: the cell itself; bf16: the pair of cells of its row)
                uint32_t gbits;
                if constexpr (sizeof(T) == 4) {
                    gbits = __float_as_uint(0.0f + __uint_as_float(gy[u][k]));
                } else {
                    const uint32_t gd = gy[u][k >> 1];
                    gbits = f32_to_bf16(0.0f + __uint_as_float((k & 1) ? (gd & 0xFFFF0000u) : (gd << 16)));
                }
                float mf = f[0];
                int am = 0;
#pragma unroll
                for (int q = 1; q < 4; ++q)
                    if (f[q] > mf) { mf = f[q]; am = q; }
                if constexpr (sizeof(T) == 4) {
                    o0[2 * k] = am == 0 ? gbits : 0u; o0[2 * k + 1] = am == 1 ? gbits : 0u;
                    o1[2 * k] = am == 2 ? gbits : 0u; o1[2 * k + 1] = am == 3 ? gbits : 0u;
                } else {
                    const uint32_t placed = (am & 1) ? (gbits << 16) : gbits;
                    o0[k] = am < 2 ? placed : 0u;
                    o1[k] = am < 2 ? 0u : placed;
                }
            }
            T *win = dx + (u ? it1.in_off : it0.in_off);
            *(u32x4 *)win = o0;
            *(u32x4 *)(win + p.iw) = o1;
        }
    }
}

template <typename T>
inline bool pool_2x2_fast(const PoolParams &p, const void *a, const void *b, size_t total) {
    constexpr int VEC = 16 / (int)sizeof(T);
    return p.h == 2 && p.w == 2 && p.sh == 2 && p.sw == 2 && p.iw % VEC == 0 && (((uintptr_t)a | (uintptr_t)b) & 15) == 0 &&
           total / (VEC / 2) < 0x7FFFFFFFull;
}
// blocks for a grid-stride pass over `groups` items, two per thread and trip.  Measured at 256 x 64 x 56 x 56: a grid
// of 16 workgroups per CU (several trips per thread) is 7 % slower than one that gives most threads a single trip,
// so the cap only bounds the grid for very large inputs
inline unsigned pool_2x2_grid(size_t groups) {
    const size_t want = (groups + 2 * kThreads - 1) / (2 * kThreads);
    const size_t cap = (size_t)(compute_units() > 0 ? compute_units() : 256) * 64;
    return (unsigned)std::max<size_t>(1, std::min(want, cap));
}

// Overlapping windows: the host visits windows of a plane one after another and each sees
// what the previous ones wrote, so a plane is walked by a single thread.
template <typename T>
__global__ __launch_bounds__(64) void max_pool2_backward_seq_kernel(T *__restrict__ dx, const T *__restrict__ dy,
                                                                     PoolParams p, size_t planes) {
    size_t plane = (size_t)blockIdx.x * 64 + threadIdx.x;
    if (plane >= planes) return;
    T *d = dx + plane * (size_t)p.ih * p.iw;
    const T *g = dy + plane * (size_t)p.oh * p.ow;
    for (int ho = 0; ho < p.oh; ++ho)
        for (int wo = 0; wo < p.ow; ++wo) {
            T *win = d + (size_t)ho * p.sh * p.iw + (size_t)wo * p.sw;
            float mf = Elem<T>::raw(win[0]);
            int am = 0;
            for (int fi = 0; fi < p.h; ++fi)
                for (int fj = 0; fj < p.w; ++fj) {
                    int off = fi * p.iw + fj;
                    float vf = Elem<T>::raw(win[off]);
                    if (vf > mf) { mf = vf; am = off; }
                    win[off] = Elem<T>::zero();
                }
            win[am] = Elem<T>::from_f32(0.0f + Elem<T>::raw(g[(size_t)ho * p.ow + wo]));
        }
}

int pool_check(const char *name, int64_t bc, int64_t ih, int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw,
               PoolParams &p) {
    if (bc < 0 || ih < 0 || iw < 0 || h < 1 || w < 1 || sh < 1 || sw < 1)
        return fail(AGH_EINVAL, "%s: invalid shape/options", name);
    if (h > ih || w > iw) return fail(AGH_EINVAL, "%s: window larger than the input", name);
    const int64_t lim = (int64_t)1 << 30;
    if (ih > lim || iw > lim || h > lim || w > lim || sh > lim || sw > lim || ih * iw > lim)
        return fail(AGH_ERANGE, "%s: dimension too large", name);
    p.ih = ih; p.iw = iw; p.h = h; p.w = w; p.sh = sh; p.sw = sw;
    p.oh = (ih - h) / sh + 1;
    p.ow = (iw - w) / sw + 1;
    p.div_ow = FastDiv((uint32_t)p.ow);
    p.div_oh = FastDiv((uint32_t)p.oh);
    return AGH_OK;
}

template <typename T>
int max_pool2_launch(const char *name, const void *x, void *y, int64_t bc, int64_t ih, int64_t iw, int64_t h,
                     int64_t w, int64_t sh, int64_t sw) {
    AGH_API_ENTER();
    PoolParams p;
    if (int rc = pool_check(name, bc, ih, iw, h, w, sh, sw, p)) return rc;
    const size_t total = (size_t)bc * p.oh * p.ow;
    if (total == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    size_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
    if (pool_2x2_fast<T>(p, x, y, total)) {
        constexpr int VEC = 16 / (int)sizeof(T);
        const size_t groups = total / (VEC / 2);
        p.div_gpr = FastDiv((uint32_t)(p.iw / VEC));
        if (p.ih == 2 * p.oh)
            hipLaunchKernelGGL((max_pool2_2x2_kernel<T, true>), dim3(pool_2x2_grid(groups)), dim3(kThreads),
                               0, stream(), (const T *)x, (T *)y, p, (uint32_t)groups);
        else
            hipLaunchKernelGGL((max_pool2_2x2_kernel<T, false>), dim3(pool_2x2_grid(groups)), dim3(kThreads),
                               0, stream(), (const T *)x, (T *)y, p, (uint32_t)groups);
        AGH_LAUNCH_CHECK(name);
        return AGH_OK;
    }
    hipLaunchKernelGGL(max_pool2_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(), (const T *)x,
                       (T *)y, p, total);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int max_pool2_backward_launch(const char *name, void *dx, const void *dy, int64_t bc, int64_t ih, int64_t iw,
                              int64_t h, int64_t w, int64_t sh, int64_t sw) {
    AGH_API_ENTER();
    PoolParams p;
    if (int rc = pool_check(name, bc, ih, iw, h, w, sh, sw, p)) return rc;
    const size_t total = (size_t)bc * p.oh * p.ow;
    if (total == 0) return AGH_OK;
    if (!dx || !dy) return fail(AGH_ENULL, "%s: null buffer", name);
    if (pool_2x2_fast<T>(p, dx, dy, total)) {
        constexpr int VEC = 16 / (int)sizeof(T);
        const size_t groups = total / (VEC / 2);
        p.div_gpr = FastDiv((uint32_t)(p.iw / VEC));
        if (p.ih == 2 * p.oh)
            hipLaunchKernelGGL((max_pool2_backward_2x2_kernel<T, true>), dim3(pool_2x2_grid(groups)),
                               dim3(kThreads), 0, stream(), (T *)dx, (const T *)dy, p, (uint32_t)groups);
        else
            hipLaunchKernelGGL((max_pool2_backward_2x2_kernel<T, false>), dim3(pool_2x2_grid(groups)),
                               dim3(kThreads), 0, stream(), (T *)dx, (const T *)dy, p, (uint32_t)groups);
    } else if (sh >= h && sw >= w) {
        size_t blocks = (total + kThreads - 1) / kThreads;
        if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
        hipLaunchKernelGGL(max_pool2_backward_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(),
                           (T *)dx, (const T *)dy, p, total);
    } else {
        size_t blocks = ((size_t)bc + 63) / 64;
        if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many planes", name);
        hipLaunchKernelGGL(max_pool2_backward_seq_kernel<T>, dim3((unsigned)blocks), dim3(64), 0, stream(), (T *)dx,
                           (const T *)dy, p, (size_t)bc);
    }
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// ------------------------------------------------------------------- relu ----
template <typename T>
__global__ __launch_bounds__(kThreads) void relu_kernel(const T *x, T *y, size_t n) {
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    size_t stride = (size_t)gridDim.x * kThreads;
    for (; i < n; i += stride) {
        T v = x[i];
        y[i] = Elem<T>::raw(v) >= 0.0f ? v : Elem<T>::zero();
    }
}
template <typename T>
__global__ __launch_bounds__(kThreads) void relu_backward_kernel(const T *x, const T *dy, T *dx, size_t n) {
    size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
    size_t stride = (size_t)gridDim.x * kThreads;
    for (; i < n; i += stride) dx[i] = Elem<T>::raw(x[i]) >= 0.0f ? dy[i] : Elem<T>::zero();
}

unsigned grid_for(size_t n) {
    size_t blocks = (n + kThreads - 1) / kThreads;
    size_t cap = (size_t)compute_units() * 32;
    if (cap == 0) cap = 8192;
    return (unsigned)(blocks < cap ? blocks : cap);
}

template <typename T>
int relu_launch(const char *name, const void *x, void *y, int64_t n) {
    AGH_API_ENTER();
    if (n < 0) return fail(AGH_EINVAL, "%s: negative length", name);
    if (n == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    hipLaunchKernelGGL(relu_kernel<T>, dim3(grid_for(n)), dim3(kThreads), 0, stream(), (const T *)x, (T *)y, (size_t)n);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}
template <typename T>
int relu_backward_launch(const char *name, const void *x, const void *dy, void *dx, int64_t n) {
    AGH_API_ENTER();
    if (n < 0) return fail(AGH_EINVAL, "%s: negative length", name);
    if (n == 0) return AGH_OK;
    if (!x || !dy || !dx) return fail(AGH_ENULL, "%s: null buffer", name);
    hipLaunchKernelGGL(relu_backward_kernel<T>, dim3(grid_for(n)), dim3(kThreads), 0, stream(), (const T *)x,
                       (const T *)dy, (T *)dx, (size_t)n);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}


// ------------------------------------------------------ relu fused with pool ----
// y = max_pool2(relu(x)) without the intermediate: the same element rule as relu_kernel and the same visiting
// order as max_pool2_kernel, applied to values that never reach memory.
template <typename T>
__device__ __forceinline__ T relu_of(T v) { return Elem<T>::raw(v) >= 0.0f ? v : Elem<T>::zero(); }

template <typename T>
__global__ __launch_bounds__(kThreads) void relu_max_pool2_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                                   PoolParams p, size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    const size_t osz = (size_t)p.oh * p.ow;
    const size_t plane = e / osz;
    const uint32_t rem = (uint32_t)(e - plane * osz);
    uint32_t ho, wo;
    p.div_ow.divmod(rem, ho, wo);
    const T *src = x + (plane * p.ih + (size_t)ho * p.sh) * p.iw + (size_t)wo * p.sw;
    T m = relu_of(src[0]);
    float mf = Elem<T>::raw(m);
    for (int fi = 0; fi < p.h; ++fi)
        for (int fj = 0; fj < p.w; ++fj) {
            T v = relu_of(src[(size_t)fi * p.iw + fj]);
            float vf = Elem<T>::raw(v);
            if (vf > mf) { m = v; mf = vf; }
        }
    y[e] = m;
}

// dx = relu_backward(x, max_pool2_backward(relu(x), dy)) for windows that do not overlap, one thread per
// INPUT cell: the cell finds the window that covers it, repeats that window's search for the first strict
// maximum of relu(x), and takes `0 + dy` if it is that maximum, 0 otherwise; a cell no window covers keeps
// relu(x), as the in-place pooling backward leaves it.  Then the relu rule of the cell's own x.  dx is
// [bs, c, ih, iw], or [bs, ih, iw, c] (`nhwc`): the matrix a convolution's weight gradient multiplies.
struct PoolReluBwdParams {
    PoolParams p;
    int c, nhwc;
    FastDiv div_iw, div_ih, div_c, div_sh, div_sw;
};

template <typename T>
__global__ __launch_bounds__(kThreads) void max_pool2_relu_backward_kernel(const T *__restrict__ x,
                                                                            const T *__restrict__ dy, T *__restrict__ dx,
                                                                            PoolReluBwdParams q, size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
    if (e >= total) return;
    const PoolParams &p = q.p;
    const size_t isz = (size_t)p.ih * p.iw;
    const uint32_t plane = (uint32_t)(e / isz);  // planes < 2^31 checked on the host
    const uint32_t rem = (uint32_t)(e - (size_t)plane * isz);
    uint32_t hy, wx, ho, rh, wo, rw;
    q.div_iw.divmod(rem, hy, wx);
    q.div_sh.divmod(hy, ho, rh);
    q.div_sw.divmod(wx, wo, rw);
    const T xv = x[e];
    T g = relu_of(xv);
    if (rh < (uint32_t)p.h && rw < (uint32_t)p.w && ho < (uint32_t)p.oh && wo < (uint32_t)p.ow) {
        const T *win = x + ((size_t)plane * p.ih + (size_t)ho * p.sh) * p.iw + (size_t)wo * p.sw;
        float mf = Elem<T>::raw(relu_of(win[0]));
        int am = 0;
        for (int fi = 0; fi < p.h; ++fi)
            for (int fj = 0; fj < p.w; ++fj) {
                const float vf = Elem<T>::raw(relu_of(win[(size_t)fi * p.iw + fj]));
                if (vf > mf) { mf = vf; am = fi * p.w + fj; }
            }
        const T gy = dy[((size_t)plane * p.oh + ho) * p.ow + wo];
        g = am == (int)(rh * p.w + rw) ? Elem<T>::from_f32(0.0f + Elem<T>::raw(gy)) : Elem<T>::zero();
    }
    const T out = Elem<T>::raw(xv) >= 0.0f ? g : Elem<T>::zero();
    size_t o = e;
    if (q.nhwc) {
        uint32_t b, ci;
        q.div_c.divmod(plane, b, ci);
        o = (((size_t)b * p.ih + hy) * p.iw + wx) * q.c + ci;
    }
    dx[o] = out;
}

// The same for 2x2 windows with stride 2 that tile the image exactly (the case the layer builder defaults to,
// layer.rs:535-539): one thread per WINDOW, so every cell is covered and the maximum is searched once.
template <typename T>
__global__ __launch_bounds__(kThreads) void max_pool2_relu_backward_2x2_kernel(const T *__restrict__ x,
                                                                                const T *__restrict__ dy,
                                                                                T *__restrict__ dx, PoolReluBwdParams q,
                                                                                size_t total) {
    size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;  // window index = index into dy
    if (e >= total) return;
    const PoolParams &p = q.p;
    const size_t osz = (size_t)p.oh * p.ow;
    const uint32_t plane = (uint32_t)(e / osz);
    const uint32_t rem = (uint32_t)(e - (size_t)plane * osz);
    uint32_t ho, wo;
    p.div_ow.divmod(rem, ho, wo);
    const size_t at = ((size_t)plane * p.ih + (size_t)ho * 2) * p.iw + (size_t)wo * 2;
    const T xv[4] = {x[at], x[at + 1], x[at + p.iw], x[at + p.iw + 1]};
    const T gy = dy[e];
    float mf = Elem<T>::raw(relu_of(xv[0]));
    int am = 0;
#pragma unroll
    for (int k = 1; k < 4; ++k) {
        const float vf = Elem<T>::raw(relu_of(xv[k]));
        if (vf > mf) { mf = vf; am = k; }
    }
    const T g = Elem<T>::from_f32(0.0f + Elem<T>::raw(gy));
    size_t o = at, ostep = 1, orow = (size_t)p.iw;
    if (q.nhwc) {
        uint32_t b, ci;
        q.div_c.divmod(plane, b, ci);
        o = (((size_t)b * p.ih + (size_t)ho * 2) * p.iw + (size_t)wo * 2) * q.c + ci;
        ostep = (size_t)q.c;
        orow = (size_t)p.iw * q.c;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const T cell = am == k ? g : Elem<T>::zero();
        dx[o + (k >> 1) * orow + (k & 1) * ostep] = Elem<T>::raw(xv[k]) >= 0.0f ? cell : Elem<T>::zero();
    }
}

template <typename T>
int relu_max_pool2_launch(const char *name, const void *x, void *y, int64_t bc, int64_t ih, int64_t iw, int64_t h,
                          int64_t w, int64_t sh, int64_t sw) {
    AGH_API_ENTER();
    PoolParams p;
    if (int rc = pool_check(name, bc, ih, iw, h, w, sh, sw, p)) return rc;
    const size_t total = (size_t)bc * p.oh * p.ow;
    if (total == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    size_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
    hipLaunchKernelGGL(relu_max_pool2_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(), (const T *)x,
                       (T *)y, p, total);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int max_pool2_relu_backward_launch(const char *name, const void *x, const void *dy, void *dx, int64_t bs, int64_t c,
                                   int64_t ih, int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw, int nhwc) {
    AGH_API_ENTER();
    if (bs < 0 || c < 0 || (c > 0 && bs > ((int64_t)1 << 31) / c))
        return fail(bs < 0 || c < 0 ? AGH_EINVAL : AGH_ERANGE, "%s: invalid batch/channel count", name);
    PoolReluBwdParams q;
    if (int rc = pool_check(name, bs * c, ih, iw, h, w, sh, sw, q.p)) return rc;
    if (sh < h || sw < w)
        return fail(AGH_EINVAL, "%s: overlapping windows (stride < size) need the separate backward calls", name);
    const size_t total = (size_t)bs * c * ih * iw;
    if (total == 0) return AGH_OK;
    if (!x || !dy || !dx) return fail(AGH_ENULL, "%s: null buffer", name);
    if (x == dx) return fail(AGH_EINVAL, "%s: dx must not alias x (every cell reads its whole window)", name);
    q.c = (int)c;
    q.nhwc = nhwc != 0;
    q.div_iw = FastDiv((uint32_t)iw);
    q.div_ih = FastDiv((uint32_t)ih);
    q.div_c = FastDiv((uint32_t)c);
    q.div_sh = FastDiv((uint32_t)sh);
    q.div_sw = FastDiv((uint32_t)sw);
    if (h == 2 && w == 2 && sh == 2 && sw == 2 && ih % 2 == 0 && iw % 2 == 0) {
        const size_t windows = total / 4;
        hipLaunchKernelGGL(max_pool2_relu_backward_2x2_kernel<T>, dim3((unsigned)((windows + kThreads - 1) / kThreads)),
                           dim3(kThreads), 0, stream(), (const T *)x, (const T *)dy, (T *)dx, q, windows);
        AGH_LAUNCH_CHECK(name);
        return AGH_OK;
    }
    size_t blocks = (total + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: too many elements", name);
    hipLaunchKernelGGL(max_pool2_relu_backward_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(),
                       (const T *)x, (const T *)dy, (T *)dx, q, total);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

}  // namespace

extern "C" {

int agh_memset(void *dst, int byte_value, size_t bytes) {
    AGH_API_ENTER();
    if (bytes == 0) return AGH_OK;
    if (!dst) return fail(AGH_ENULL, "agh_memset: null pointer");
    uint32_t b = (uint32_t)(byte_value & 0xFF);
    uint32_t pattern = b | (b << 8) | (b << 16) | (b << 24);
    hipLaunchKernelGGL(fill_bytes_kernel, dim3(grid_for(bytes / 16 + 16)), dim3(kThreads), 0, stream(),
                       (uint8_t *)dst, pattern, bytes);
    AGH_LAUNCH_CHECK("agh_memset");
    return AGH_OK;
}

#define AGH_CONV_ARGS int64_t bs, int64_t c, int64_t ih, int64_t iw, int64_t fh, int64_t fw, int64_t ph, int64_t pw, \
                      int64_t sh, int64_t sw, int64_t dh, int64_t dw
#define AGH_CONV_PASS bs, c, ih, iw, fh, fw, ph, pw, sh, sw, dh, dw

int agh_im2col_conv2_f32(const void *x, void *y, AGH_CONV_ARGS) {
    return im2col_launch<uint32_t>("agh_im2col_conv2_f32", x, y, AGH_CONV_PASS);
}
int agh_im2col_conv2_bf16(const void *x, void *y, AGH_CONV_ARGS) {
    return im2col_launch<uint16_t>("agh_im2col_conv2_bf16", x, y, AGH_CONV_PASS);
}
int agh_col2im_conv2_f32(const void *x, void *y, AGH_CONV_ARGS) {
    return col2im_launch<float>("agh_col2im_conv2_f32", x, y, AGH_CONV_PASS);
}
int agh_col2im_conv2_bf16(const void *x, void *y, AGH_CONV_ARGS) {
    return col2im_launch<uint16_t>("agh_col2im_conv2_bf16", x, y, AGH_CONV_PASS);
}
int agh_conv2_backward_input_f32(const void *dy, const void *w, void *dx, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                                 int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t sh, int64_t sw,
                                 int64_t dh, int64_t dw) {
    return conv2_backward_input_launch<float>("agh_conv2_backward_input_f32", dy, w, dx, bs, c, ih, iw, oc, fh, fw, ph, pw,
                                              sh, sw, dh, dw);
}
int agh_conv2_backward_input_bf16(const void *dy, const void *w, void *dx, int64_t bs, int64_t c, int64_t ih, int64_t iw,
                                  int64_t oc, int64_t fh, int64_t fw, int64_t ph, int64_t pw, int64_t sh, int64_t sw,
                                  int64_t dh, int64_t dw) {
    return conv2_backward_input_launch<uint16_t>("agh_conv2_backward_input_bf16", dy, w, dx, bs, c, ih, iw, oc, fh, fw, ph,
                                                 pw, sh, sw, dh, dw);
}

#define AGH_POOL_ARGS int64_t bc, int64_t ih, int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw
#define AGH_POOL_PASS bc, ih, iw, h, w, sh, sw

int agh_max_pool2_f32(const void *x, void *y, AGH_POOL_ARGS) {
    return max_pool2_launch<float>("agh_max_pool2_f32", x, y, AGH_POOL_PASS);
}
int agh_max_pool2_bf16(const void *x, void *y, AGH_POOL_ARGS) {
    return max_pool2_launch<uint16_t>("agh_max_pool2_bf16", x, y, AGH_POOL_PASS);
}
int agh_max_pool2_backward_f32(void *dx, const void *dy, AGH_POOL_ARGS) {
    return max_pool2_backward_launch<float>("agh_max_pool2_backward_f32", dx, dy, AGH_POOL_PASS);
}
int agh_max_pool2_backward_bf16(void *dx, const void *dy, AGH_POOL_ARGS) {
    return max_pool2_backward_launch<uint16_t>("agh_max_pool2_backward_bf16", dx, dy, AGH_POOL_PASS);
}

int agh_relu_max_pool2_f32(const void *x, void *y, AGH_POOL_ARGS) {
    return relu_max_pool2_launch<float>("agh_relu_max_pool2_f32", x, y, AGH_POOL_PASS);
}
int agh_relu_max_pool2_bf16(const void *x, void *y, AGH_POOL_ARGS) {
    return relu_max_pool2_launch<uint16_t>("agh_relu_max_pool2_bf16", x, y, AGH_POOL_PASS);
}
int agh_max_pool2_relu_backward_f32(const void *x, const void *dy, void *dx, int64_t bs, int64_t c, int64_t ih,
                                    int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw, int nhwc) {
    return max_pool2_relu_backward_launch<float>("agh_max_pool2_relu_backward_f32", x, dy, dx, bs, c, ih, iw, h, w, sh,
                                                 sw, nhwc);
}
int agh_max_pool2_relu_backward_bf16(const void *x, const void *dy, void *dx, int64_t bs, int64_t c, int64_t ih,
                                     int64_t iw, int64_t h, int64_t w, int64_t sh, int64_t sw, int nhwc) {
    return max_pool2_relu_backward_launch<uint16_t>("agh_max_pool2_relu_backward_bf16", x, dy, dx, bs, c, ih, iw, h, w,
                                                    sh, sw, nhwc);
}
int agh_relu_f32(const void *x, void *y, int64_t n) { return relu_launch<float>("agh_relu_f32", x, y, n); }
int agh_relu_bf16(const void *x, void *y, int64_t n) { return relu_launch<uint16_t>("agh_relu_bf16", x, y, n); }
int agh_relu_backward_f32(const void *x, const void *dy, void *dx, int64_t n) {
    return relu_backward_launch<float>("agh_relu_backward_f32", x, dy, dx, n);
}
int agh_relu_backward_bf16(const void *x, const void *dy, void *dx, int64_t n) {
    return relu_backward_launch<uint16_t>("agh_relu_backward_bf16", x, dy, dx, n);
}

}  // extern "C"

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

    for (int e = threadIdx.x; e < taps * p.ocpad; e += blockDim.x) {
        const int tap = e / p.ocpad, o = e - tap * p.ocpad;
        ws[e] = o < p.oc ? Elem<T>::to_f32(w[(size_t)o * taps + tap]) : 0.0f;
    }
    const T *xb = x + (size_t)b0 * img_sz;
    for (int e = threadIdx.x; e < nimg * img_sz; e += blockDim.x) xs[e] = Elem<T>::to_f32(xb[e]);
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

}  // extern "C"

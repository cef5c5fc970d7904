/*
 * CPU restatement of autograph's HOST path for the dense-contraction hot path.
 *
 * THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE.  Only tests/, the smoke check and
 * the bench's cpu_baseline leg may load it; the shipped library never links it and
 * never falls back to it.
 *
 * Every function cites the reference file:line it restates (paths relative to the
 * reference checkout).  Arithmetic that lives in third-party crates absent from the
 * reference tree is restated from their published algorithms:
 *   - half >= 2.1 (Cargo.toml:55)  bf16 <-> f32 conversion (round-to-nearest-even,
 *     NaN keeps the top mantissa bits and gets the quiet bit)
 *   - ndarray >= 0.15.6 linalg::general_mat_mul generic fallback (left fold in T)
 *   - matrixmultiply sgemm: only its result up to rounding order is restated
 *     (blocked f32 accumulate); its exact rounding order is "parity unpinned".
 *
 * What pins each function is listed in tests/test_oracle.py.
 */
#include <stdint.h>
#include <stddef.h>
#include <stdlib.h>
#include <string.h>
#include <math.h>
#ifdef _OPENMP
#include <omp.h>
#endif

typedef uint16_t bf16_t;
typedef int64_t i64;

/* ---------------------------------------------------------------- bf16 ---- */

/* half::bf16::from_f32 (crate `half`, bfloat/convert.rs): RNE, NaN -> (x>>16)|0x40. */
static inline bf16_t f32_to_bf16(float v) {
    uint32_t x;
    memcpy(&x, &v, 4);
    if ((x & 0x7FFFFFFFu) > 0x7F800000u) return (bf16_t)((x >> 16) | 0x0040u);
    const uint32_t round_bit = 0x00008000u;
    if ((x & round_bit) != 0 && (x & (3 * round_bit - 1)) != 0) return (bf16_t)((x >> 16) + 1);
    return (bf16_t)(x >> 16);
}

/* half::bf16::to_f32: NaN gets the quiet bit, everything else is a plain shift. */
static inline float bf16_to_f32(bf16_t h) {
    uint32_t x;
    if ((h & 0x7FFFu) > 0x7F80u) x = ((uint32_t)(h | 0x0040u)) << 16;
    else x = ((uint32_t)h) << 16;
    float f;
    memcpy(&f, &x, 4);
    return f;
}

uint16_t orc_f32_to_bf16(float v) { return f32_to_bf16(v); }
float orc_bf16_to_f32(uint16_t h) { return bf16_to_f32(h); }

void orc_f32_to_bf16_n(const float *x, uint16_t *y, i64 n) {
    for (i64 i = 0; i < n; ++i) y[i] = f32_to_bf16(x[i]);
}
void orc_bf16_to_f32_n(const uint16_t *x, float *y, i64 n) {
    for (i64 i = 0; i < n; ++i) y[i] = bf16_to_f32(x[i]);
}

/* bf16 `a + b` / `a * b` as the half crate does them: widen, operate in f32, round. */
static inline bf16_t bf16_add(bf16_t a, bf16_t b) { return f32_to_bf16(bf16_to_f32(a) + bf16_to_f32(b)); }
static inline bf16_t bf16_mul(bf16_t a, bf16_t b) { return f32_to_bf16(bf16_to_f32(a) * bf16_to_f32(b)); }

/* ------------------------------------------------------- shape formulas ---- */

/* Im2ColConv2Options::output_shape, src/ops.rs:28-40:  o = (i + 2p - d(f-1) - 1)/s + 1 */
i64 orc_conv_out(i64 i, i64 f, i64 p, i64 s, i64 d) { return (i + 2 * p - d * (f - 1) - 1) / s + 1; }
/* Col2ImConv2Options::output_shape, src/ops.rs:67-79: o = (i-1)s + d(f-1) + 1 - 2p */
i64 orc_col2im_out(i64 i, i64 f, i64 p, i64 s, i64 d) { return (i - 1) * s + d * (f - 1) + 1 - 2 * p; }
/* MaxPool2Options::output_shape, src/ops.rs:93-103: o = (i - x)/s + 1 */
i64 orc_pool_out(i64 i, i64 x, i64 s) { return (i - x) / s + 1; }

/* --------------------------------------------------------------- im2col ---- */

/* src/tensor/ops.rs:741-813 (host Im2ColConv2 for ArrayBase): pure gather,
 * y[(b,ho,wo),(ci,fi,fj)] = x[b,ci,-ph+fi*dh+sh*ho, -pw+fj*dw+sw*wo] or T::default().
 * Batch items are dealt round-robin to threads (src/tensor/parallel.rs:33-60). */
#define DEF_IM2COL(NAME, T)                                                                      \
    void NAME(const T *x, T *y, i64 bs, i64 c, i64 ih, i64 iw, i64 fh, i64 fw, i64 ph, i64 pw,    \
              i64 sh, i64 sw, i64 dh, i64 dw) {                                                   \
        const i64 oh = orc_conv_out(ih, fh, ph, sh, dh), ow = orc_conv_out(iw, fw, pw, sw, dw);   \
        _Pragma("omp parallel for schedule(static, 1)") for (i64 b = 0; b < bs; ++b) {            \
            const T *xb = x + b * c * ih * iw;                                                    \
            T *yb = y + b * oh * ow * c * fh * fw;                                                \
            for (i64 hid = 0; hid < oh; ++hid)                                                    \
                for (i64 wid = 0; wid < ow; ++wid)                                                \
                    for (i64 cid = 0; cid < c; ++cid)                                             \
                        for (i64 fi = 0; fi < fh; ++fi)                                           \
                            for (i64 fj = 0; fj < fw; ++fj) {                                     \
                                i64 hidx = -ph + fi * dh + sh * hid;                              \
                                i64 widx = -pw + fj * dw + sw * wid;                              \
                                T v = 0;                                                          \
                                if (hidx >= 0 && hidx < ih && widx >= 0 && widx < iw)             \
                                    v = xb[(cid * ih + hidx) * iw + widx];                        \
                                yb[(((hid * ow + wid) * c + cid) * fh + fi) * fw + fj] = v;       \
                            }                                                                     \
        }                                                                                         \
    }
DEF_IM2COL(orc_im2col_conv2_b32, uint32_t)
DEF_IM2COL(orc_im2col_conv2_b16, uint16_t)

/* --------------------------------------------------------------- col2im ---- */

/* src/tensor/ops.rs:891-964 (host Col2ImConv2): output starts at +0 (Array::zeros,
 * :911) and every `+=` is done in T, in loop order cid, hid, wid, fi, fj (:935-939).
 * `ih,iw` is the patch grid (options.shape). */
void orc_col2im_conv2_f32(const float *x, float *y, i64 bs, i64 c, i64 ih, i64 iw, i64 fh, i64 fw,
                          i64 ph, i64 pw, i64 sh, i64 sw, i64 dh, i64 dw) {
    const i64 oh = orc_col2im_out(ih, fh, ph, sh, dh), ow = orc_col2im_out(iw, fw, pw, sw, dw);
#pragma omp parallel for schedule(static, 1)
    for (i64 b = 0; b < bs; ++b) {
        const float *xb = x + b * ih * iw * c * fh * fw;
        float *yb = y + b * c * oh * ow;
        for (i64 i = 0; i < c * oh * ow; ++i) yb[i] = 0.0f;
        for (i64 cid = 0; cid < c; ++cid)
            for (i64 hid = 0; hid < ih; ++hid)
                for (i64 wid = 0; wid < iw; ++wid)
                    for (i64 fi = 0; fi < fh; ++fi)
                        for (i64 fj = 0; fj < fw; ++fj) {
                            i64 hidy = -ph + fi * dh + sh * hid;
                            i64 widy = -pw + fj * dw + sw * wid;
                            if (hidy >= 0 && hidy < oh && widy >= 0 && widy < ow) {
                                yb[(cid * oh + hidy) * ow + widy] +=
                                    xb[(((hid * iw + wid) * c + cid) * fh + fi) * fw + fj];
                            }
                        }
    }
}

void orc_col2im_conv2_bf16(const bf16_t *x, bf16_t *y, i64 bs, i64 c, i64 ih, i64 iw, i64 fh, i64 fw,
                           i64 ph, i64 pw, i64 sh, i64 sw, i64 dh, i64 dw) {
    const i64 oh = orc_col2im_out(ih, fh, ph, sh, dh), ow = orc_col2im_out(iw, fw, pw, sw, dw);
#pragma omp parallel for schedule(static, 1)
    for (i64 b = 0; b < bs; ++b) {
        const bf16_t *xb = x + b * ih * iw * c * fh * fw;
        bf16_t *yb = y + b * c * oh * ow;
        for (i64 i = 0; i < c * oh * ow; ++i) yb[i] = 0;
        for (i64 cid = 0; cid < c; ++cid)
            for (i64 hid = 0; hid < ih; ++hid)
                for (i64 wid = 0; wid < iw; ++wid)
                    for (i64 fi = 0; fi < fh; ++fi)
                        for (i64 fj = 0; fj < fw; ++fj) {
                            i64 hidy = -ph + fi * dh + sh * hid;
                            i64 widy = -pw + fj * dw + sw * wid;
                            if (hidy >= 0 && hidy < oh && widy >= 0 && widy < ow) {
                                bf16_t *o = &yb[(cid * oh + hidy) * ow + widy];
                                *o = bf16_add(*o, xb[(((hid * iw + wid) * c + cid) * fh + fi) * fw + fj]);
                            }
                        }
    }
}

/* ------------------------------------------------------------- max pool ---- */

/* src/tensor/ops.rs:1040-1088: m = first element; a later element replaces it only
 * when `x > m` in T (strict; NaN never wins, a leading NaN sticks). The result is a
 * bit copy of one input element.  `bc` = bs*c planes. */
void orc_max_pool2_f32(const float *x, float *y, i64 bc, i64 ih, i64 iw, i64 h, i64 w, i64 sh, i64 sw) {
    const i64 oh = orc_pool_out(ih, h, sh), ow = orc_pool_out(iw, w, sw);
#pragma omp parallel for schedule(static)
    for (i64 p = 0; p < bc; ++p)
        for (i64 hid = 0; hid < oh; ++hid)
            for (i64 wid = 0; wid < ow; ++wid) {
                float m = 0.0f;
                for (i64 fi = 0; fi < h; ++fi)
                    for (i64 fj = 0; fj < w; ++fj) {
                        float v = x[(p * ih + fi + sh * hid) * iw + fj + sw * wid];
                        if ((fi == 0 && fj == 0) || v > m) m = v;
                    }
                y[(p * oh + hid) * ow + wid] = m;
            }
}

void orc_max_pool2_bf16(const bf16_t *x, bf16_t *y, i64 bc, i64 ih, i64 iw, i64 h, i64 w, i64 sh, i64 sw) {
    const i64 oh = orc_pool_out(ih, h, sh), ow = orc_pool_out(iw, w, sw);
#pragma omp parallel for schedule(static)
    for (i64 p = 0; p < bc; ++p)
        for (i64 hid = 0; hid < oh; ++hid)
            for (i64 wid = 0; wid < ow; ++wid) {
                bf16_t m = 0;
                for (i64 fi = 0; fi < h; ++fi)
                    for (i64 fj = 0; fj < w; ++fj) {
                        bf16_t v = x[(p * ih + fi + sh * hid) * iw + fj + sw * wid];
                        /* half's PartialOrd for bf16 orders exactly like the widened f32 values */
                        if ((fi == 0 && fj == 0) || bf16_to_f32(v) > bf16_to_f32(m)) m = v;
                    }
                y[(p * oh + hid) * ow + wid] = m;
            }
}

/* src/tensor/ops.rs:1144-1207: dx enters holding x.  Windows are visited in
 * (hid, wid) order inside a plane; each window finds its first strict max among the
 * CURRENT dx values while zeroing every cell it visits, then does
 * `dx[argmax] += dy` in T.  Cells no window covers keep their x value. */
void orc_max_pool2_backward_f32(float *dx, const float *dy, i64 bc, i64 ih, i64 iw, i64 h, i64 w,
                                i64 sh, i64 sw) {
    const i64 oh = orc_pool_out(ih, h, sh), ow = orc_pool_out(iw, w, sw);
#pragma omp parallel for schedule(static)
    for (i64 p = 0; p < bc; ++p)
        for (i64 hid = 0; hid < oh; ++hid)
            for (i64 wid = 0; wid < ow; ++wid) {
                float m = 0.0f;
                i64 hm = 0, wm = 0;
                for (i64 fi = 0; fi < h; ++fi)
                    for (i64 fj = 0; fj < w; ++fj) {
                        i64 hidx = fi + sh * hid, widx = fj + sw * wid;
                        float *d = &dx[(p * ih + hidx) * iw + widx];
                        if ((fi == 0 && fj == 0) || *d > m) { m = *d; hm = hidx; wm = widx; }
                        *d = 0.0f;
                    }
                dx[(p * ih + hm) * iw + wm] += dy[(p * oh + hid) * ow + wid];
            }
}

void orc_max_pool2_backward_bf16(bf16_t *dx, const bf16_t *dy, i64 bc, i64 ih, i64 iw, i64 h, i64 w,
                                 i64 sh, i64 sw) {
    const i64 oh = orc_pool_out(ih, h, sh), ow = orc_pool_out(iw, w, sw);
#pragma omp parallel for schedule(static)
    for (i64 p = 0; p < bc; ++p)
        for (i64 hid = 0; hid < oh; ++hid)
            for (i64 wid = 0; wid < ow; ++wid) {
                bf16_t m = 0;
                i64 hm = 0, wm = 0;
                for (i64 fi = 0; fi < h; ++fi)
                    for (i64 fj = 0; fj < w; ++fj) {
                        i64 hidx = fi + sh * hid, widx = fj + sw * wid;
                        bf16_t *d = &dx[(p * ih + hidx) * iw + widx];
                        if ((fi == 0 && fj == 0) || bf16_to_f32(*d) > bf16_to_f32(m)) { m = *d; hm = hidx; wm = widx; }
                        *d = 0;
                    }
                bf16_t *o = &dx[(p * ih + hm) * iw + wm];
                *o = bf16_add(*o, dy[(p * oh + hid) * ow + wid]);
            }
}

/* ----------------------------------------------------------- relu, bias ---- */

/* src/learn/neural_network/layer.rs:1526-1540: x >= 0 ? x : 0  (so -0 stays -0, NaN -> 0). */
void orc_relu_f32(const float *x, float *y, i64 n) {
    for (i64 i = 0; i < n; ++i) y[i] = x[i] >= 0.0f ? x[i] : 0.0f;
}
void orc_relu_bf16(const bf16_t *x, bf16_t *y, i64 n) {
    for (i64 i = 0; i < n; ++i) y[i] = bf16_to_f32(x[i]) >= 0.0f ? x[i] : 0;
}
void orc_relu_backward_f32(const float *x, const float *dy, float *dx, i64 n) {
    for (i64 i = 0; i < n; ++i) dx[i] = x[i] >= 0.0f ? dy[i] : 0.0f;
}
void orc_relu_backward_bf16(const bf16_t *x, const bf16_t *dy, bf16_t *dx, i64 n) {
    for (i64 i = 0; i < n; ++i) dx[i] = bf16_to_f32(x[i]) >= 0.0f ? dy[i] : 0;
}

/* Dense bias: autograd.rs:571-599 -> scaled_add(1, bias broadcast over rows)
 * (src/tensor/ops.rs:192-204, BinaryOp::Add y = alpha*x + y in T, :1319-1330). */
void orc_bias_add_rows_f32(float *y, const float *bias, i64 m, i64 n) {
    for (i64 i = 0; i < m; ++i)
        for (i64 j = 0; j < n; ++j) y[i * n + j] = 1.0f * bias[j] + y[i * n + j];
}
void orc_bias_add_rows_bf16(bf16_t *y, const bf16_t *bias, i64 m, i64 n) {
    const bf16_t one = 0x3F80;
    for (i64 i = 0; i < m; ++i)
        for (i64 j = 0; j < n; ++j) y[i * n + j] = bf16_add(bf16_mul(one, bias[j]), y[i * n + j]);
}

/* ----------------------------------------------------------------- gemm ---- */

/* Strided C = alpha*A*B + beta*C with element offsets and signed element strides,
 * the tuple `gemm()` extracts at src/tensor/linalg.rs:281-299.  beta == 0 never
 * reads C (linalg.rs:215-218). */

/* f64-accumulated checker for f32 inputs (the quantity every f32 result is compared
 * with under the 1e-5*sqrt(K) rule). */
void orc_gemm_f32_f64acc(i64 m, i64 k, i64 n, double alpha, const float *a, i64 off_a, i64 rsa, i64 csa,
                         const float *b, i64 off_b, i64 rsb, i64 csb, double beta, const float *c_in,
                         double *c_out /* dense row-major m*n */, i64 off_c, i64 rsc, i64 csc) {
#pragma omp parallel for schedule(static)
    for (i64 i = 0; i < m; ++i)
        for (i64 j = 0; j < n; ++j) {
            double s = 0.0;
            for (i64 x = 0; x < k; ++x)
                s += (double)a[off_a + i * rsa + x * csa] * (double)b[off_b + x * rsb + j * csb];
            double r = alpha * s;
            if (beta != 0.0) r += beta * (double)c_in[off_c + i * rsc + j * csc];
            c_out[i * n + j] = r;
        }
}

/* Same for bf16 inputs: products of two bf16 values are exact in f64. */
void orc_gemm_bf16_f64acc(i64 m, i64 k, i64 n, double alpha, const bf16_t *a, i64 off_a, i64 rsa, i64 csa,
                          const bf16_t *b, i64 off_b, i64 rsb, i64 csb, double beta, const bf16_t *c_in,
                          double *c_out, i64 off_c, i64 rsc, i64 csc) {
#pragma omp parallel for schedule(static)
    for (i64 i = 0; i < m; ++i)
        for (i64 j = 0; j < n; ++j) {
            double s = 0.0;
            for (i64 x = 0; x < k; ++x)
                s += (double)bf16_to_f32(a[off_a + i * rsa + x * csa]) *
                     (double)bf16_to_f32(b[off_b + x * rsb + j * csb]);
            double r = alpha * s;
            if (beta != 0.0) r += beta * (double)bf16_to_f32(c_in[off_c + i * rsc + j * csc]);
            c_out[i * n + j] = r;
        }
}

/* The reference DEVICE kernel's numerics for bf16 (linalg.rs:244, :127, :217):
 * f32 accumulator over k ascending, one final cast.  Used as the "f32-accumulated
 * reference" for bf16 outputs. */
void orc_gemm_bf16_f32acc(i64 m, i64 k, i64 n, float alpha, const bf16_t *a, i64 off_a, i64 rsa, i64 csa,
                          const bf16_t *b, i64 off_b, i64 rsb, i64 csb, float beta, bf16_t *c, i64 off_c,
                          i64 rsc, i64 csc) {
#pragma omp parallel for schedule(static)
    for (i64 i = 0; i < m; ++i)
        for (i64 j = 0; j < n; ++j) {
            float s = 0.0f;
            for (i64 x = 0; x < k; ++x) {
                /* built with -ffp-contract=off: multiply, then add, as c += a*b does without FMA */
                s += bf16_to_f32(a[off_a + i * rsa + x * csa]) * bf16_to_f32(b[off_b + x * rsb + j * csb]);
            }
            bf16_t *o = &c[off_c + i * rsc + j * csc];
            if (beta == 0.0f) *o = f32_to_bf16(alpha * s);
            else {
                *o = f32_to_bf16(alpha * s + beta * bf16_to_f32(*o));
            }
        }
}

/* HOST bf16 dot (linalg.rs:394-401 -> ndarray general_mat_mul generic fallback):
 * single thread, `c = c*beta + alpha * fold(0, s + a*b)` with every multiply and add
 * rounded to bf16.  Timing baseline only; its exact loop order is parity unpinned. */
void orc_gemm_bf16_hostfold(i64 m, i64 k, i64 n, const bf16_t *a, i64 off_a, i64 rsa, i64 csa,
                            const bf16_t *b, i64 off_b, i64 rsb, i64 csb, bf16_t *c /* row-major m*n */) {
    const bf16_t one = 0x3F80, zero = 0;
    for (i64 i = 0; i < m; ++i)
        for (i64 j = 0; j < n; ++j) {
            bf16_t s = 0;
            for (i64 x = 0; x < k; ++x)
                s = bf16_add(s, bf16_mul(a[off_a + i * rsa + x * csa], b[off_b + x * rsb + j * csb]));
            c[i * n + j] = bf16_add(bf16_mul(zero, zero), bf16_mul(one, s));
        }
}

/* HOST f32 dot (linalg.rs:394-401 -> matrixmultiply::sgemm, feature
 * matrixmultiply-threading, Cargo.toml:59-63): a packed, cache-blocked sgemm with the
 * strides folded into packing, run on at most 4 threads as matrixmultiply does.
 * Blocking constants follow matrixmultiply's published ones (MC=64, KC=256, NC=1024,
 * 8x8 micro-kernel on FMA hardware).  Rounding order: parity unpinned. */
#define MR 8
#define NR 8
#define KC 256
#define MC 64
#define NC 1024
typedef float v8f __attribute__((vector_size(32)));

static void sgemm_pack_a(float *dst, const float *a, i64 rsa, i64 csa, i64 mc, i64 kc) {
    for (i64 i0 = 0; i0 < mc; i0 += MR)
        for (i64 p = 0; p < kc; ++p)
            for (i64 i = 0; i < MR; ++i) *dst++ = (i0 + i < mc) ? a[(i0 + i) * rsa + p * csa] : 0.0f;
}
static void sgemm_pack_b(float *dst, const float *b, i64 rsb, i64 csb, i64 kc, i64 nc) {
    for (i64 j0 = 0; j0 < nc; j0 += NR)
        for (i64 p = 0; p < kc; ++p)
            for (i64 j = 0; j < NR; ++j) *dst++ = (j0 + j < nc) ? b[p * rsb + (j0 + j) * csb] : 0.0f;
}
__attribute__((optimize("fp-contract=fast")))
static void sgemm_ukernel(i64 kc, const float *pa, const float *pb, float acc[MR][NR]) {
    v8f r[MR];
    for (int i = 0; i < MR; ++i) r[i] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
    for (i64 p = 0; p < kc; ++p) {
        v8f bv;
        memcpy(&bv, pb + p * NR, 32);
        for (int i = 0; i < MR; ++i) r[i] += pa[p * MR + i] * bv;
    }
    for (int i = 0; i < MR; ++i) memcpy(acc[i], &r[i], 32);
}

void orc_gemm_f32_host(i64 m, i64 k, i64 n, float alpha, const float *a, i64 off_a, i64 rsa, i64 csa,
                       const float *b, i64 off_b, i64 rsb, i64 csb, float beta, float *c, i64 off_c,
                       i64 rsc, i64 csc, int threads) {
    a += off_a; b += off_b; c += off_c;
    if (threads < 1) threads = 1;
    if (threads > 4) threads = 4;
    if (k == 0 || alpha == 0.0f) {
        for (i64 i = 0; i < m; ++i)
            for (i64 j = 0; j < n; ++j) {
                float *o = &c[i * rsc + j * csc];
                *o = beta == 0.0f ? 0.0f : beta * *o;
            }
        return;
    }
    float *pb = (float *)aligned_alloc(64, sizeof(float) * KC * (NC + NR));
    float *pa_all = (float *)aligned_alloc(64, sizeof(float) * (size_t)threads * KC * (MC + MR));
    for (i64 jc = 0; jc < n; jc += NC) {
        i64 nc = n - jc < NC ? n - jc : NC;
        for (i64 pc = 0; pc < k; pc += KC) {
            i64 kc = k - pc < KC ? k - pc : KC;
            sgemm_pack_b(pb, b + pc * rsb + jc * csb, rsb, csb, kc, nc);
            const int first = pc == 0;
            i64 nblk = (m + MC - 1) / MC;
#pragma omp parallel for schedule(static, 1) num_threads(threads)
            for (i64 ib = 0; ib < nblk; ++ib) {
                i64 ic = ib * MC;
                i64 mc = m - ic < MC ? m - ic : MC;
                int tid = 0;
#ifdef _OPENMP
                tid = omp_get_thread_num();
#endif
                float *pa = pa_all + (size_t)tid * KC * (MC + MR);
                sgemm_pack_a(pa, a + ic * rsa + pc * csa, rsa, csa, mc, kc);
                for (i64 jr = 0; jr < nc; jr += NR)
                    for (i64 ir = 0; ir < mc; ir += MR) {
                        float acc[MR][NR];
                        sgemm_ukernel(kc, pa + ir * kc, pb + jr * kc, acc);
                        for (i64 i = 0; i < MR && ir + i < mc; ++i)
                            for (i64 j = 0; j < NR && jr + j < nc; ++j) {
                                float *o = &c[(ic + ir + i) * rsc + (jc + jr + j) * csc];
                                float v = alpha * acc[i][j];
                                if (first) *o = beta == 0.0f ? v : v + beta * *o;
                                else *o += v;
                            }
                    }
            }
        }
    }
    free(pb);
    free(pa_all);
}

/* ------------------------------------------------------ conv2 reference ---- */

/* The 7-deep loop the reference's own tests use as the convolution definition
 * (tests/integration_tests.rs:1127-1174), accumulating in f64 here so it can serve as
 * the checker for both f32 and (after widening) bf16 inputs. */
void orc_conv2_naive_f64(const float *x, const float *w, double *y, i64 bs, i64 ic, i64 ih, i64 iw, i64 oc,
                         i64 fh, i64 fw, i64 ph, i64 pw, i64 sh, i64 sw, i64 dh, i64 dw) {
    const i64 oh = orc_conv_out(ih, fh, ph, sh, dh), ow = orc_conv_out(iw, fw, pw, sw, dw);
#pragma omp parallel for schedule(static)
    for (i64 bid = 0; bid < bs; ++bid)
        for (i64 cy = 0; cy < oc; ++cy)
            for (i64 hy = 0; hy < oh; ++hy)
                for (i64 wy = 0; wy < ow; ++wy) {
                    double s = 0.0;
                    for (i64 cx = 0; cx < ic; ++cx)
                        for (i64 fi = 0; fi < fh; ++fi) {
                            i64 hx = -ph + sh * hy + dh * fi;
                            if (hx < 0 || hx >= ih) continue;
                            for (i64 fj = 0; fj < fw; ++fj) {
                                i64 wx = -pw + sw * wy + dw * fj;
                                if (wx < 0 || wx >= iw) continue;
                                s += (double)x[((bid * ic + cx) * ih + hx) * iw + wx] *
                                     (double)w[((cy * ic + cx) * fh + fi) * fw + fj];
                            }
                        }
                    y[((bid * oc + cy) * oh + hy) * ow + wy] = s;
                }
}

/* ------------------------------------------------- LeNet5 f32 host path ---- */

/* Layer list: benches/neural-network-benches/src/autograph_backend.rs:88-162
 * (conv 1->6 5x5, relu, pool 2x2, conv 6->16 5x5, relu, pool 2x2, flatten,
 * dense 256->128, relu, dense 128->84, relu, dense 84->10 + bias).
 * Convolutions run as conv2_im2col does (layer.rs:950-1005): im2col, dot with the
 * [oc, ic*fh*fw] weight matrix transposed, NHWC -> NCHW copy.  (The reference host
 * runs its f32 convs through conv_direct instead; same sums in another order.)
 * Scratch is allocated per call, as the reference allocates every intermediate. */
static void conv_im2col_f32(const float *x, const float *w, float *y, i64 bs, i64 ic, i64 ih, i64 iw,
                            i64 oc, i64 fh, i64 fw, int threads) {
    const i64 oh = ih - fh + 1, ow = iw - fw + 1, rows = bs * oh * ow, kk = ic * fh * fw;
    float *cols = (float *)malloc(sizeof(float) * rows * kk);
    float *out = (float *)malloc(sizeof(float) * rows * oc);
    orc_im2col_conv2_b32((const uint32_t *)x, (uint32_t *)cols, bs, ic, ih, iw, fh, fw, 0, 0, 1, 1, 1, 1);
    orc_gemm_f32_host(rows, kk, oc, 1.0f, cols, 0, kk, 1, w, 0, 1, kk, 0.0f, out, 0, oc, 1, threads);
#pragma omp parallel for schedule(static)
    for (i64 b = 0; b < bs; ++b)
        for (i64 o = 0; o < oc; ++o)
            for (i64 p = 0; p < oh * ow; ++p) y[(b * oc + o) * oh * ow + p] = out[(b * oh * ow + p) * oc + o];
    free(cols);
    free(out);
}

/* Host f32 Conv2 for default options as the reference runs it: a direct convolution
 * (layer.rs:936-943 -> layer/conv_direct.rs:23-83, :760-946), images dealt to threads
 * (rayon broadcast over the batch), SIMD along the output row.  Restated as an axpy of one
 * filter tap over one output plane at a time; summation order is (ic, fi, fj) like
 * conv_direct's, FMA contraction allowed as with its `mul_add` under +fma. */
__attribute__((optimize("fp-contract=fast")))
void orc_conv2_direct_f32(const float *x, const float *w, float *y, i64 bs, i64 ic, i64 ih, i64 iw, i64 oc, i64 fh,
                          i64 fw) {
    const i64 oh = ih - fh + 1, ow = iw - fw + 1;
#pragma omp parallel for schedule(static, 1)
    for (i64 b = 0; b < bs; ++b)
        for (i64 o = 0; o < oc; ++o) {
            float *yp = y + (b * oc + o) * oh * ow;
            for (i64 i = 0; i < oh * ow; ++i) yp[i] = 0.0f;
            for (i64 c = 0; c < ic; ++c) {
                const float *xp = x + (b * ic + c) * ih * iw;
                for (i64 fi = 0; fi < fh; ++fi)
                    for (i64 fj = 0; fj < fw; ++fj) {
                        const float wv = w[((o * ic + c) * fh + fi) * fw + fj];
                        for (i64 ho = 0; ho < oh; ++ho) {
                            const float *xr = xp + (ho + fi) * iw + fj;
                            float *yr = yp + ho * ow;
                            for (i64 wo = 0; wo < ow; ++wo) yr[wo] += wv * xr[wo];
                        }
                    }
            }
        }
}

/* ------------------------------------- conv_direct, packed and register-tiled ---- */

/* The reference host's f32 Conv2 for default options as it actually runs (layer.rs:936-943 ->
 * layer/conv_direct.rs:84-96 `conv2_direct_forward`): pack the input to [bs, ic/8, ih, iw][8 channels]
 * (:368-437; not packed when ic == 1, :288-291), pack the weights to [oc/8, ic/TCX, fh, fw][TCX][8 output
 * channels] (:487-557), run the register-tiled kernel (:760-946), unpack [bs, oc/8, oh, ow][8] to NCHW
 * (:692-758).  The kernel keeps a TBY x TWY tile of 8-wide accumulators (TBY blocks of 8 output channels x TWY
 * output columns; TBY = min(oc/8, 4), TWY = min(15 / (TBY + 1), ow) when compiled with FMA, :766-774, :925-926)
 * and, per filter tap and input channel, broadcasts TWY input values and multiplies them into TBY weight
 * vectors with `mul_add` (:799-820).  Images are dealt to threads round robin (`broadcast(Some(bs))`,
 * tensor/parallel.rs:151-168).  `wide::f32x8` is __m256 here.  Summation order per output: (ic block, fi, fj,
 * channel within the block), each step one fused multiply-add. */
#include <immintrin.h>

static inline i64 div_up(i64 a, i64 b) { return a / b + (a % b != 0); }

/* f32x8::transpose of an 8 x 8 tile (rows in r[0..8]) */
static inline void transpose8x8(__m256 r[8]) {
    __m256 t0 = _mm256_unpacklo_ps(r[0], r[1]), t1 = _mm256_unpackhi_ps(r[0], r[1]);
    __m256 t2 = _mm256_unpacklo_ps(r[2], r[3]), t3 = _mm256_unpackhi_ps(r[2], r[3]);
    __m256 t4 = _mm256_unpacklo_ps(r[4], r[5]), t5 = _mm256_unpackhi_ps(r[4], r[5]);
    __m256 t6 = _mm256_unpacklo_ps(r[6], r[7]), t7 = _mm256_unpackhi_ps(r[6], r[7]);
    __m256 u0 = _mm256_shuffle_ps(t0, t2, 0x44), u1 = _mm256_shuffle_ps(t0, t2, 0xEE);
    __m256 u2 = _mm256_shuffle_ps(t1, t3, 0x44), u3 = _mm256_shuffle_ps(t1, t3, 0xEE);
    __m256 u4 = _mm256_shuffle_ps(t4, t6, 0x44), u5 = _mm256_shuffle_ps(t4, t6, 0xEE);
    __m256 u6 = _mm256_shuffle_ps(t5, t7, 0x44), u7 = _mm256_shuffle_ps(t5, t7, 0xEE);
    r[0] = _mm256_permute2f128_ps(u0, u4, 0x20); r[1] = _mm256_permute2f128_ps(u1, u5, 0x20);
    r[2] = _mm256_permute2f128_ps(u2, u6, 0x20); r[3] = _mm256_permute2f128_ps(u3, u7, 0x20);
    r[4] = _mm256_permute2f128_ps(u0, u4, 0x31); r[5] = _mm256_permute2f128_ps(u1, u5, 0x31);
    r[6] = _mm256_permute2f128_ps(u2, u6, 0x31); r[7] = _mm256_permute2f128_ps(u3, u7, 0x31);
}

/* pack_input2_host_f32 (conv_direct.rs:368-437): x [bs, ic, ih, iw] -> xp [bs, ic_blocks, ih, iw][8], the eight
 * channels of a block next to each other, missing channels zero; 8 x 8 tiles transposed in registers. */
static void cd_pack_input(const float *x, float *xp, i64 bs, i64 ic, i64 ih, i64 iw, int threads) {
    const i64 icb = div_up(ic, 8), plane = ih * iw;
#pragma omp parallel num_threads(threads)
    {
        const i64 tid = omp_get_thread_num(), nt = omp_get_num_threads();
        for (i64 b = tid; b < bs; b += nt)
            for (i64 cb = 0; cb < icb; ++cb) {
                const float *xs = x + (b * ic + cb * 8) * plane;
                float *xd = xp + (b * icb + cb) * plane * 8;
                const i64 nch = ic - cb * 8 < 8 ? ic - cb * 8 : 8;
                for (i64 h = 0; h < ih; ++h) {
                    i64 w0 = 0;
                    for (; w0 + 8 <= iw; w0 += 8) {
                        __m256 t[8];
                        for (i64 c = 0; c < 8; ++c)
                            t[c] = c < nch ? _mm256_loadu_ps(xs + c * plane + h * iw + w0) : _mm256_setzero_ps();
                        transpose8x8(t);
                        for (i64 j = 0; j < 8; ++j) _mm256_storeu_ps(xd + (h * iw + w0 + j) * 8, t[j]);
                    }
                    if (w0 < iw) {
                        float tile[8][8];
                        memset(tile, 0, sizeof(tile));
                        for (i64 c = 0; c < nch; ++c)
                            for (i64 j = 0; w0 + j < iw; ++j) tile[c][j] = xs[c * plane + h * iw + w0 + j];
                        __m256 t[8];
                        for (i64 c = 0; c < 8; ++c) t[c] = _mm256_loadu_ps(tile[c]);
                        transpose8x8(t);
                        for (i64 j = 0; w0 + j < iw; ++j) _mm256_storeu_ps(xd + (h * iw + w0 + j) * 8, t[j]);
                    }
                }
            }
    }
}

/* pack_weight2_host_f32<TCX> (conv_direct.rs:487-557): w [oc, ic, fh, fw] -> wp [oc_blocks, ic_blocks, fh, fw][TCX][8],
 * lane ciy of vector cix = w[8*ob + ciy, TCX*cb + cix, fi, fj]; lanes and vectors beyond oc / ic are zero. */
static void cd_pack_weight(const float *w, float *wp, i64 oc, i64 ic, i64 fh, i64 fw, i64 tcx) {
    const i64 ocb = div_up(oc, 8), icb = div_up(ic, tcx);
    memset(wp, 0, sizeof(float) * (size_t)(ocb * icb * fh * fw * tcx * 8));
    for (i64 ob = 0; ob < ocb; ++ob)
        for (i64 cb = 0; cb < icb; ++cb)
            for (i64 fi = 0; fi < fh; ++fi)
                for (i64 fj = 0; fj < fw; ++fj)
                    for (i64 ciy = 0; ciy < 8 && ob * 8 + ciy < oc; ++ciy)
                        for (i64 cix = 0; cix < tcx && cb * tcx + cix < ic; ++cix)
                            wp[((((ob * icb + cb) * fh + fi) * fw + fj) * tcx + cix) * 8 + ciy] =
                                w[(((ob * 8 + ciy) * ic + cb * tcx + cix) * fh + fi) * fw + fj];
}

/* unpack_output2_host_f32 (conv_direct.rs:692-758): yp [bs, oc_blocks, oh, ow][8] -> y [bs, oc, oh, ow] */
static void cd_unpack_output(const float *yp, float *y, i64 bs, i64 oc, i64 oh, i64 ow, int threads) {
    const i64 ocb = div_up(oc, 8), plane = oh * ow;
#pragma omp parallel num_threads(threads)
    {
        const i64 tid = omp_get_thread_num(), nt = omp_get_num_threads();
        for (i64 b = tid; b < bs; b += nt)
            for (i64 ob = 0; ob < ocb; ++ob) {
                const float *ys = yp + (b * ocb + ob) * plane * 8;
                float *yd = y + (b * oc + ob * 8) * plane;
                const i64 nch = oc - ob * 8 < 8 ? oc - ob * 8 : 8;
                for (i64 h = 0; h < oh; ++h) {
                    i64 w0 = 0;
                    for (; w0 + 8 <= ow; w0 += 8) {
                        __m256 t[8];
                        for (i64 j = 0; j < 8; ++j) t[j] = _mm256_loadu_ps(ys + (h * ow + w0 + j) * 8);
                        transpose8x8(t);
                        for (i64 c = 0; c < nch; ++c) _mm256_storeu_ps(yd + c * plane + h * ow + w0, t[c]);
                    }
                    if (w0 < ow) {
                        __m256 t[8];
                        for (i64 j = 0; j < 8; ++j) t[j] = w0 + j < ow ? _mm256_loadu_ps(ys + (h * ow + w0 + j) * 8) : _mm256_setzero_ps();
                        transpose8x8(t);
                        float row[8];
                        for (i64 c = 0; c < nch; ++c) {
                            _mm256_storeu_ps(row, t[c]);
                            for (i64 j = 0; w0 + j < ow; ++j) yd[c * plane + h * ow + w0 + j] = row[j];
                        }
                    }
                }
            }
    }
}

/* `kernel` + the tile loops of `inner` (conv_direct.rs:778-922) for one image, with TCX, TBY, TWY compile-time
 * constants at every call site (the function is inlined into cd_image_* below), so the accumulator tile lives in
 * registers as in the reference's const-generic instantiations. */
static inline __attribute__((always_inline)) void cd_image(const float *x, const float *wp, float *yp, i64 ic, i64 icb,
                                                            i64 ih, i64 iw, i64 ocb, i64 fh, i64 fw, i64 oh, i64 ow,
                                                            const int TCX, const int TBY, const int TWY) {
    for (i64 chunk = 0; chunk * TBY < ocb; ++chunk) {
        const i64 tby = ocb - chunk * TBY < TBY ? ocb - chunk * TBY : TBY;
        const float *wc = wp + chunk * TBY * icb * fh * fw * TCX * 8;
        float *yc = yp + chunk * TBY * oh * ow * 8;
        for (i64 cb = 0; cb < icb; ++cb) {
            const i64 tcx = ic - cb * TCX < TCX ? ic - cb * TCX : TCX;
            const float *xb = x + cb * ih * iw * TCX;
            for (i64 hy = 0; hy < oh; ++hy)
                for (i64 wy = 0; wy < ow; wy += TWY) {
                    const i64 twy = ow - wy < TWY ? ow - wy : TWY;
                    __m256 acc[4][7];
                    for (int b = 0; b < TBY; ++b)
                        for (int t = 0; t < TWY; ++t) acc[b][t] = _mm256_setzero_ps();
                    if (cb > 0)
                        for (int b = 0; b < TBY && b < tby; ++b)
                            for (int t = 0; t < TWY && t < twy; ++t)
                                acc[b][t] = _mm256_loadu_ps(yc + ((b * oh + hy) * ow + wy + t) * 8);
                    __m256 xv[7], wv[4];
                    for (int t = 0; t < TWY; ++t) xv[t] = _mm256_setzero_ps();
                    for (int b = 0; b < TBY; ++b) wv[b] = _mm256_setzero_ps();
                    for (i64 fi = 0; fi < fh; ++fi)
                        for (i64 fj = 0; fj < fw; ++fj)
                            for (i64 cix = 0; cix < tcx; ++cix) {
                                if (twy == TWY) {
                                    for (int t = 0; t < TWY; ++t)
                                        xv[t] = _mm256_broadcast_ss(xb + ((hy + fi) * iw + wy + fj + t) * TCX + cix);
                                } else {
                                    for (int t = 0; t < TWY && t < twy; ++t)
                                        xv[t] = _mm256_broadcast_ss(xb + ((hy + fi) * iw + wy + fj + t) * TCX + cix);
                                }
                                for (int b = 0; b < TBY && b < tby; ++b)
                                    wv[b] = _mm256_loadu_ps(wc + ((((b * icb + cb) * fh + fi) * fw + fj) * TCX + cix) * 8);
                                for (int b = 0; b < TBY; ++b)
                                    for (int t = 0; t < TWY; ++t) acc[b][t] = _mm256_fmadd_ps(xv[t], wv[b], acc[b][t]);
                            }
                    for (int b = 0; b < TBY && b < tby; ++b)
                        for (int t = 0; t < TWY && t < twy; ++t)
                            _mm256_storeu_ps(yc + ((b * oh + hy) * ow + wy + t) * 8, acc[b][t]);
                }
        }
    }
}

#define CD_ARGS const float *x, const float *wp, float *yp, i64 ic, i64 icb, i64 ih, i64 iw, i64 ocb, i64 fh, i64 fw, i64 oh, i64 ow
#define CD_PASS x, wp, yp, ic, icb, ih, iw, ocb, fh, fw, oh, ow
#define CD_INST(TCX, TBY, TWY) \
    static __attribute__((noinline)) void cd_image_##TCX##_##TBY##_##TWY(CD_ARGS) { cd_image(CD_PASS, TCX, TBY, TWY); }
#define CD_INST_TCX(TCX)                                                                                              \
    CD_INST(TCX, 1, 1) CD_INST(TCX, 1, 2) CD_INST(TCX, 1, 3) CD_INST(TCX, 1, 4) CD_INST(TCX, 1, 5) CD_INST(TCX, 1, 6)  \
    CD_INST(TCX, 1, 7) CD_INST(TCX, 2, 1) CD_INST(TCX, 2, 2) CD_INST(TCX, 2, 3) CD_INST(TCX, 2, 4) CD_INST(TCX, 2, 5)  \
    CD_INST(TCX, 3, 1) CD_INST(TCX, 3, 2) CD_INST(TCX, 3, 3) CD_INST(TCX, 4, 1) CD_INST(TCX, 4, 2) CD_INST(TCX, 4, 3)
CD_INST_TCX(1)
CD_INST_TCX(8)

typedef void (*cd_image_fn)(CD_ARGS);
#define CD_ROW(TCX, TBY) \
    {cd_image_##TCX##_##TBY##_1, cd_image_##TCX##_##TBY##_2, cd_image_##TCX##_##TBY##_3, 0, 0, 0, 0}
static cd_image_fn cd_pick(i64 tcx, i64 tby, i64 twy) {
    static const cd_image_fn t1[4][7] = {
        {cd_image_1_1_1, cd_image_1_1_2, cd_image_1_1_3, cd_image_1_1_4, cd_image_1_1_5, cd_image_1_1_6, cd_image_1_1_7},
        {cd_image_1_2_1, cd_image_1_2_2, cd_image_1_2_3, cd_image_1_2_4, cd_image_1_2_5, 0, 0}, CD_ROW(1, 3), CD_ROW(1, 4)};
    static const cd_image_fn t8[4][7] = {
        {cd_image_8_1_1, cd_image_8_1_2, cd_image_8_1_3, cd_image_8_1_4, cd_image_8_1_5, cd_image_8_1_6, cd_image_8_1_7},
        {cd_image_8_2_1, cd_image_8_2_2, cd_image_8_2_3, cd_image_8_2_4, cd_image_8_2_5, 0, 0}, CD_ROW(8, 3), CD_ROW(8, 4)};
    return (tcx == 1 ? t1 : t8)[tby - 1][twy - 1];
}

/* conv2_direct_forward (conv_direct.rs:84-96) for default options: x [bs, ic, ih, iw], w [oc, ic, fh, fw] ->
 * y [bs, oc, ih-fh+1, iw-fw+1].  threads <= 0: all cores (rayon's default pool). */
void orc_conv2_direct_packed_f32(const float *x, const float *w, float *y, i64 bs, i64 ic, i64 ih, i64 iw, i64 oc,
                                 i64 fh, i64 fw, int threads) {
    const i64 oh = ih - fh + 1, ow = iw - fw + 1;
    if (bs <= 0 || oc <= 0 || oh <= 0 || ow <= 0) return;
    if (threads <= 0) threads = omp_get_max_threads();
    if ((i64)threads > bs) threads = (int)bs;
    const i64 tcx = ic == 1 ? 1 : 8;
    const i64 icb = div_up(ic, tcx), ocb = div_up(oc, 8);
    const i64 tby = ocb < 4 ? ocb : 4;
    i64 twy = 15 / (tby + 1);
    if (twy > ow) twy = ow;
    float *xp = NULL;
    if (tcx == 8) {
        xp = (float *)aligned_alloc(64, sizeof(float) * (size_t)(bs * icb * ih * iw * 8));
        cd_pack_input(x, xp, bs, ic, ih, iw, threads);
    }
    float *wp = (float *)aligned_alloc(64, (sizeof(float) * (size_t)(ocb * icb * fh * fw * tcx * 8) + 63) / 64 * 64);
    cd_pack_weight(w, wp, oc, ic, fh, fw, tcx);
    float *yp = (float *)aligned_alloc(64, (sizeof(float) * (size_t)(bs * ocb * oh * ow * 8) + 63) / 64 * 64);
    const cd_image_fn fn = cd_pick(tcx, tby, twy);
    const float *xs = tcx == 8 ? xp : x;
    const i64 x_image = icb * ih * iw * tcx, y_image = ocb * oh * ow * 8;
#pragma omp parallel num_threads(threads)
    {
        const i64 tid = omp_get_thread_num(), nt = omp_get_num_threads();
        for (i64 b = tid; b < bs; b += nt) fn(xs + b * x_image, wp, yp + b * y_image, ic, icb, ih, iw, ocb, fh, fw, oh, ow);
    }
    cd_unpack_output(yp, y, bs, oc, oh, ow, threads);
    free(xp);
    free(wp);
    free(yp);
}

/* direct == 2: convolutions through orc_conv2_direct_packed_f32, the packed register-tiled form the reference host
 * runs for f32; direct == 1: through the plain axpy form orc_conv2_direct_f32; direct == 0: through im2col + sgemm
 * (what conv2_im2col does). */
void orc_lenet5_forward_f32_alg(const float *x, i64 bs, const float *w1, const float *w2, const float *wd1,
                                const float *wd2, const float *wd3, const float *b3, float *logits, int threads,
                                int direct);

void orc_lenet5_forward_f32(const float *x, i64 bs, const float *w1, const float *w2, const float *wd1,
                            const float *wd2, const float *wd3, const float *b3, float *logits, int threads) {
    orc_lenet5_forward_f32_alg(x, bs, w1, w2, wd1, wd2, wd3, b3, logits, threads, 0);
}

void orc_lenet5_forward_f32_alg(const float *x, i64 bs, const float *w1, const float *w2, const float *wd1,
                                const float *wd2, const float *wd3, const float *b3, float *logits, int threads,
                                int direct) {
    float *c1 = (float *)malloc(sizeof(float) * bs * 6 * 24 * 24);
    float *p1 = (float *)malloc(sizeof(float) * bs * 6 * 12 * 12);
    float *c2 = (float *)malloc(sizeof(float) * bs * 16 * 8 * 8);
    float *p2 = (float *)malloc(sizeof(float) * bs * 16 * 4 * 4);
    float *d1 = (float *)malloc(sizeof(float) * bs * 128);
    float *d2 = (float *)malloc(sizeof(float) * bs * 84);
    if (direct == 2) orc_conv2_direct_packed_f32(x, w1, c1, bs, 1, 28, 28, 6, 5, 5, 0);
    else if (direct) orc_conv2_direct_f32(x, w1, c1, bs, 1, 28, 28, 6, 5, 5);
    else conv_im2col_f32(x, w1, c1, bs, 1, 28, 28, 6, 5, 5, threads);
    orc_relu_f32(c1, c1, bs * 6 * 24 * 24);
    orc_max_pool2_f32(c1, p1, bs * 6, 24, 24, 2, 2, 2, 2);
    if (direct == 2) orc_conv2_direct_packed_f32(p1, w2, c2, bs, 6, 12, 12, 16, 5, 5, 0);
    else if (direct) orc_conv2_direct_f32(p1, w2, c2, bs, 6, 12, 12, 16, 5, 5);
    else conv_im2col_f32(p1, w2, c2, bs, 6, 12, 12, 16, 5, 5, threads);
    orc_relu_f32(c2, c2, bs * 16 * 8 * 8);
    orc_max_pool2_f32(c2, p2, bs * 16, 8, 8, 2, 2, 2, 2);
    orc_gemm_f32_host(bs, 256, 128, 1.0f, p2, 0, 256, 1, wd1, 0, 128, 1, 0.0f, d1, 0, 128, 1, threads);
    orc_relu_f32(d1, d1, bs * 128);
    orc_gemm_f32_host(bs, 128, 84, 1.0f, d1, 0, 128, 1, wd2, 0, 84, 1, 0.0f, d2, 0, 84, 1, threads);
    orc_relu_f32(d2, d2, bs * 84);
    orc_gemm_f32_host(bs, 84, 10, 1.0f, d2, 0, 84, 1, wd3, 0, 10, 1, 0.0f, logits, 0, 10, 1, threads);
    orc_bias_add_rows_f32(logits, b3, bs, 10);
    free(c1); free(p1); free(c2); free(p2); free(d1); free(d2);
}

/* ------------------------------------------------- training tail (host) ---- */

/* Strided copy of up to 4 dims, same element type: `assign` with BinaryOp::Identity, alpha = 1
 * (src/tensor/ops.rs:257-318): y[i] = x[i] over the index space `d`, element strides sx / sy
 * (a stride 0 on x is a broadcast).  es = element size in bytes. */
void orc_assign4(const void *x, i64 off_x, const i64 *sx, void *y, i64 off_y, const i64 *sy, const i64 *d, i64 es) {
    const unsigned char *xb = (const unsigned char *)x;
    unsigned char *yb = (unsigned char *)y;
    for (i64 i0 = 0; i0 < d[0]; ++i0)
        for (i64 i1 = 0; i1 < d[1]; ++i1)
            for (i64 i2 = 0; i2 < d[2]; ++i2)
                for (i64 i3 = 0; i3 < d[3]; ++i3) {
                    const i64 ix = off_x + i0 * sx[0] + i1 * sx[1] + i2 * sx[2] + i3 * sx[3];
                    const i64 iy = off_y + i0 * sy[0] + i1 * sy[1] + i2 * sy[2] + i3 * sy[3];
                    memcpy(yb + iy * es, xb + ix * es, (size_t)es);
                }
}

/* scaled_add: y = alpha * x + y with BinaryOp::Add (src/tensor/ops.rs:294-296 `op.eval(alpha * x, y)`):
 * the product and the sum are each one operation in T.  alpha is given in T's precision already
 * (optimizer.rs:420-423 casts -learning_rate to the parameter type first). */
void orc_scaled_add_f32(float *y, float alpha, const float *x, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        volatile float prod = alpha * x[i];
        y[i] = prod + y[i];
    }
}
void orc_scaled_add_bf16(bf16_t *y, float alpha, const bf16_t *x, i64 n) {
    const bf16_t a = f32_to_bf16(alpha);
    for (i64 i = 0; i < n; ++i) y[i] = bf16_add(bf16_mul(a, x[i]), y[i]);
}

/* The same on views (src/tensor/ops.rs:192-204 `scaled_add` -> `assign(BinaryOp::Add, alpha, rhs, self)`, :257-318:
 * `rhs.broadcast(self.raw_dim())` then `*y = op.eval(alpha * x.cast(), *y)` per element, eval = a + b at :1319-1330).
 * Index space d[0..4], signed element strides, stride 0 on x = broadcast. */
void orc_scaled_add_strided_f32(float *y, i64 off_y, const i64 *sy, float alpha, const float *x, i64 off_x, const i64 *sx,
                                const i64 *d) {
    for (i64 i0 = 0; i0 < d[0]; ++i0)
        for (i64 i1 = 0; i1 < d[1]; ++i1)
            for (i64 i2 = 0; i2 < d[2]; ++i2)
                for (i64 i3 = 0; i3 < d[3]; ++i3) {
                    const i64 ix = off_x + i0 * sx[0] + i1 * sx[1] + i2 * sx[2] + i3 * sx[3];
                    const i64 iy = off_y + i0 * sy[0] + i1 * sy[1] + i2 * sy[2] + i3 * sy[3];
                    volatile float prod = alpha * x[ix];
                    y[iy] = prod + y[iy];
                }
}
void orc_scaled_add_strided_bf16(bf16_t *y, i64 off_y, const i64 *sy, float alpha, const bf16_t *x, i64 off_x,
                                 const i64 *sx, const i64 *d) {
    const bf16_t a = f32_to_bf16(alpha);
    for (i64 i0 = 0; i0 < d[0]; ++i0)
        for (i64 i1 = 0; i1 < d[1]; ++i1)
            for (i64 i2 = 0; i2 < d[2]; ++i2)
                for (i64 i3 = 0; i3 < d[3]; ++i3) {
                    const i64 ix = off_x + i0 * sx[0] + i1 * sx[1] + i2 * sx[2] + i3 * sx[3];
                    const i64 iy = off_y + i0 * sy[0] + i1 * sy[1] + i2 * sy[2] + i3 * sy[3];
                    y[iy] = bf16_add(bf16_mul(a, x[ix]), y[iy]);
                }
}

/* accuracy_host (src/learn/criterion.rs:30-47): rows whose target score is strictly greater than every other
 * score.  A target >= classes panics on the host; here it does not count (the device kernel's rule, :281-284). */
i64 orc_accuracy_f32(const float *x, const uint8_t *t, i64 bs, i64 classes) {
    i64 n = 0;
    for (i64 i = 0; i < bs; ++i) {
        if (t[i] >= classes) continue;
        const float xt = x[i * classes + t[i]];
        int ok = 1;
        for (i64 j = 0; j < classes; ++j)
            if (j != t[i] && !(xt > x[i * classes + j])) ok = 0;
        n += ok;
    }
    return n;
}
i64 orc_accuracy_bf16(const bf16_t *x, const uint8_t *t, i64 bs, i64 classes) {
    i64 n = 0;
    for (i64 i = 0; i < bs; ++i) {
        if (t[i] >= classes) continue;
        const float xt = bf16_to_f32(x[i * classes + t[i]]);
        int ok = 1;
        for (i64 j = 0; j < classes; ++j)
            if (j != t[i] && !(xt > bf16_to_f32(x[i * classes + j]))) ok = 0;
        n += ok;
    }
    return n;
}

/* SGD with momentum (optimizer.rs:430-465, kernel :509-512): in f32, v = m*v + dw; w -= lr*v; then
 * both cast back to T. */
void orc_sgd_momentum_f32(float *w, const float *dw, float lr, float m, float *v, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        volatile float mv = m * v[i];
        const float vn = mv + dw[i];
        volatile float step = lr * vn;
        v[i] = vn;
        w[i] = w[i] - step;
    }
}
void orc_sgd_momentum_bf16(bf16_t *w, const bf16_t *dw, float lr, float m, bf16_t *v, i64 n) {
    for (i64 i = 0; i < n; ++i) {
        volatile float mv = m * bf16_to_f32(v[i]);
        const float vn = mv + bf16_to_f32(dw[i]);
        volatile float step = lr * vn;
        v[i] = f32_to_bf16(vn);
        w[i] = f32_to_bf16(bf16_to_f32(w[i]) - step);
    }
}

/* Sum over axis 0 of a row-major [rows, cols] array, as ndarray's sum_axis does it when the axis is
 * not the one with the smallest stride (reduce.rs:59-62 -> ndarray `res = res + &subview` per row):
 * zeros, then one add in T per row, rows ascending.  This is the bias gradient (autograd.rs:490-542). */
void orc_sum_axis0_f32(const float *x, float *y, i64 rows, i64 cols) {
    for (i64 j = 0; j < cols; ++j) y[j] = 0.0f;
    for (i64 i = 0; i < rows; ++i)
        for (i64 j = 0; j < cols; ++j) y[j] = y[j] + x[i * cols + j];
}
void orc_sum_axis0_bf16(const bf16_t *x, bf16_t *y, i64 rows, i64 cols) {
    for (i64 j = 0; j < cols; ++j) y[j] = 0;
    for (i64 i = 0; i < rows; ++i)
        for (i64 j = 0; j < cols; ++j) y[j] = bf16_add(y[j], x[i * cols + j]);
}

/* cross_entropy_loss_host (src/learn/criterion.rs:205-226): per row, m = max in f32, s = sum of
 * exp(x - m) in f32 in element order, loss += ln(s) - (x[t] - m), rows in order, all f32. */
static float ce_loss_rows(const float *row_f32, i64 classes, i64 t) {
    float m = row_f32[0];
    for (i64 j = 0; j < classes; ++j) m = fmaxf(m, row_f32[j]);
    float s = 0.0f;
    for (i64 j = 0; j < classes; ++j) s += expf(row_f32[j] - m);
    return logf(s) - (row_f32[t] - m);
}
float orc_cross_entropy_loss_f32(const float *x, const uint8_t *t, i64 bs, i64 classes) {
    float y = 0.0f;
    for (i64 i = 0; i < bs; ++i) y += ce_loss_rows(x + i * classes, classes, t[i]);
    return y;
}
float orc_cross_entropy_loss_bf16(const bf16_t *x, const uint8_t *t, i64 bs, i64 classes) {
    float y = 0.0f;
    float *row = (float *)malloc((size_t)classes * sizeof(float));
    for (i64 i = 0; i < bs; ++i) {
        for (i64 j = 0; j < classes; ++j) row[j] = bf16_to_f32(x[i * classes + j]);
        y += ce_loss_rows(row, classes, t[i]);
    }
    free(row);
    return y;
}

/* cross_entropy_loss_backward host branch (src/learn/neural_network/criterion.rs:79-103):
 * dy /= bs; dx = T(dy * (exp(x - m) / s - [j == t])) with f32 arithmetic. */
static void ce_backward_row(const float *row, float *out, i64 classes, i64 t, float dy) {
    float m = row[0];
    for (i64 j = 0; j < classes; ++j) m = fmaxf(m, row[j]);
    float s = 0.0f;
    for (i64 j = 0; j < classes; ++j) s += expf(row[j] - m);
    for (i64 j = 0; j < classes; ++j) {
        const float onehot = (j == t) ? 1.0f : 0.0f;
        volatile float p = expf(row[j] - m) / s;
        volatile float diff = p - onehot;
        out[j] = dy * diff;
    }
}
void orc_cross_entropy_backward_f32(const float *x, const uint8_t *t, float dy, float *dx, i64 bs, i64 classes) {
    dy /= (float)bs;
    for (i64 i = 0; i < bs; ++i) ce_backward_row(x + i * classes, dx + i * classes, classes, t[i], dy);
}
void orc_cross_entropy_backward_bf16(const bf16_t *x, const uint8_t *t, float dy, bf16_t *dx, i64 bs, i64 classes) {
    dy /= (float)bs;
    float *row = (float *)malloc((size_t)classes * 2 * sizeof(float));
    float *out = row + classes;
    for (i64 i = 0; i < bs; ++i) {
        for (i64 j = 0; j < classes; ++j) row[j] = bf16_to_f32(x[i * classes + j]);
        ce_backward_row(row, out, classes, t[i], dy);
        for (i64 j = 0; j < classes; ++j) dx[i * classes + j] = f32_to_bf16(out[j]);
    }
    free(row);
}

int orc_max_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

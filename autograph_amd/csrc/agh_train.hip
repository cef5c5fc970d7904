// Kernels around the contraction path that a training step needs: strided copy (`assign`),
// `scaled_add`, SGD with momentum, the axis-0 sum behind the bias gradient, and cross-entropy
// loss / gradient.  All follow the reference's HOST arithmetic: every operation the host performs
// in the element type is rounded to the element type here too, sums run in the host's order.
#include "agh_internal.h"

using namespace agh;

namespace {

constexpr int kThreads = 256;

unsigned grid_for(size_t n) {
    size_t blocks = (n + kThreads - 1) / kThreads;
    size_t cap = (size_t)compute_units() * 32;
    if (cap == 0) cap = 8192;
    return (unsigned)(blocks < cap ? blocks : cap);
}

// ---------------------------------------------------------------- assign ----
struct AssignParams {
    int64_t sx[4], sy[4];
    FastDiv div1, div2, div3;  // by d1*d2*d3, d2*d3, d3
    uint32_t d23, d3;
};

// One thread per element, index space walked with the last dimension fastest, so a destination in
// standard layout is written with consecutive lanes on consecutive elements.
template <typename T>
__global__ __launch_bounds__(kThreads) void assign_kernel(const T *__restrict__ x, T *__restrict__ y, AssignParams p,
                                                           uint32_t total) {
    for (uint32_t e = blockIdx.x * kThreads + threadIdx.x; e < total; e += gridDim.x * kThreads) {
        uint32_t i0, r0, i1, r1, i2, i3;
        p.div1.divmod(e, i0, r0);
        p.div2.divmod(r0, i1, r1);
        p.div3.divmod(r1, i2, i3);
        const int64_t ix = i0 * p.sx[0] + i1 * p.sx[1] + i2 * p.sx[2] + i3 * p.sx[3];
        const int64_t iy = i0 * p.sy[0] + i1 * p.sy[1] + i2 * p.sy[2] + i3 * p.sy[3];
        y[iy] = x[ix];
    }
}

// Batched 2-D transposition through LDS, for copies whose source and destination are both contiguous, but along
// different dimensions (NHWC <-> NCHW, `t().to_standard_layout()`): index space [b0, b1, R, C] with the source
// contiguous along R and the destination along C.  A workgroup moves a 64 x 64 tile: 16-byte loads along R, one
// 32-bit LDS slot per element in a tile of odd pitch (both the scattering writes and the gathering reads are
// conflict-free), 16-byte stores along C.  VEC = 1 is the same walk element by element for unaligned views.
struct TransposeParams {
    int64_t sx_b0, sx_b1, sx_c;  // source strides of the batch dimensions and of C (its stride along R is 1)
    int64_t sy_b0, sy_b1, sy_r;  // destination strides of the batch dimensions and of R (its stride along C is 1)
    int R, C, tiles_r, tiles_c;
    FastDiv div_tiles, div_tc, div_b1;
};
constexpr int kTT = 64, kTPitch = kTT + 1;

template <typename T, int VEC>
__global__ __launch_bounds__(kThreads) void transpose_tile_kernel(const T *__restrict__ x, T *__restrict__ y, TransposeParams p) {
    __shared__ uint32_t tile[kTT * kTPitch];
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    constexpr int EPW = 4 / (int)sizeof(T);  // elements per 32-bit word of a vector register
    uint32_t bidx, t, tr, tc, b0, b1;
    p.div_tiles.divmod(blockIdx.x, bidx, t);
    p.div_tc.divmod(t, tr, tc);
    p.div_b1.divmod(bidx, b0, b1);
    const int r_base = tr * kTT, c_base = tc * kTT;
    const T *xs = x + (int64_t)b0 * p.sx_b0 + (int64_t)b1 * p.sx_b1;
    T *yd = y + (int64_t)b0 * p.sy_b0 + (int64_t)b1 * p.sy_b1;
    constexpr int VPT = kTT * kTT / VEC / kThreads, VPL = kTT / VEC;  // vectors per thread, vectors per tile line
    // ---- load along R ----
    u32x4 reg[VPT];
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int v = threadIdx.x + k * kThreads, rv = v % VPL, c = v / VPL;
        const int r = r_base + rv * VEC, cg = c_base + c;
        reg[k] = u32x4{0, 0, 0, 0};
        if (r < p.R && cg < p.C) {
            const T *src = xs + (int64_t)cg * p.sx_c + r;
            if constexpr (VEC * sizeof(T) == 16) reg[k] = __builtin_nontemporal_load((const u32x4 *)src);
            else reg[k].x = (uint32_t)*src;
        }
    }
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int v = threadIdx.x + k * kThreads, rv = v % VPL, c = v / VPL;
        const uint32_t w[4] = {reg[k].x, reg[k].y, reg[k].z, reg[k].w};
#pragma unroll
        for (int i = 0; i < VEC; ++i) {
            uint32_t e = w[i / EPW];
            if constexpr (sizeof(T) == 2) e = (e >> (16 * (i % EPW))) & 0xFFFFu;
            tile[(rv * VEC + i) * kTPitch + c] = e;
        }
    }
    __syncthreads();
    // ---- store along C ----
#pragma unroll
    for (int k = 0; k < VPT; ++k) {
        const int v = threadIdx.x + k * kThreads, cv = v % VPL, r = v / VPL;
        const int rg = r_base + r, c = c_base + cv * VEC;
        if (rg < p.R && c < p.C) {
            uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < VEC; ++i) {
                const uint32_t e = tile[r * kTPitch + cv * VEC + i];
                if constexpr (sizeof(T) == 2) w[i / EPW] |= e << (16 * (i % EPW));
                else w[i] = e;
            }
            T *dst = yd + (int64_t)rg * p.sy_r + c;
            if constexpr (VEC * sizeof(T) == 16) __builtin_nontemporal_store(u32x4{w[0], w[1], w[2], w[3]}, (u32x4 *)dst);
            else *dst = (T)w[0];
        }
    }
}

// Recognises the transposition pattern after dropping unit dimensions and merging dimensions that are contiguous
// in both views; returns 1 when the copy is not of that kind (the caller takes the element-wise kernel).
template <typename T>
int transpose_try(const char *name, const T *x, const int64_t (&sx)[4], T *y, const int64_t (&sy)[4], const int64_t (&d)[4]) {
    int64_t dd[4], ax[4], ay[4];
    int n = 0;
    for (int i = 0; i < 4; ++i) {
        if (d[i] == 1) continue;
        if (n > 0 && ax[n - 1] == sx[i] * d[i] && ay[n - 1] == sy[i] * d[i]) {  // dimension n-1 and i are one dimension
            dd[n - 1] *= d[i]; ax[n - 1] = sx[i]; ay[n - 1] = sy[i];
        } else {
            dd[n] = d[i]; ax[n] = sx[i]; ay[n] = sy[i]; ++n;
        }
    }
    int ir = -1, ic = -1;
    for (int i = 0; i < n; ++i) {
        if (ax[i] == 1 && ir < 0) ir = i;
        if (ay[i] == 1 && ic < 0) ic = i;
    }
    if (ir < 0 || ic < 0 || ir == ic || dd[ir] < 16 || dd[ic] < 16) return 1;
    int64_t bd[2] = {1, 1}, bsx[2] = {0, 0}, bsy[2] = {0, 0};
    int nb = 0;
    for (int i = 0; i < n; ++i)
        if (i != ir && i != ic) { bd[nb] = dd[i]; bsx[nb] = ax[i]; bsy[nb] = ay[i]; ++nb; }
    TransposeParams p;
    p.sx_b0 = bsx[0]; p.sx_b1 = bsx[1]; p.sx_c = ax[ic];
    p.sy_b0 = bsy[0]; p.sy_b1 = bsy[1]; p.sy_r = ay[ir];
    p.R = (int)dd[ir]; p.C = (int)dd[ic];
    p.tiles_r = (p.R + kTT - 1) / kTT; p.tiles_c = (p.C + kTT - 1) / kTT;
    const int64_t tiles = (int64_t)p.tiles_r * p.tiles_c, blocks = tiles * bd[0] * bd[1];
    if (blocks > 0x7FFFFFFFll) return 1;
    p.div_tiles = FastDiv((uint32_t)tiles);
    p.div_tc = FastDiv((uint32_t)p.tiles_c);
    p.div_b1 = FastDiv((uint32_t)bd[1]);
    constexpr int V = 16 / (int)sizeof(T);
    auto mult = [](int64_t v) { return v % V == 0; };
    const bool vec = p.R % V == 0 && p.C % V == 0 && mult(p.sx_c) && mult(p.sx_b0) && mult(p.sx_b1) && mult(p.sy_r) &&
                     mult(p.sy_b0) && mult(p.sy_b1) && (((uintptr_t)x | (uintptr_t)y) & 15) == 0;
    if (vec) hipLaunchKernelGGL((transpose_tile_kernel<T, V>), dim3((unsigned)blocks), dim3(kThreads), 0, stream(), x, y, p);
    else hipLaunchKernelGGL((transpose_tile_kernel<T, 1>), dim3((unsigned)blocks), dim3(kThreads), 0, stream(), x, y, p);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int assign_launch(const char *name, const void *x, int64_t off_x, const int64_t (&sx)[4], void *y, int64_t off_y,
                  const int64_t (&sy)[4], const int64_t (&d)[4]) {
    AGH_API_ENTER();
    int64_t total = 1;
    for (int i = 0; i < 4; ++i) {
        if (d[i] < 0) return fail(AGH_EINVAL, "%s: negative dimension", name);
        if (d[i] > ((int64_t)1 << 30)) return fail(AGH_ERANGE, "%s: dimension too large", name);
        total *= d[i];
        if (total > ((int64_t)1 << 31) - 1) return fail(AGH_ERANGE, "%s: more than 2^31-1 elements", name);
    }
    if (total == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    // large transposing copies go through LDS tiles; everything else one element per thread
    if (total >= 4096) {
        const int rc = transpose_try<T>(name, (const T *)x + off_x, sx, (T *)y + off_y, sy, d);
        if (rc != 1) return rc;
    }
    AssignParams p;
    for (int i = 0; i < 4; ++i) { p.sx[i] = sx[i]; p.sy[i] = sy[i]; }
    p.div1 = FastDiv((uint32_t)(d[1] * d[2] * d[3]));
    p.div2 = FastDiv((uint32_t)(d[2] * d[3]));
    p.div3 = FastDiv((uint32_t)d[3]);
    hipLaunchKernelGGL(assign_kernel<T>, dim3(grid_for((size_t)total)), dim3(kThreads), 0, stream(),
                       (const T *)x + off_x, (T *)y + off_y, p, (uint32_t)total);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

// ------------------------------------------------------------ scaled_add ----
template <typename T>
__global__ __launch_bounds__(kThreads) void scaled_add_kernel(T *__restrict__ y, float alpha, const T *__restrict__ x, size_t n) {
    const float a = Elem<T>::to_f32(Elem<T>::from_f32(alpha));  // alpha is cast to the element type first
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads) {
        const T prod = Elem<T>::from_f32(a * Elem<T>::to_f32(x[i]));
        y[i] = Elem<T>::from_f32(Elem<T>::to_f32(prod) + Elem<T>::to_f32(y[i]));
    }
}

// The same operation on views: index space [d0, d1, d2, d3] walked with d3 fastest, signed element strides, a
// stride 0 on x broadcasts.  VEC > 1: d3 is walked in groups of VEC elements that are contiguous in y (sy3 == 1)
// and either contiguous (sx3 == 1) or one broadcast element (sx3 == 0) in x; groups are 16-byte loads and stores.
struct ScaledAddParams {
    int64_t sx[4], sy[4];
    FastDiv div1, div2, div3;  // by d1*d2*g3, d2*g3, g3 with g3 = d3 / VEC
};

template <typename T, int VEC>
__global__ __launch_bounds__(kThreads) void scaled_add_strided_kernel(T *__restrict__ y, float alpha, const T *__restrict__ x,
                                                                       ScaledAddParams p, uint32_t total) {
    typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
    const float a = Elem<T>::to_f32(Elem<T>::from_f32(alpha));
    for (uint32_t e = blockIdx.x * kThreads + threadIdx.x; e < total; e += gridDim.x * kThreads) {
        uint32_t i0, r0, i1, r1, i2, i3;
        p.div1.divmod(e, i0, r0);
        p.div2.divmod(r0, i1, r1);
        p.div3.divmod(r1, i2, i3);
        const int64_t ix = i0 * p.sx[0] + i1 * p.sx[1] + i2 * p.sx[2] + (int64_t)(i3 * VEC) * p.sx[3];
        const int64_t iy = i0 * p.sy[0] + i1 * p.sy[1] + i2 * p.sy[2] + (int64_t)(i3 * VEC) * p.sy[3];
        if constexpr (VEC == 1) {
            const T prod = Elem<T>::from_f32(a * Elem<T>::to_f32(x[ix]));
            y[iy] = Elem<T>::from_f32(Elem<T>::to_f32(prod) + Elem<T>::to_f32(y[iy]));
        } else {
            T xv[VEC], yv[VEC];
            *(u32x4 *)yv = *(const u32x4 *)(y + iy);
            if (p.sx[3] != 0) *(u32x4 *)xv = *(const u32x4 *)(x + ix);
            else {
                const T b = x[ix];
#pragma unroll
                for (int u = 0; u < VEC; ++u) xv[u] = b;
            }
#pragma unroll
            for (int u = 0; u < VEC; ++u) {
                const T prod = Elem<T>::from_f32(a * Elem<T>::to_f32(xv[u]));
                yv[u] = Elem<T>::from_f32(Elem<T>::to_f32(prod) + Elem<T>::to_f32(yv[u]));
            }
            *(u32x4 *)(y + iy) = *(const u32x4 *)yv;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(kThreads) void sgd_momentum_kernel(T *__restrict__ w, const T *__restrict__ dw, float lr, float m,
                                                                 T *__restrict__ v, size_t n) {
    for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n; i += (size_t)gridDim.x * kThreads) {
        const float mv = m * Elem<T>::to_f32(v[i]);
        const float vn = mv + Elem<T>::to_f32(dw[i]);
        const float step = lr * vn;
        v[i] = Elem<T>::from_f32(vn);
        w[i] = Elem<T>::from_f32(Elem<T>::to_f32(w[i]) - step);
    }
}

// ------------------------------------------------------------- sum axis 0 ----
// One thread per column, rows added one at a time in the element type, starting from zero.
template <typename T>
__global__ __launch_bounds__(kThreads) void sum_axis0_kernel(const T *__restrict__ x, T *__restrict__ y, int64_t rows, int64_t cols) {
    const int64_t j = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (j >= cols) return;
    T acc = Elem<T>::zero();
    // rows are added one at a time in the element type, in row order; eight are requested before the first add
    int64_t i = 0;
    for (; i + 8 <= rows; i += 8) {
        T v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) v[u] = x[(i + u) * cols + j];
#pragma unroll
        for (int u = 0; u < 8; ++u) acc = Elem<T>::from_f32(Elem<T>::to_f32(acc) + Elem<T>::to_f32(v[u]));
    }
    for (; i < rows; ++i) acc = Elem<T>::from_f32(Elem<T>::to_f32(acc) + Elem<T>::to_f32(x[i * cols + j]));
    y[j] = acc;
}

// ---------------------------------------------------------- cross entropy ----
template <typename T>
__device__ __forceinline__ void row_max_sum(const T *row, int classes, float &m, float &s) {
    m = Elem<T>::to_f32(row[0]);
    for (int j = 0; j < classes; ++j) m = fmaxf(m, Elem<T>::to_f32(row[j]));
    s = 0.0f;
    for (int j = 0; j < classes; ++j) s += expf(Elem<T>::to_f32(row[j]) - m);
}

// A single workgroup: rows are evaluated 256 at a time, then one thread adds the 256 row losses to
// the running total in row order, which is the order of the host's loop.
template <typename T>
__global__ __launch_bounds__(kThreads) void cross_entropy_loss_kernel(const T *__restrict__ x, const uint8_t *__restrict__ t,
                                                                       int64_t bs, int classes, float *__restrict__ out) {
    __shared__ float part[kThreads];
    float total = 0.0f;
    for (int64_t base = 0; base < bs; base += kThreads) {
        const int64_t r = base + threadIdx.x;
        float l = 0.0f;
        if (r < bs) {
            const T *row = x + r * classes;
            float m, s;
            row_max_sum(row, classes, m, s);
            l = logf(s) - (Elem<T>::to_f32(row[t[r]]) - m);
        }
        part[threadIdx.x] = l;
        __syncthreads();
        if (threadIdx.x == 0) {
            const int cnt = (int)min((int64_t)kThreads, bs - base);
            for (int i = 0; i < cnt; ++i) total += part[i];
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) *out = total;
}

template <typename T>
__global__ __launch_bounds__(kThreads) void cross_entropy_backward_kernel(const T *__restrict__ x, const uint8_t *__restrict__ t,
                                                                           float dy, T *__restrict__ dx, int64_t bs, int classes) {
    const int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (r >= bs) return;
    const T *row = x + r * classes;
    float m, s;
    row_max_sum(row, classes, m, s);
    const int tr = t[r];
    for (int j = 0; j < classes; ++j) {
        const float p = expf(Elem<T>::to_f32(row[j]) - m) / s;
        const float diff = p - (j == tr ? 1.0f : 0.0f);
        dx[r * classes + j] = Elem<T>::from_f32(dy * diff);
    }
}

// ---------------------------------------------------------------- accuracy ----
// One thread per row: the prediction counts when the target's score is strictly greater than every other score of the
// row (a tie, a NaN or a target >= classes does not count).  Every workgroup adds up its rows' flags in LDS and
// writes one count: straight to `out` when the grid is a single workgroup, else to its slot of `partial`, which
// accuracy_sum_kernel adds up.  No atomics, so `out` may be pinned host memory.
template <typename T>
__global__ __launch_bounds__(kThreads) void accuracy_kernel(const T *__restrict__ x, const uint8_t *__restrict__ t, int64_t bs,
                                                             int classes, uint32_t *__restrict__ partial, uint32_t *__restrict__ out) {
    __shared__ uint32_t cnt[kThreads / 64];
    uint32_t mine = 0;
    for (int64_t r = (int64_t)blockIdx.x * kThreads + threadIdx.x; r < bs; r += (int64_t)gridDim.x * kThreads) {
        const int tr = t[r];
        if (tr >= classes) continue;
        const T *row = x + r * classes;
        const float xt = Elem<T>::raw(row[tr]);
        bool ok = true;
        for (int j = 0; j < classes; ++j) ok = ok && (j == tr || xt > Elem<T>::raw(row[j]));
        mine += ok ? 1u : 0u;
    }
    for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off, 64);
    if ((threadIdx.x & 63) == 0) cnt[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t s = 0;
        for (int w = 0; w < kThreads / 64; ++w) s += cnt[w];
        if (gridDim.x == 1) *out = s;
        else partial[blockIdx.x] = s;
    }
}

__global__ __launch_bounds__(kThreads) void accuracy_sum_kernel(const uint32_t *__restrict__ partial, int n, uint32_t *__restrict__ out) {
    __shared__ uint32_t cnt[kThreads / 64];
    uint32_t mine = 0;
    for (int i = threadIdx.x; i < n; i += kThreads) mine += partial[i];
    for (int off = 32; off > 0; off >>= 1) mine += __shfl_down(mine, off, 64);
    if ((threadIdx.x & 63) == 0) cnt[threadIdx.x >> 6] = mine;
    __syncthreads();
    if (threadIdx.x == 0) {
        uint32_t s = 0;
        for (int w = 0; w < kThreads / 64; ++w) s += cnt[w];
        *out = s;
    }
}

template <typename T>
int scaled_add_launch(const char *name, void *y, float alpha, const void *x, int64_t n) {
    AGH_API_ENTER();
    if (n < 0) return fail(AGH_EINVAL, "%s: negative length", name);
    if (n == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    hipLaunchKernelGGL(scaled_add_kernel<T>, dim3(grid_for((size_t)n)), dim3(kThreads), 0, stream(), (T *)y,
                       alpha, (const T *)x, (size_t)n);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int scaled_add_strided_launch(const char *name, void *y, int64_t off_y, const int64_t (&sy)[4], float alpha, const void *x,
                              int64_t off_x, const int64_t (&sx)[4], const int64_t (&d)[4]) {
    AGH_API_ENTER();
    int64_t total = 1;
    for (int i = 0; i < 4; ++i) {
        if (d[i] < 0) return fail(AGH_EINVAL, "%s: negative dimension", name);
        if (d[i] > ((int64_t)1 << 30)) return fail(AGH_ERANGE, "%s: dimension too large", name);
        total *= d[i];
        if (total > ((int64_t)1 << 31) - 1) return fail(AGH_ERANGE, "%s: more than 2^31-1 elements", name);
    }
    if (total == 0) return AGH_OK;
    if (!x || !y) return fail(AGH_ENULL, "%s: null buffer", name);
    for (int i = 0; i < 4; ++i)
        if (d[i] > 1 && sy[i] == 0) return fail(AGH_EINVAL, "%s: the destination cannot be a broadcast view (stride 0 along dimension %d)", name, i);
    const T *xp = (const T *)x + off_x;
    T *yp = (T *)y + off_y;
    constexpr int V = 16 / (int)sizeof(T);
    auto mult = [](int64_t v) { return v % V == 0; };
    // 16-byte groups along d3: y contiguous there, x contiguous or broadcast, every other step a whole number of groups
    bool vec = d[3] % V == 0 && sy[3] == 1 && (sx[3] == 1 || sx[3] == 0) && ((uintptr_t)yp & 15) == 0;
    for (int i = 0; i < 3 && vec; ++i) vec = d[i] == 1 || (mult(sy[i]) && (sx[3] == 0 || mult(sx[i])));
    if (vec && sx[3] == 1) vec = ((uintptr_t)xp & 15) == 0;
    const int64_t g3 = vec ? d[3] / V : d[3];
    ScaledAddParams p;
    for (int i = 0; i < 4; ++i) { p.sx[i] = sx[i]; p.sy[i] = sy[i]; }
    p.div1 = FastDiv((uint32_t)(d[1] * d[2] * g3));
    p.div2 = FastDiv((uint32_t)(d[2] * g3));
    p.div3 = FastDiv((uint32_t)g3);
    const uint32_t items = (uint32_t)(total / d[3] * g3);
    if (vec)
        hipLaunchKernelGGL((scaled_add_strided_kernel<T, V>), dim3(grid_for(items)), dim3(kThreads), 0, stream(), yp, alpha, xp, p, items);
    else
        hipLaunchKernelGGL((scaled_add_strided_kernel<T, 1>), dim3(grid_for(items)), dim3(kThreads), 0, stream(), yp, alpha, xp, p, items);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int accuracy_launch(const char *name, const void *x, const void *t, int64_t bs, int64_t classes, void *correct_out) {
    uint32_t *correct = (uint32_t *)correct_out;
    AGH_API_ENTER();
    if (bs < 0 || classes < 1) return fail(AGH_EINVAL, "%s: invalid shape", name);
    if (classes > 256) return fail(AGH_ERANGE, "%s: targets are u8, at most 256 classes", name);
    if (!correct) return fail(AGH_ENULL, "%s: null output", name);
    if (bs > 0 && (!x || !t)) return fail(AGH_ENULL, "%s: null buffer", name);
    int64_t blocks = (bs + kThreads - 1) / kThreads;
    if (blocks < 1) blocks = 1;
    if (blocks > 1024) blocks = 1024;
    uint32_t *partial = nullptr;
    if (blocks > 1) {
        void *ws = nullptr;
        if (int rc = workspace((size_t)blocks * sizeof(uint32_t), &ws)) return rc;
        partial = (uint32_t *)ws;
    }
    hipLaunchKernelGGL(accuracy_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(), (const T *)x, (const uint8_t *)t, bs,
                       (int)classes, partial, correct);
    AGH_LAUNCH_CHECK(name);
    if (blocks > 1) {
        hipLaunchKernelGGL(accuracy_sum_kernel, dim3(1), dim3(kThreads), 0, stream(), partial, (int)blocks, correct);
        AGH_LAUNCH_CHECK(name);
    }
    return AGH_OK;
}

template <typename T>
int sgd_momentum_launch(const char *name, void *w, const void *dw, float lr, float m, void *v, int64_t n) {
    AGH_API_ENTER();
    if (n < 0) return fail(AGH_EINVAL, "%s: negative length", name);
    if (n == 0) return AGH_OK;
    if (!w || !dw || !v) return fail(AGH_ENULL, "%s: null buffer", name);
    hipLaunchKernelGGL(sgd_momentum_kernel<T>, dim3(grid_for((size_t)n)), dim3(kThreads), 0, stream(), (T *)w,
                       (const T *)dw, lr, m, (T *)v, (size_t)n);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int sum_axis0_launch(const char *name, const void *x, void *y, int64_t rows, int64_t cols) {
    AGH_API_ENTER();
    if (rows < 0 || cols < 0) return fail(AGH_EINVAL, "%s: negative shape", name);
    if (cols == 0) return AGH_OK;
    if (!y || (!x && rows > 0)) return fail(AGH_ENULL, "%s: null buffer", name);
    const int64_t blocks = (cols + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFll) return fail(AGH_ERANGE, "%s: too many columns", name);
    hipLaunchKernelGGL(sum_axis0_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(), (const T *)x, (T *)y,
                       rows, cols);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

int ce_check(const char *name, const void *x, const void *t, int64_t bs, int64_t classes) {
    if (bs < 0 || classes < 1) return fail(AGH_EINVAL, "%s: invalid shape", name);
    if (classes > 256) return fail(AGH_ERANGE, "%s: targets are u8, at most 256 classes", name);
    if (bs > 0 && (!x || !t)) return fail(AGH_ENULL, "%s: null buffer", name);
    return AGH_OK;
}

template <typename T>
int ce_loss_launch(const char *name, const void *x, const void *t, int64_t bs, int64_t classes, float *loss) {
    AGH_API_ENTER();
    if (int rc = ce_check(name, x, t, bs, classes)) return rc;
    if (!loss) return fail(AGH_ENULL, "%s: null output", name);
    hipLaunchKernelGGL(cross_entropy_loss_kernel<T>, dim3(1), dim3(kThreads), 0, stream(), (const T *)x,
                       (const uint8_t *)t, bs, (int)classes, loss);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

template <typename T>
int ce_backward_launch(const char *name, const void *x, const void *t, float dy, void *dx, int64_t bs, int64_t classes) {
    AGH_API_ENTER();
    if (int rc = ce_check(name, x, t, bs, classes)) return rc;
    if (bs == 0) return AGH_OK;
    if (!dx) return fail(AGH_ENULL, "%s: null output", name);
    const int64_t blocks = (bs + kThreads - 1) / kThreads;
    if (blocks > 0x7FFFFFFFll) return fail(AGH_ERANGE, "%s: batch too large", name);
    // `dy /= batch_size` first, in f32, as the host does
    hipLaunchKernelGGL(cross_entropy_backward_kernel<T>, dim3((unsigned)blocks), dim3(kThreads), 0, stream(),
                       (const T *)x, (const uint8_t *)t, dy / (float)bs, (T *)dx, bs, (int)classes);
    AGH_LAUNCH_CHECK(name);
    return AGH_OK;
}

}  // namespace

#define AGH_ASSIGN_ARGS                                                                                              \
    const void *x, int64_t off_x, int64_t sx0, int64_t sx1, int64_t sx2, int64_t sx3, void *y, int64_t off_y,      \
        int64_t sy0, int64_t sy1, int64_t sy2, int64_t sy3, int64_t d0, int64_t d1, int64_t d2, int64_t d3

extern "C" {

int agh_assign_f32(AGH_ASSIGN_ARGS) {
    const int64_t sx[4] = {sx0, sx1, sx2, sx3}, sy[4] = {sy0, sy1, sy2, sy3}, d[4] = {d0, d1, d2, d3};
    return assign_launch<uint32_t>("agh_assign_f32", x, off_x, sx, y, off_y, sy, d);
}
int agh_assign_bf16(AGH_ASSIGN_ARGS) {
    const int64_t sx[4] = {sx0, sx1, sx2, sx3}, sy[4] = {sy0, sy1, sy2, sy3}, d[4] = {d0, d1, d2, d3};
    return assign_launch<uint16_t>("agh_assign_bf16", x, off_x, sx, y, off_y, sy, d);
}

int agh_scaled_add_f32(void *y, float alpha, const void *x, int64_t n) {
    return scaled_add_launch<float>("agh_scaled_add_f32", y, alpha, x, n);
}
int agh_scaled_add_bf16(void *y, float alpha, const void *x, int64_t n) {
    return scaled_add_launch<uint16_t>("agh_scaled_add_bf16", y, alpha, x, n);
}

#define AGH_SCALED_ADD_STRIDED_ARGS                                                                              \
    void *y, int64_t off_y, int64_t sy0, int64_t sy1, int64_t sy2, int64_t sy3, float alpha, const void *x,     \
        int64_t off_x, int64_t sx0, int64_t sx1, int64_t sx2, int64_t sx3, int64_t d0, int64_t d1, int64_t d2, int64_t d3
int agh_scaled_add_strided_f32(AGH_SCALED_ADD_STRIDED_ARGS) {
    const int64_t sx[4] = {sx0, sx1, sx2, sx3}, sy[4] = {sy0, sy1, sy2, sy3}, d[4] = {d0, d1, d2, d3};
    return scaled_add_strided_launch<float>("agh_scaled_add_strided_f32", y, off_y, sy, alpha, x, off_x, sx, d);
}
int agh_scaled_add_strided_bf16(AGH_SCALED_ADD_STRIDED_ARGS) {
    const int64_t sx[4] = {sx0, sx1, sx2, sx3}, sy[4] = {sy0, sy1, sy2, sy3}, d[4] = {d0, d1, d2, d3};
    return scaled_add_strided_launch<uint16_t>("agh_scaled_add_strided_bf16", y, off_y, sy, alpha, x, off_x, sx, d);
}

int agh_accuracy_f32(const void *x, const void *target_u8, int64_t bs, int64_t classes, void *correct) {
    return accuracy_launch<float>("agh_accuracy_f32", x, target_u8, bs, classes, correct);
}
int agh_accuracy_bf16(const void *x, const void *target_u8, int64_t bs, int64_t classes, void *correct) {
    return accuracy_launch<uint16_t>("agh_accuracy_bf16", x, target_u8, bs, classes, correct);
}

int agh_sgd_momentum_f32(void *w, const void *dw, float learning_rate, float momentum, void *velocity, int64_t n) {
    return sgd_momentum_launch<float>("agh_sgd_momentum_f32", w, dw, learning_rate, momentum, velocity, n);
}
int agh_sgd_momentum_bf16(void *w, const void *dw, float learning_rate, float momentum, void *velocity, int64_t n) {
    return sgd_momentum_launch<uint16_t>("agh_sgd_momentum_bf16", w, dw, learning_rate, momentum, velocity, n);
}

int agh_sum_axis0_f32(const void *x, void *y, int64_t rows, int64_t cols) {
    return sum_axis0_launch<float>("agh_sum_axis0_f32", x, y, rows, cols);
}
int agh_sum_axis0_bf16(const void *x, void *y, int64_t rows, int64_t cols) {
    return sum_axis0_launch<uint16_t>("agh_sum_axis0_bf16", x, y, rows, cols);
}

int agh_cross_entropy_loss_f32(const void *x, const void *target_u8, int64_t bs, int64_t classes, float *loss) {
    return ce_loss_launch<float>("agh_cross_entropy_loss_f32", x, target_u8, bs, classes, loss);
}
int agh_cross_entropy_loss_bf16(const void *x, const void *target_u8, int64_t bs, int64_t classes, float *loss) {
    return ce_loss_launch<uint16_t>("agh_cross_entropy_loss_bf16", x, target_u8, bs, classes, loss);
}
int agh_cross_entropy_backward_f32(const void *x, const void *target_u8, float dy, void *dx, int64_t bs, int64_t classes) {
    return ce_backward_launch<float>("agh_cross_entropy_backward_f32", x, target_u8, dy, dx, bs, classes);
}
int agh_cross_entropy_backward_bf16(const void *x, const void *target_u8, float dy, void *dx, int64_t bs, int64_t classes) {
    return ce_backward_launch<uint16_t>("agh_cross_entropy_backward_bf16", x, target_u8, dy, dx, bs, classes);
}

}  // extern "C"

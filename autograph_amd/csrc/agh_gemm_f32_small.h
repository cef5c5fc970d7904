// f32 products with few outputs and a short k (the Dense layers of small networks: 1000 x 256 x 128 and below).
//
// Such a launch is a chain of latencies, not arithmetic: the tiled kernels stage operand tiles through LDS behind
// barriers and walk k in one wave per tile, which costs 6 to 8 us where the matrix pipes are busy for well under one.
// Here a workgroup owns ONE 16 x 16 tile of D and its four waves split k: a wave reads its k range of the 16 P rows and
// 16 Q rows straight into registers (all reads in flight at once; 16-byte loads along k where k is an operand's
// unit-stride axis, element loads for any other strides), multiplies with v_mfma_f32_16x16x4_f32 (MFMA e of a piece of
// four k takes element e on both sides: a permutation of k that is the same for P and Q), and the four partial tiles
// are added in wave order through LDS.  Lane (g, i) then
// holds D[p0 + 4g .. 4g+3][q0 + i]: four consecutive p, one 16-byte store.  Same arithmetic per output as the tiled
// kernels up to the order of the f32 sums, fixed for a given shape.
#pragma once
#include "agh_gemm_kernel.h"

namespace agh {
namespace gemm {

typedef float f32x4_s __attribute__((ext_vector_type(4)));

// four consecutive k of one operand row, from clamped addresses (never a fault, the caller zeroes what lies behind
// its k range): one 16-byte load when k is the unit-stride axis (VEC; K a multiple of 4), else four loads
template <bool VEC>
__device__ __forceinline__ float4 small_piece(const float *row, int64_t ks, int k, int K) {
    if constexpr (VEC) {
        return *(const float4 *)(row + min(k, K - 4));
    } else {
        float4 v;
        v.x = row[(int64_t)min(k, K - 1) * ks];
        v.y = row[(int64_t)min(k + 1, K - 1) * ks];
        v.z = row[(int64_t)min(k + 2, K - 1) * ks];
        v.w = row[(int64_t)min(k + 3, K - 1) * ks];
        return v;
    }
}

// CH: pieces (4 values of k) per operand and wave in flight at a time: a wave covers 16 * CH values of k per trip
template <int CH, bool PVEC, bool QVEC>
__global__ __launch_bounds__(256) void gemm_f32_small_kernel(Args g, int k_per_wave) {
    __shared__ f32x4_s red[3][64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, grp = lane >> 4, i = lane & 15;
    const int tp = (int)(blockIdx.x % (unsigned)g.tiles_p), tq = (int)(blockIdx.x / (unsigned)g.tiles_p);
    const int p0 = tp * 16, q0 = tq * 16;
    const float *prow = (const float *)g.P + (int64_t)min(p0 + i, g.NP - 1) * g.ps;
    const float *qrow = (const float *)g.Q + (int64_t)min(q0 + i, g.NQ - 1) * g.qs;
    const int kb = wave * k_per_wave, kend = min(g.K, kb + k_per_wave);
    f32x4_s acc = {0.0f, 0.0f, 0.0f, 0.0f};
    for (int k0 = kb; k0 < kend; k0 += 16 * CH) {
        float4 pa[CH], qb[CH];
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            pa[c] = small_piece<PVEC>(prow, g.pk, k0 + 16 * c + 4 * grp, g.K);
            qb[c] = small_piece<QVEC>(qrow, g.qk, k0 + 16 * c + 4 * grp, g.K);
        }
#pragma unroll
        for (int c = 0; c < CH; ++c) {
            const int k = k0 + 16 * c + 4 * grp;
            const float a[4] = {pa[c].x, pa[c].y, pa[c].z, pa[c].w}, b[4] = {qb[c].x, qb[c].y, qb[c].z, qb[c].w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const bool live = k + e < kend;  // both sides zeroed: 0 * inf would poison the sum
                acc = __builtin_amdgcn_mfma_f32_16x16x4f32(live ? a[e] : 0.0f, live ? b[e] : 0.0f, acc, 0, 0, 0);
            }
        }
    }
    if (wave != 0) red[wave - 1][lane] = acc;
    __syncthreads();
    if (wave != 0) return;
    acc += red[0][lane];
    acc += red[1][lane];
    acc += red[2][lane];

    const int p = p0 + 4 * grp, q = q0 + i;
    if (q >= g.NQ || p >= g.NP) return;
    float *D = (float *)g.D;
    const float *bias = (const float *)g.bias;
    const bool has_bias = g.has_bias != 0;
    if (g.store_mode == ST_VEC) {  // NP is a multiple of 4 here: the four p are all inside
        float *dst = D + (int64_t)q * g.dq + p;
        float4 old = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (g.beta != 0.0f) old = *(const float4 *)dst;
        float bv[4] = {0.0f, 0.0f, 0.0f, 0.0f};
        if (has_bias) {
#pragma unroll
            for (int r = 0; r < 4; ++r) bv[r] = bias[(int64_t)(g.bias_on_p ? p + r : q) * g.bias_stride];
        }
        float4 out;
        out.x = finish<float>(acc[0], g.alpha, g.beta, old.x, has_bias, bv[0], g.act);
        out.y = finish<float>(acc[1], g.alpha, g.beta, old.y, has_bias, bv[1], g.act);
        out.z = finish<float>(acc[2], g.alpha, g.beta, old.z, has_bias, bv[2], g.act);
        out.w = finish<float>(acc[3], g.alpha, g.beta, old.w, has_bias, bv[3], g.act);
        *(float4 *)dst = out;
    } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            if (p + r >= g.NP) break;
            float *dst = D + (int64_t)q * g.dq + (int64_t)(p + r) * g.dp;
            const float old = g.beta != 0.0f ? *dst : 0.0f;
            const float bv = has_bias ? bias[(int64_t)(g.bias_on_p ? p + r : q) * g.bias_stride] : 0.0f;
            *dst = finish<float>(acc[r], g.alpha, g.beta, old, has_bias, bv, g.act);
        }
    }
}

// Takes products of at most 1024 tiles with k <= 1024, any strides (an operand whose k axis is the unit-stride one and
// 16-byte loadable is read 16 bytes at a time, any other element by element); 1 = not this kernel's, else a status
// code.  AGH_GEMM_SMALL=0 / 1 overrides the size rule (measurements, tests).
inline int gemm_f32_small_try(Args &g, int lp, int lq, bool vec_store, int64_t batch) {
    if (batch != 1 || g.K < 1) return 1;
    const int64_t tiles_p = (g.NP + 15) / 16, tiles_q = (g.NQ + 15) / 16, tiles = tiles_p * tiles_q;
    // a forced tile configuration or split count (AGH_GEMM_CFG / AGH_GEMM_SPLITS) means the tiled kernels are wanted
    const char *env = getenv("AGH_GEMM_SMALL");
    const bool forced_tiles = getenv("AGH_GEMM_CFG") != nullptr || getenv("AGH_GEMM_SPLITS") != nullptr;
    const bool want = (env && *env) ? atoi(env) != 0 : (!forced_tiles && tiles <= 1024 && g.K <= 1024);
    if (!want || tiles > 0x7FFFFFFF) return 1;
    g.tiles_p = (int)tiles_p;
    g.tiles_q = (int)tiles_q;
    g.store_mode = vec_store ? ST_VEC : ST_SCALAR;
    const int k_per_wave = (g.K + 63) / 64 * 16;
    const dim3 grid((unsigned)tiles), block(256);
    const bool pv = lp == LD_K, qv = lq == LD_K;
#define AGH_SMALL(CHV) \
    do { \
        if (pv && qv) hipLaunchKernelGGL((gemm_f32_small_kernel<CHV, true, true>), grid, block, 0, stream(), g, k_per_wave); \
        else if (pv) hipLaunchKernelGGL((gemm_f32_small_kernel<CHV, true, false>), grid, block, 0, stream(), g, k_per_wave); \
        else if (qv) hipLaunchKernelGGL((gemm_f32_small_kernel<CHV, false, true>), grid, block, 0, stream(), g, k_per_wave); \
        else hipLaunchKernelGGL((gemm_f32_small_kernel<CHV, false, false>), grid, block, 0, stream(), g, k_per_wave); \
    } while (0)
    if (k_per_wave <= 32) AGH_SMALL(2);
    else AGH_SMALL(4);
#undef AGH_SMALL
    AGH_LAUNCH_CHECK("small f32 gemm launch");
    return AGH_OK;
}

}  // namespace gemm
}  // namespace agh

// Host side of the GEMM entry points: argument checks (the reference's bail!s at
// src/tensor/linalg.rs:256-279), orientation / loader / tile selection, split-K planning
// (the job of linalg.rs:306-340) and the launches.  Included once per element type.
#pragma once
#include <stdlib.h>
#include <string.h>

#include <type_traits>

#include "agh_gemm_kernel.h"

namespace agh {
namespace gemm {

struct TileCfg {
    int bp, bq;
    float eff;       // relative MFMA efficiency of the tile shape (bigger tiles reuse operands more)
    int wgs_per_cu;  // workgroups a CU can hold (LDS / register bound)
    bool scalar_ok;  // has instantiations with the element-wise loader
};

// index = config id used by launch_cfg below
static const TileCfg kCfgs[] = {
    {256, 256, 1.00f, 1, false},
    {128, 256, 0.85f, 1, false},
    {256, 128, 0.85f, 1, false},
    {128, 128, 0.70f, 2, false},
    {64, 64, 0.35f, 4, true},
    {32, 128, 0.28f, 4, true},
    {128, 32, 0.28f, 4, true},
};
static constexpr int kNumCfgs = sizeof(kCfgs) / sizeof(kCfgs[0]);
// rate of a CU on 64 x 64 direct-to-LDS bf16 tiles relative to a 256 x 256 workgroup on a full chip: one workgroup with
// the CU to itself (ring of eight stages), two sharing it (rings of four)
static constexpr double kDirect64Alone = 0.27, kDirect64Shared = 0.19;

template <typename T, int BP, int BQ, int WGP, int WGQ, int LP, int LQ>
int launch_one(const Args &g, int splits) {
    auto kern = gemm_kernel<T, BP, BQ, WGP, WGQ, LP, LQ>;
    constexpr size_t smem = 2 * (size_t)(BP + BQ) * 128;
    static bool attr_done = false;
    if (!attr_done) {
        if (smem > 48 * 1024)
            AGH_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_done = true;
    }
    dim3 grid((unsigned)(g.tiles_p * g.tiles_q), (unsigned)splits, (unsigned)g.batch);
    hipLaunchKernelGGL(kern, grid, dim3(WGP * WGQ * 64), smem, stream(), g);
    AGH_LAUNCH_CHECK("gemm kernel launch");
    return AGH_OK;
}

#ifdef AGH_GEMM_WITH_BF16_DIRECT
// direct-to-LDS bf16 kernels: defined and explicitly instantiated in agh_gemm_bf16_dl_<tile>.hip
// (one translation unit per tile shape, so they compile in parallel)
template <int BP, int BQ, int WGP, int WGQ, int LP, int LQ, int NS>
int launch_one_dl(const Args &g, int splits);
#endif

inline int env_int(const char *name, int dflt);

#ifdef AGH_GEMM_WITH_BF16_DIRECT
// Two LDS stages, but a ring of four for a grid of 128 x 128 tiles that gives a CU one workgroup at most and has 20
// k-tiles or more: alone on its CU such a workgroup waits for loads most of the time (2048^3: 22.8 us with two stages,
// 17.9 us with four; at 16 k-tiles the four tiles requested up front cost 0.3 us more than they save).
// AGH_GEMM_RING=2|4 forces either.
template <int BP, int BQ, int WGP, int WGQ, int LP, int LQ>
int launch_dl_ring(const Args &g, int splits) {
    if constexpr (BP == 64 && BQ == 64) {
        // A k-tile of the 64 x 64 tile is eight MFMAs a wave, a small fraction of a load's latency: always a ring of
        // four stages (64 KB, two workgroups per CU).  Eight stages measured slower at every size (1024^3: 6.2 against
        // 5.6 us, 2048^3: 32.2 against 29.3 us).
        return launch_one_dl<BP, BQ, WGP, WGQ, LP, LQ, 4>(g, splits);
    } else {
        if constexpr (BP == 128 && BQ == 128) {
            const int64_t wgs = (int64_t)g.tiles_p * g.tiles_q * splits * g.batch;
            // split-K streams its operands from HBM once (no second workgroup re-reads them out of L2), where the deeper
            // ring pays from 8 k-tiles on (128x4096x4096 in 8 splits: 19.5 against 20.5 us; in 4: 17.2 against 20.1)
            const bool alone = wgs <= (compute_units() > 0 ? compute_units() : 256) &&
                               (g.k_per_split >= 20 * 64 || (splits > 1 && g.k_per_split >= 8 * 64));
            if (env_int("AGH_GEMM_RING", alone ? 4 : 2) == 4)
                return launch_one_dl<BP, BQ, WGP, WGQ, LP, LQ, 4>(g, splits);
        }
        // 128 x 256 and 256 x 128: three stages of 48 KB (a CU holds one such workgroup either way; 3 to 10 % faster than
        // two at every size measured, 2048^3 to 8192^3)
        return launch_one_dl<BP, BQ, WGP, WGQ, LP, LQ, BP * BQ == 128 * 256 ? 3 : 2>(g, splits);
    }
}
#endif

#ifdef AGH_GEMM_WITH_F32_DIRECT
// direct-to-LDS f32 kernel for 64 x 64 tiles (agh_gemm_f32_dl.h)
template <int TP, int TQ, int NS, int LP, int LQ, int KS = 1>
int launch_f32_dl(const Args &g, int splits) {
    if constexpr (KS == 1 && TP * TQ <= 4) {
        // a grid that gives a CU one workgroup at most: eight waves, every k-tile split between two (AGH_GEMM_KSPLIT=0|1
        // forbids / forces it)
        const int64_t wgs = (int64_t)g.tiles_p * g.tiles_q * splits * g.batch;
        const int ks = env_int("AGH_GEMM_KSPLIT", wgs <= (compute_units() > 0 ? compute_units() : 256) ? 1 : 0);
        if (ks) return launch_f32_dl<TP, TQ, NS, LP, LQ, 2>(g, splits);
    }
    auto kern = gemm_f32_dl_kernel<TP, TQ, NS, LP, LQ, KS>;
    constexpr size_t smem = F32DlGeo<TP, TQ, NS, LP, LQ>::SMEM_BYTES;
    static bool attr_done = false;
    if (!attr_done) {
        if (smem > 48 * 1024)
            AGH_HIP(hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
        attr_done = true;
    }
    dim3 grid((unsigned)(g.tiles_p * g.tiles_q), (unsigned)splits, (unsigned)g.batch);
    hipLaunchKernelGGL(kern, grid, dim3(256 * KS), smem, stream(), g);
    AGH_LAUNCH_CHECK("gemm kernel launch");
    return AGH_OK;
}
#endif

template <typename T, int BP, int BQ, int WGP, int WGQ, bool SCALAR_OK>
int launch_loaders(const Args &g, int splits, int lp, int lq, bool direct) {
#ifdef AGH_GEMM_WITH_F32_DIRECT
    if constexpr (std::is_same<T, float>::value && BP % 64 == 0 && BQ % 64 == 0) {
        // both operands vector-loadable (any k: a last k-tile shorter than 32 is loaded with zeros behind k = K)
        // (AGH_GEMM_DIRECT=0 forces the register-staged kernel).  64 x 64: a ring of four stages, one or two
        // workgroups per CU; 128 x 128: two stages (a k-tile is four times as long), two workgroups per CU; the
        // larger tiles: two stages, one workgroup per CU.
        constexpr int TPW = BP / 64, TQW = BQ / 64, NS = BP == 64 ? 4 : 2;
        if (lp != LD_S && lq != LD_S && g.K > 0 && env_int("AGH_GEMM_DIRECT", 1) != 0) {
            switch (lp * 3 + lq) {
                case LD_K * 3 + LD_K: return launch_f32_dl<TPW, TQW, NS, LD_K, LD_K>(g, splits);
                case LD_K * 3 + LD_R: return launch_f32_dl<TPW, TQW, NS, LD_K, LD_R>(g, splits);
                case LD_R * 3 + LD_K: return launch_f32_dl<TPW, TQW, NS, LD_R, LD_K>(g, splits);
                case LD_R * 3 + LD_R: return launch_f32_dl<TPW, TQW, NS, LD_R, LD_R>(g, splits);
                default: break;
            }
        }
    }
#endif
#ifdef AGH_GEMM_WITH_BF16_DIRECT
    if constexpr (std::is_same<T, uint16_t>::value && (!SCALAR_OK || (BP == 64 && BQ == 64))) {
        if (direct && lp != LD_S && lq != LD_S) {
            switch (lp * 3 + lq) {
                case LD_K * 3 + LD_K: return launch_dl_ring<BP, BQ, WGP, WGQ, LD_K, LD_K>(g, splits);
                case LD_K * 3 + LD_R: return launch_dl_ring<BP, BQ, WGP, WGQ, LD_K, LD_R>(g, splits);
                case LD_R * 3 + LD_K: return launch_dl_ring<BP, BQ, WGP, WGQ, LD_R, LD_K>(g, splits);
                case LD_R * 3 + LD_R: return launch_dl_ring<BP, BQ, WGP, WGQ, LD_R, LD_R>(g, splits);
                default: break;
            }
        }
    }
#endif
    switch (lp * 3 + lq) {
        case LD_K * 3 + LD_K: return launch_one<T, BP, BQ, WGP, WGQ, LD_K, LD_K>(g, splits);
        case LD_K * 3 + LD_R: return launch_one<T, BP, BQ, WGP, WGQ, LD_K, LD_R>(g, splits);
        case LD_R * 3 + LD_K: return launch_one<T, BP, BQ, WGP, WGQ, LD_R, LD_K>(g, splits);
        case LD_R * 3 + LD_R: return launch_one<T, BP, BQ, WGP, WGQ, LD_R, LD_R>(g, splits);
        default: break;
    }
    if constexpr (SCALAR_OK) {
        switch (lp * 3 + lq) {
            case LD_K * 3 + LD_S: return launch_one<T, BP, BQ, WGP, WGQ, LD_K, LD_S>(g, splits);
            case LD_R * 3 + LD_S: return launch_one<T, BP, BQ, WGP, WGQ, LD_R, LD_S>(g, splits);
            case LD_S * 3 + LD_K: return launch_one<T, BP, BQ, WGP, WGQ, LD_S, LD_K>(g, splits);
            case LD_S * 3 + LD_R: return launch_one<T, BP, BQ, WGP, WGQ, LD_S, LD_R>(g, splits);
            case LD_S * 3 + LD_S: return launch_one<T, BP, BQ, WGP, WGQ, LD_S, LD_S>(g, splits);
            default: break;
        }
    }
    return fail(AGH_EINVAL, "gemm: no kernel for loader pair (%d,%d)", lp, lq);
}

template <typename T>
int launch_cfg(int cfg, const Args &g, int splits, int lp, int lq, bool direct) {
    switch (cfg) {
        case 0: return launch_loaders<T, 256, 256, 2, 2, false>(g, splits, lp, lq, direct);
        case 1: return launch_loaders<T, 128, 256, 2, 2, false>(g, splits, lp, lq, direct);
        case 2: return launch_loaders<T, 256, 128, 2, 2, false>(g, splits, lp, lq, direct);
        case 3: return launch_loaders<T, 128, 128, 2, 2, false>(g, splits, lp, lq, direct);
        case 4: return launch_loaders<T, 64, 64, 2, 2, true>(g, splits, lp, lq, direct);
        case 5: return launch_loaders<T, 32, 128, 1, 4, true>(g, splits, lp, lq, false);
        case 6: return launch_loaders<T, 128, 32, 4, 1, true>(g, splits, lp, lq, false);
        default: return fail(AGH_EINVAL, "gemm: bad tile config %d", cfg);
    }
}

inline bool aligned(const void *p, size_t a) { return ((uintptr_t)p % a) == 0; }

// Which loader can serve an operand seen as NR rows x K with element strides (rs, ks).
template <typename T>
int pick_loader(const void *base, int64_t rs, int64_t ks, int NR, int K) {
    constexpr int EPC = Geo<T>::EPC;
    if (!aligned(base, 16)) return LD_S;
    if (ks == 1 && K % EPC == 0 && (rs % EPC == 0 || NR == 1)) return LD_K;
    if (rs == 1 && NR % EPC == 0 && (ks % EPC == 0 || K == 1)) return LD_R;
    return LD_S;
}

// Optional override for experiments: AGH_GEMM_CFG=<config id>, AGH_GEMM_SPLITS=<n>.
inline int env_int(const char *name, int dflt) {
    const char *s = getenv(name);
    return (s && *s) ? atoi(s) : dflt;
}

template <typename T>
int gemm_entry(const char *name, int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a,
               int64_t rsa, int64_t csa, const void *b, int64_t off_b, int64_t rsb, int64_t csb, float beta, void *c,
               int64_t off_c, int64_t rsc, int64_t csc, const void *bias, int64_t off_bias, int64_t bias_stride,
               int act, int64_t batch = 1, int64_t batch_a = 0, int64_t batch_b = 0, int64_t batch_c = 0,
               bool fixed_scratch = false) {
    AGH_API_ENTER();
    if (m < 0 || k < 0 || n < 0 || batch < 0) return fail(AGH_EINVAL, "%s: negative dimension", name);
    if (batch > 65535) return fail(AGH_ERANGE, "%s: batch count above 65535", name);
    if (batch == 0) return AGH_OK;
    const int64_t lim = ((int64_t)1 << 31) - 512;
    if (m > lim || k > lim || n > lim) return fail(AGH_ERANGE, "%s: dimension does not fit 31 bits", name);
    if (act != AGH_ACT_NONE && act != AGH_ACT_RELU) return fail(AGH_EINVAL, "%s: unknown activation %d", name, act);
    if (m == 0 || n == 0) return AGH_OK;
    if (!c) return fail(AGH_ENULL, "%s: null c", name);
    if (k > 0 && (!a || !b)) return fail(AGH_ENULL, "%s: null a or b", name);
    if (m > 1 && rsc == 0) return fail(AGH_EINVAL, "%s: c row stride is 0", name);
    if (n > 1 && csc == 0) return fail(AGH_EINVAL, "%s: c column stride is 0", name);
    constexpr int EPC = Geo<T>::EPC;
    constexpr int BK = 8 * EPC;

    const T *A = (const T *)a + off_a;
    const T *B = (const T *)b + off_b;
    T *C = (T *)c + off_c;

    Args g;
    memset(&g, 0, sizeof(g));
    // p runs along C's unit-stride axis when it has one (rows of C otherwise: p = n axis)
    const bool p_is_n = !(rsc == 1 && csc != 1);
    if (p_is_n) {
        g.P = B; g.ps = csb; g.pk = rsb; g.NP = (int)n;
        g.Q = A; g.qs = rsa; g.qk = csa; g.NQ = (int)m;
        g.dp = csc; g.dq = rsc;
        g.bias_on_p = 1;
        g.batch_p = batch_b; g.batch_q = batch_a;
    } else {
        g.P = A; g.ps = rsa; g.pk = csa; g.NP = (int)m;
        g.Q = B; g.qs = csb; g.qk = rsb; g.NQ = (int)n;
        g.dp = rsc; g.dq = csc;
        g.bias_on_p = 0;
        g.batch_p = batch_a; g.batch_q = batch_b;
    }
    g.D = C;
    g.batch = (int)batch;
    g.batch_d = batch_c;
    g.K = (int)k;
    g.alpha = alpha;
    g.beta = beta;
    g.has_bias = bias != nullptr;
    g.bias = bias ? (const void *)((const T *)bias + off_bias) : nullptr;
    g.bias_stride = bias_stride;
    g.act = act;
    g.NPpad = (g.NP + 3) & ~3;

    int lp = k > 0 ? pick_loader<T>(g.P, g.ps, g.pk, g.NP, g.K) : LD_S;
    int lq = k > 0 ? pick_loader<T>(g.Q, g.qs, g.qk, g.NQ, g.K) : LD_S;
    // every matrix of a batch must satisfy the same alignment as the first
    const bool batch_aligned = batch == 1 || (g.batch_p % EPC == 0 && g.batch_q % EPC == 0);
    if (!batch_aligned) lp = lq = LD_S;
    const bool any_scalar = (lp == LD_S || lq == LD_S);
    const bool vec_store = g.dp == 1 && g.NP % 4 == 0 && (g.dq % 4 == 0 || g.NQ == 1) && aligned(C, 4 * sizeof(T)) &&
                           (batch == 1 || g.batch_d % 4 == 0);

#ifdef AGH_GEMM_WITH_F32_SMALL
    if constexpr (sizeof(T) == 4) {
        const int rc = gemm_f32_small_try(g, lp, lq, vec_store, batch);
        if (rc != 1) return rc;
    }
#endif

    // ---- tile shape: minimise (rounds of workgroups) x (tile area) / efficiency ----
    const int cus = compute_units() > 0 ? compute_units() : 256;
    // (any k: a last k-tile shorter than 64 is loaded with zeros behind k = K)
    const bool direct_ok = sizeof(T) == 2 && !any_scalar && g.K > 0 && env_int("AGH_GEMM_DIRECT", 1) != 0;
    int best = -1;
    double best_cost = 0;
    for (int i = 0; i < kNumCfgs; ++i) {
        const TileCfg &t = kCfgs[i];
        if (any_scalar && !t.scalar_ok) continue;
        const int64_t tiles = (int64_t)((g.NP + t.bp - 1) / t.bp) * ((g.NQ + t.bq - 1) / t.bq) * batch;
        if (tiles > 0x7FFFFFFF) continue;
        // a CU works through ceil(tiles / CUs) tiles; co-resident workgroups share its MFMA rate
        const int64_t rounds = (tiles + cus - 1) / cus;
        // where the direct-to-LDS bf16 kernel applies (the four large tiles), the register-staged small tiles
        // are a poor second: measured 2x slower at 1024^3 (16.4 us against 8.9 us) although they put four times as
        // many CUs to work
        double eff = (direct_ok && !kCfgs[i].scalar_ok) || !direct_ok ? t.eff : t.eff * 0.25;
        const bool bf16_direct64 = direct_ok && t.bp == 64 && t.bq == 64;
        // the 64 x 64 direct tile is measured at 0.8 of the 256 x 256 tile's rate per CU (3072^3: 118 TFLOP/s, where
        // 144 tiles of 256 x 256 leave 112 CUs idle)
        // f32: the 64 x 64 and 128 x 128 tiles have direct-to-LDS kernels (agh_gemm_f32_dl.h)
        const bool f32_dl_ok = sizeof(T) == 4 && !any_scalar && g.K > 0 && env_int("AGH_GEMM_DIRECT", 1) != 0;
        const bool f32_direct = f32_dl_ok && t.bp == 64 && t.bq == 64;
        if (f32_direct) eff = 0.80;
        if (f32_dl_ok && t.bp == 128 && t.bq == 128) eff = 0.95;  // 4096^3: 135 TFLOP/s, the 256 x 256 tile's rate
        // a tile's prologue and epilogue cost about four k-tiles of time when the CU holds one workgroup, next
        // to nothing when a second workgroup multiplies meanwhile: decides short-k shapes (conv GEMM, k = 576).
        // The f32 direct kernel's k-tile is short (sixteen MFMAs a wave): filling its four-stage ring and storing
        // the tile cost about six of them (at k = 576 the 128 x 128 tile is 9 % faster, from k = 1536 on slower).
        const double kt = (double)((g.K + BK - 1) / BK);
        eff *= kt / (kt + (f32_direct ? 6.0 : t.wgs_per_cu == 1 ? 4.0 : 0.5));
        double cost = (double)rounds * t.bp * t.bq / eff;
        // many small tiles do not run in lockstep rounds: a CU takes the next tile when one of its two is done, and the
        // launch ends a fraction of a tile after tiles / CUs tile times (3584^3 on 64 x 64 tiles: 12.25 tiles a CU,
        // 12.5 tile times measured, 790 us against 871 us on the 256 x 256 tile)
        if (f32_direct && tiles >= 4 * (int64_t)cus) cost = ((double)tiles / cus + 0.25) * t.bp * t.bq / eff;
        // bf16 direct-to-LDS tiles: a full chip of them runs at the power limit, where the rate depends on the tile
        // shape (bigger tiles move fewer operand bytes per flop) and not on how many CUs take part, while a
        // launch that leaves CUs idle runs the busy ones at a higher clock.  Measured per k-tile of a 256 x 256
        // tile: 1.32 us with 256 workgroups (8192^3, 4096^3), 0.97 us with 144 (3072^3).  The cost is summed over
        // rounds of co-resident workgroups, each round at the lower of the two rates.
        if (direct_ok && !t.scalar_ok) {
            // rates relative to a 256 x 256 workgroup on a full chip.  kAlone: a 128 x 128 workgroup with a CU to itself
            // (2048^3: 22.8 us on two LDS stages, 17.9 us on the ring of four a launch of at most one workgroup per CU
            // and 20 k-tiles or more takes) against two sharing it
            static const double kUnthrottled[4] = {1.36, 1.0, 1.0, 0.946}, kAtPowerLimit[4] = {1.0, 0.855, 0.855, 0.85};
            const double kAlone[4] = {1.36, 1.0, 1.0, tiles <= cus && kt >= 20 ? 0.75 : 0.59};
            const int64_t slots = (int64_t)cus * t.wgs_per_cu, rest = tiles % slots;
            const double area = (double)t.bp * t.bq;
            // a round of n co-resident workgroups: each CU at its unthrottled rate or at its share of the chip's
            // power-limited rate, whichever is lower
            auto round_cost = [&](int64_t n) {
                const bool shared = n > cus;
                const double rate = std::min(shared ? kUnthrottled[i] : kAlone[i],
                                             kAtPowerLimit[i] * cus / (double)std::min<int64_t>(n, cus));
                return (shared ? t.wgs_per_cu : 1) * area / rate;
            };
            cost = ((double)(tiles / slots) * round_cost(slots) + (rest ? round_cost(rest) : 0.0)) *
                   (kt + (t.wgs_per_cu == 1 ? 4.0 : 2.0)) / kt;
        }
        // The 64 x 64 direct-to-LDS bf16 tile: a CU's fill path from L2 bounds it (16 KB per k-tile against the 32 KB a
        // 128 x 128 tile moves for four times the flop), so a tile takes about half the time of a 128 x 128 one; filling
        // its ring and storing the tile cost about six of its k-tiles.
        if (bf16_direct64) {
            const int64_t slots = (int64_t)cus * 2;
            const double per_tile = (double)t.bp * t.bq / (tiles <= cus ? kDirect64Alone : kDirect64Shared);
            cost = (double)((tiles + slots - 1) / slots) * (tiles <= cus ? 1 : 2) * per_tile * (kt + 6.0) / kt;
        }
        if (best < 0 || cost < best_cost) { best = i; best_cost = cost; }
    }
    best = env_int("AGH_GEMM_CFG", best);
    if (best < 0 || best >= kNumCfgs || (any_scalar && !kCfgs[best].scalar_ok))
        return fail(AGH_ERANGE, "%s: no tile configuration for this shape", name);
    const TileCfg &t = kCfgs[best];
    g.tiles_p = (g.NP + t.bp - 1) / t.bp;
    g.tiles_q = (g.NQ + t.bq - 1) / t.bq;

    // ---- split-K when the tile grid cannot fill the chip and k is long ----
    const int64_t tiles = (int64_t)g.tiles_p * g.tiles_q * batch;
    const int64_t slots = (int64_t)cus;
    int splits = 1;
    const int ktiles = (g.K + BK - 1) / BK;
    if (tiles * 2 <= slots && ktiles >= 32 && batch == 1) {
        int64_t s = slots / tiles;
        // at least four k-tiles a split; twelve for the bf16 128 x 128 direct tile, whose four-stage ring makes fewer,
        // longer splits the better trade (128x4096x4096: 17.0-17.2 us in 4 to 6 splits, 19.5 in 8)
        const int kmin = direct_ok && best == 3 ? 12 : 4;
        if (s > ktiles / kmin) s = ktiles / kmin;
        if (s > 256) s = 256;
        if (s > 1) splits = (int)s;
    }
    if (batch == 1) splits = env_int("AGH_GEMM_SPLITS", splits);
    if (splits < 1) splits = 1;
    if (splits > ktiles && ktiles > 0) splits = ktiles;
    if (ktiles == 0) splits = 1;
    int tiles_per_split = ktiles > 0 ? (ktiles + splits - 1) / splits : 1;
    splits = ktiles > 0 ? (ktiles + tiles_per_split - 1) / tiles_per_split : 1;
    g.k_per_split = tiles_per_split * BK;

    // bf16 with both operands vector-loadable takes the
    // direct-to-LDS kernel (AGH_GEMM_DIRECT=0 forces the register-staged one)
    const bool direct = direct_ok;

    if (splits > 1) {
        void *ws = nullptr;
        const size_t bytes = (size_t)splits * g.NQ * g.NPpad * sizeof(float);
        if (int rc = fixed_scratch ? static_workspace(bytes, &ws) : workspace(bytes, &ws)) return rc;
        g.ws = (float *)ws;
        g.store_mode = ST_SPLITK;
        if (int rc = launch_cfg<T>(best, g, splits, lp, lq, direct)) return rc;
        const size_t total = (size_t)g.NQ * g.NP;
        int lanes = 1;  // threads per output element: about eight partials each
        while (lanes < 16 && lanes * 16 <= splits) lanes *= 2;
        if (lanes == 1 && vec_store && g.NPpad == g.NP) {
            hipLaunchKernelGGL(splitk_reduce_vec4_kernel<T>, dim3((unsigned)((total / 4 + 255) / 256)), dim3(256), 0,
                               stream(), g, splits);
            AGH_LAUNCH_CHECK("split-K reduce launch");
            return AGH_OK;
        }
        const size_t blocks = (total * lanes + 255) / 256;
        if (blocks > 0x7FFFFFFFull) return fail(AGH_ERANGE, "%s: output too large for split-K", name);
        hipLaunchKernelGGL(splitk_reduce_kernel<T>, dim3((unsigned)blocks), dim3(256), 0, stream(), g, splits, lanes);
        AGH_LAUNCH_CHECK("split-K reduce launch");
        return AGH_OK;
    }
    g.store_mode = vec_store ? ST_VEC : ST_SCALAR;
    // the direct-to-LDS kernel can transpose its output tile through LDS and store full 16-byte
    // chunks when nothing has to be read back from C
    if (direct && best <= 4 && vec_store && beta == 0.0f && g.NP % 8 == 0 && (g.dq % 8 == 0 || g.NQ == 1) &&
        aligned(C, 16) && (batch == 1 || g.batch_d % 8 == 0))
        g.store_mode = ST_STAGED;
    return launch_cfg<T>(best, g, 1, lp, lq, direct);
}

}  // namespace gemm
}  // namespace agh

// bf16 GEMM entry points (v_mfma_f32_32x32x16_bf16, f32 accumulate, one RNE at the end).
#define AGH_GEMM_WITH_BF16_DIRECT 1
#include "agh_gemm_host.h"

extern "C" {

int agh_gemm_bf16(int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                  const void *b, int64_t off_b, int64_t rsb, int64_t csb, float beta, void *c, int64_t off_c,
                  int64_t rsc, int64_t csc) {
    return agh::gemm::gemm_entry<uint16_t>("agh_gemm_bf16", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb, csb, beta,
                                           c, off_c, rsc, csc, nullptr, 0, 0, AGH_ACT_NONE);
}

int agh_gemm_bf16_noalloc(int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a, int64_t rsa,
                          int64_t csa, const void *b, int64_t off_b, int64_t rsb, int64_t csb, float beta, void *c,
                          int64_t off_c, int64_t rsc, int64_t csc) {
    // same planning and kernels; split-K partials go to the library's fixed scratch buffer
    return agh::gemm::gemm_entry<uint16_t>("agh_gemm_bf16_noalloc", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb, csb,
                                           beta, c, off_c, rsc, csc, nullptr, 0, 0, AGH_ACT_NONE, 1, 0, 0, 0, true);
}

int agh_gemm_bf16_bias_act(int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a, int64_t rsa,
                           int64_t csa, const void *b, int64_t off_b, int64_t rsb, int64_t csb, float beta, void *c,
                           int64_t off_c, int64_t rsc, int64_t csc, const void *bias, int64_t off_bias,
                           int64_t bias_stride, int act) {
    return agh::gemm::gemm_entry<uint16_t>("agh_gemm_bf16_bias_act", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb,
                                           csb, beta, c, off_c, rsc, csc, bias, off_bias, bias_stride, act);
}

int agh_gemm_bf16_batched(int64_t batch, int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a,
                          int64_t rsa, int64_t csa, int64_t batch_stride_a, const void *b, int64_t off_b, int64_t rsb,
                          int64_t csb, int64_t batch_stride_b, float beta, void *c, int64_t off_c, int64_t rsc,
                          int64_t csc, int64_t batch_stride_c, const void *bias, int64_t off_bias, int64_t bias_stride,
                          int act) {
    return agh::gemm::gemm_entry<uint16_t>("agh_gemm_bf16_batched", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb, csb,
                                       beta, c, off_c, rsc, csc, bias, off_bias, bias_stride, act, batch,
                                       batch_stride_a, batch_stride_b, batch_stride_c);
}

}  // extern "C"

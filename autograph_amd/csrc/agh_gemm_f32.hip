// f32 GEMM entry points (v_mfma_f32_32x32x2_f32: full f32 multiplies and accumulation).
#define AGH_GEMM_WITH_F32_DIRECT
#define AGH_GEMM_WITH_F32_SMALL
#include "agh_gemm_f32_dl.h"
#include "agh_gemm_f32_small.h"
#include "agh_gemm_host.h"

extern "C" {

int agh_gemm_f32(int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a, int64_t rsa, int64_t csa,
                 const void *b, int64_t off_b, int64_t rsb, int64_t csb, float beta, void *c, int64_t off_c,
                 int64_t rsc, int64_t csc) {
    return agh::gemm::gemm_entry<float>("agh_gemm_f32", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb, csb, beta, c,
                                        off_c, rsc, csc, nullptr, 0, 0, AGH_ACT_NONE);
}

int agh_gemm_f32_bias_act(int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a, int64_t rsa,
                          int64_t csa, const void *b, int64_t off_b, int64_t rsb, int64_t csb, float beta, void *c,
                          int64_t off_c, int64_t rsc, int64_t csc, const void *bias, int64_t off_bias,
                          int64_t bias_stride, int act) {
    return agh::gemm::gemm_entry<float>("agh_gemm_f32_bias_act", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb, csb,
                                        beta, c, off_c, rsc, csc, bias, off_bias, bias_stride, act);
}

int agh_gemm_f32_batched(int64_t batch, int64_t m, int64_t k, int64_t n, float alpha, const void *a, int64_t off_a,
                          int64_t rsa, int64_t csa, int64_t batch_stride_a, const void *b, int64_t off_b, int64_t rsb,
                          int64_t csb, int64_t batch_stride_b, float beta, void *c, int64_t off_c, int64_t rsc,
                          int64_t csc, int64_t batch_stride_c, const void *bias, int64_t off_bias, int64_t bias_stride,
                          int act) {
    return agh::gemm::gemm_entry<float>("agh_gemm_f32_batched", m, k, n, alpha, a, off_a, rsa, csa, b, off_b, rsb, csb,
                                       beta, c, off_c, rsc, csc, bias, off_bias, bias_stride, act, batch,
                                       batch_stride_a, batch_stride_b, batch_stride_c);
}

}  // extern "C"

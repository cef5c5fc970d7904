// Launch wrappers of the direct-to-LDS bf16 GEMM kernels.  Each agh_gemm_bf16_dl_<tile>.hip includes
// this header and instantiates the four loader pairs of one tile shape.
#pragma once
#include "agh_gemm_bf16_dl.h"

namespace agh {
namespace gemm {

template <int BP, int BQ, int WGP, int WGQ, int LP, int LQ, int NS>
int launch_one_dl(const Args &g, int splits) {
    dim3 grid((unsigned)(g.tiles_p * g.tiles_q), (unsigned)splits, (unsigned)g.batch);
    // the LDS stages are static
    if (g.store_mode == ST_STAGED)
        hipLaunchKernelGGL((gemm_bf16_dl_kernel<BP, BQ, WGP, WGQ, LP, LQ, true, NS>), grid, dim3(WGP * WGQ * 64), 0, stream(), g);
    else
        hipLaunchKernelGGL((gemm_bf16_dl_kernel<BP, BQ, WGP, WGQ, LP, LQ, false, NS>), grid, dim3(WGP * WGQ * 64), 0, stream(), g);
    AGH_LAUNCH_CHECK("gemm (direct-to-LDS) kernel launch");
    return AGH_OK;
}

#define AGH_DL_INSTANTIATE(BP, BQ, WGP, WGQ, NS)                                          \
    template int launch_one_dl<BP, BQ, WGP, WGQ, LD_K, LD_K, NS>(const Args &, int);      \
    template int launch_one_dl<BP, BQ, WGP, WGQ, LD_K, LD_R, NS>(const Args &, int);      \
    template int launch_one_dl<BP, BQ, WGP, WGQ, LD_R, LD_K, NS>(const Args &, int);      \
    template int launch_one_dl<BP, BQ, WGP, WGQ, LD_R, LD_R, NS>(const Args &, int);

}  // namespace gemm
}  // namespace agh

// Direct-to-LDS bf16 GEMM kernels, 256x256 tile, 2x2 waves: all four loader pairs.
#include "agh_gemm_bf16_dl_launch.h"

namespace agh {
namespace gemm {
AGH_DL_INSTANTIATE(256, 256, 2, 2, 2)
}  // namespace gemm
}  // namespace agh

// Direct-to-LDS bf16 GEMM kernels, 128x128 tile, 2x2 waves: all four loader pairs.
#include "agh_gemm_bf16_dl_launch.h"

namespace agh {
namespace gemm {
AGH_DL_INSTANTIATE(128, 128, 2, 2, 2)
}  // namespace gemm
}  // namespace agh

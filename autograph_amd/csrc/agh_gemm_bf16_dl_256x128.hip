// Direct-to-LDS bf16 GEMM kernels, 256x128 tile, 2x2 waves, three LDS stages: all four loader pairs.
#include "agh_gemm_bf16_dl_launch.h"

namespace agh {
namespace gemm {
AGH_DL_INSTANTIATE(256, 128, 2, 2, 3)
}  // namespace gemm
}  // namespace agh

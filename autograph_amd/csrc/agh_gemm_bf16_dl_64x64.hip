// Direct-to-LDS bf16 GEMM kernels, 64x64 tile, 2x2 waves, a ring of four LDS stages: all four loader pairs.
#include "agh_gemm_bf16_dl_launch.h"

namespace agh {
namespace gemm {
AGH_DL_INSTANTIATE(64, 64, 2, 2, 4)
}  // namespace gemm
}  // namespace agh

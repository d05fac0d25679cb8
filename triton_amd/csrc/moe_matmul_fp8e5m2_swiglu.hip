// Instantiates the tiled MXFP4 grouped matmul kernels (moe_matmul_impl.h) with the fused SwiGLU epilogue.
#include "moe_matmul_impl.h"

namespace tamd {
int tiled_mm_swiglu_fp8e5m2(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  return dispatch_x16_act<TAMD_FP8_E5M2, TAMD_ACT_SWIGLU>(a, block_m, grid_m, st);
}
}  // namespace tamd

// Instantiates the grouped matmul kernels for float8_e4m3fn activations: the tiled kernel built on the scaled MFMA
// (moe_matmul_impl.h) and, for row blocks of 16, the streaming kernel (moe_matmul_stream.h) with the rows expanded
// to bf16 as they are loaded.
#include "moe_matmul_stream.h"

namespace tamd {
int dispatch_mm_fp8e4m3(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  if (block_m == 0 && a.M <= 256 && stream16_applicable(a)) {
    // dense with few rows: row blocks of 16 through the streaming kernel (every CU busy, weights re-read from L2)
    block_m = 16;
    grid_m = ((a.M + 15) / 16) * a.n_experts;
  }
  if (block_m == 16 && stream16_applicable(a)) {
    if (a.activation == TAMD_ACT_SWIGLU) return launch_stream16<TAMD_BF16, TAMD_ACT_SWIGLU, true>(a, grid_m, st);
    return launch_stream16<TAMD_BF16, TAMD_ACT_NONE, true>(a, grid_m, st);
  }
  return dispatch_x16<TAMD_FP8_E4M3>(a, block_m, grid_m, st);
}
}  // namespace tamd

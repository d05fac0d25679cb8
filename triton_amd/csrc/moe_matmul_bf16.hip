// Instantiates the grouped matmul kernels for one activation type: the streaming kernel for row blocks of
// 16 (moe_matmul_stream.h), the tiled MXFP4 kernel for everything else (moe_matmul_impl.h), and the kernel for
// unquantised weights of the same type (moe_matmul_dense.h).
#include "moe_matmul_dense.h"
#include "moe_matmul_stream.h"

namespace tamd {
int dispatch_mm_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  if (block_m == 0 && a.M <= 256 && stream16_applicable(a)) {
    // dense with few rows: row blocks of 16 through the streaming kernel (every CU busy, weights re-read from L2)
    block_m = 16;
    grid_m = ((a.M + 15) / 16) * a.n_experts;
  }
  if (block_m == 16 && stream16_applicable(a)) {
    if (a.activation == TAMD_ACT_SWIGLU) return launch_stream16<TAMD_BF16, TAMD_ACT_SWIGLU>(a, grid_m, st);
    return launch_stream16<TAMD_BF16, TAMD_ACT_NONE>(a, grid_m, st);
  }
  return dispatch_x16<TAMD_BF16>(a, block_m, grid_m, st);
}

int dispatch_mm_w16_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  return dispatch_w16<TAMD_BF16>(a, block_m, grid_m, st);
}
}  // namespace tamd

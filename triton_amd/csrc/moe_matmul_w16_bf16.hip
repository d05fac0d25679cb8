// Instantiates the grouped matmul kernel for unquantised bf16 weights (moe_matmul_dense.h).
#include "moe_matmul_dense.h"

namespace tamd {
int dispatch_mm_w16_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  return dispatch_w16<TAMD_BF16>(a, block_m, grid_m, st);
}
}  // namespace tamd

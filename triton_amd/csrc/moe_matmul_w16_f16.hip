// Instantiates the grouped matmul kernel for unquantised f16 weights (moe_matmul_dense.h).
#include "moe_matmul_dense.h"

namespace tamd {
int dispatch_mm_w16_f16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  return dispatch_w16<TAMD_F16>(a, block_m, grid_m, st);
}
}  // namespace tamd

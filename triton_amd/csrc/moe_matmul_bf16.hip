// Instantiates the grouped matmul kernels of moe_matmul_impl.h for one activation type.
#include "moe_matmul_impl.h"

namespace tamd {
int dispatch_mm_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  return dispatch_x16<TAMD_BF16>(a, block_m, grid_m, st);
}
}  // namespace tamd

// Instantiates the tiled MXFP4 grouped matmul kernels (moe_matmul_impl.h) for fp16 activations with the plain epilogue
// (the SwiGLU ones are compiled in moe_matmul_f16_swiglu.hip) and routes row blocks of 16 to the streaming kernel
// (moe_matmul_stream.h), which is compiled in moe_matmul_stream_f16.hip.
#include "moe_matmul_stream.h"

namespace tamd {
int dispatch_mm_f16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  if (block_m == 0 && dense_prefers_k_groups(a)) {
    block_m = 32;
    grid_m = ((a.M + 31) / 32) * a.n_experts;
  } else if (block_m == 0 && a.M <= 256 && stream16_applicable(a)) {
    // dense with few rows: row blocks of 16 through the streaming kernel (every CU busy, weights re-read from L2)
    block_m = 16;
    grid_m = ((a.M + 15) / 16) * a.n_experts;
  }
  if (block_m == 16 && stream16_applicable(a)) return stream_mm_f16(a, grid_m, st);
  if (a.activation == TAMD_ACT_SWIGLU) return tiled_mm_swiglu_f16(a, block_m, grid_m, st);
  return dispatch_x16_act<TAMD_F16, TAMD_ACT_NONE>(a, block_m, grid_m, st);
}
}  // namespace tamd

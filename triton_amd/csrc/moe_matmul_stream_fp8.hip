// Instantiates the streaming kernel for row blocks of 16 (moe_matmul_stream.h) for float8_e4m3fn activations (expanded to bf16 as they are loaded).
#include "moe_matmul_stream.h"

namespace tamd {
int stream_mm_fp8e4m3(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  if (a.activation == TAMD_ACT_SWIGLU) return launch_stream16<TAMD_BF16, TAMD_ACT_SWIGLU, 1>(a, grid_m, st);
  return launch_stream16<TAMD_BF16, TAMD_ACT_NONE, 1>(a, grid_m, st);
}
}  // namespace tamd

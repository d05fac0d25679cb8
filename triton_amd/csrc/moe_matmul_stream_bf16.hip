// Instantiates the streaming kernel for row blocks of 16 (moe_matmul_stream.h) for bf16 activations.
#include "moe_matmul_stream.h"

namespace tamd {
int stream_mm_bf16(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  if (a.activation == TAMD_ACT_SWIGLU) return launch_stream16<TAMD_BF16, TAMD_ACT_SWIGLU>(a, grid_m, st);
  return launch_stream16<TAMD_BF16, TAMD_ACT_NONE>(a, grid_m, st);
}
}  // namespace tamd

// C ABI entry point of the grouped / dense matmul: validation and dispatch.  The kernels live in
// moe_matmul_impl.h and are instantiated once per activation type in moe_matmul_{bf16,f16,fp8}.hip
// (separate translation units so that they compile in parallel).
#include "common.h"

namespace tamd {
int dispatch_mm_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int dispatch_mm_f16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int dispatch_mm_fp8e4m3(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int dispatch_mm_fp8e5m2(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int dispatch_mm_w16_bf16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
int dispatch_mm_w16_f16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st);
}  // namespace tamd

using namespace tamd;

extern "C" int tamd_matmul(const tamd_matmul_args *args, void *stream) {
  if (!args) return TAMD_E_INVALID;
  tamd_matmul_args a = *args;
  if (a.M < 0 || a.N < 0 || a.K < 0 || a.n_experts < 1) return TAMD_E_INVALID;
  if (a.n_experts == 1) a.w_stride_e = a.w_mx_stride_e = a.bias_stride_e = 0;  // never used; keeps the alignment checks honest
  if (a.M == 0 || a.N == 0) return 0;
  // K == 0 would be a bias-only problem; no kernel is built for it, and the K loops assume at least one stage
  if (a.K == 0) return TAMD_E_UNSUPPORTED;
  if (!a.x || !a.w || !a.y) return TAMD_E_INVALID;
  if (a.activation != TAMD_ACT_NONE && a.activation != TAMD_ACT_SWIGLU) return TAMD_E_INVALID;
  if (a.activation == TAMD_ACT_SWIGLU && (a.N % 2) != 0) return TAMD_E_INVALID;
  if (a.y_mx_scale && (a.y_dtype != TAMD_FP8_E4M3 || a.y_expected_scale || a.y_actual_scale)) return TAMD_E_UNSUPPORTED;
  if (a.y_dtype != TAMD_BF16 && a.y_dtype != TAMD_F16 && a.y_dtype != TAMD_F32 && a.y_dtype != TAMD_FP8_E4M3 &&
      a.y_dtype != TAMD_FP8_E5M2)
    return TAMD_E_INVALID;
  if (a.bias && a.bias_dtype != TAMD_F32 && a.bias_dtype != TAMD_BF16 && a.bias_dtype != TAMD_F16)
    return TAMD_E_INVALID;
  const bool ragged = a.block_schedule != nullptr;
  if (ragged && (!a.slice_sizes || !a.slice_offs || a.grid_m < 0)) return TAMD_E_INVALID;
  hipStream_t st = (hipStream_t)stream;

  const bool x8 = a.x_dtype == TAMD_FP8_E4M3 || a.x_dtype == TAMD_FP8_E5M2;
  if (a.w_dtype == TAMD_MXFP4 && (a.x_dtype == TAMD_BF16 || a.x_dtype == TAMD_F16 || x8)) {
    const int esz = x8 ? 1 : 2;
    if (!a.w_mx_scale) return TAMD_E_INVALID;
    if (a.K % 32 != 0) return TAMD_E_INVALID;
    // weights / scales must be contiguous along K ("column-major" mxfp weights)
    const bool cdna4_sc = a.w_mx_layout == TAMD_SCALE_CDNA4;
    if (a.w_mx_layout != TAMD_SCALE_STRIDED && !cdna4_sc) return TAMD_E_INVALID;
    const bool w_blocks = a.w_layout == TAMD_W_CDNA4_BLOCKS;
    if (a.w_layout != TAMD_W_STRIDED && !w_blocks) return TAMD_E_INVALID;
    if (w_blocks) {
      // only the expert pitch is used; a matrix is ceil(N/64) x ceil(K/128) blocks of 4 KB
      a.w_stride_k = 1, a.w_stride_n = 0;
      if ((int64_t)((a.N + 63) / 64) * ((a.K + 127) / 128) * 4096 >= (int64_t)0x7FFFFF00) return TAMD_E_UNSUPPORTED;
    }
    if (a.w_stride_k != 1 || (!cdna4_sc && a.w_mx_stride_k != 1)) return TAMD_E_UNSUPPORTED;
    if (cdna4_sc && (!aligned(a.w_mx_scale, 16) || a.w_mx_stride_e % 16 != 0)) return TAMD_E_ALIGNMENT;
    if (!aligned(a.w, 16) || a.w_stride_n % 16 != 0 || a.w_stride_e % 16 != 0) return TAMD_E_ALIGNMENT;
    if (!aligned(a.x, 16) || (a.x_stride_m * esz) % 16 != 0 || (a.x_stride_z * esz) % 16 != 0) return TAMD_E_ALIGNMENT;
    // 32-bit buffer offsets: one batch of activations and one expert's weights must each span < 2 GiB
    const int64_t x_rows = a.x_rows > 0 ? a.x_rows : a.M;
    if (x_rows * a.x_stride_m * esz >= (int64_t)0x7FFFFF00 || (int64_t)a.N * a.w_stride_n >= (int64_t)0x7FFFFF00 ||
        (int64_t)a.N * (cdna4_sc ? (int64_t)(a.K / 32 + 7) : a.w_mx_stride_n) >= (int64_t)0x7FFFFF00)
      return TAMD_E_UNSUPPORTED;
    if (a.x_mx_scale) {
      // block scales of the activations: MXFP8 (e4m3 values) through the scaled MFMA only
      if (!x8) return TAMD_E_UNSUPPORTED;
      if (a.x_mx_stride_m < a.K / 32 || x_rows * a.x_mx_stride_m >= (int64_t)0x7FFFFF00) return TAMD_E_UNSUPPORTED;
    }
    int block_m, grid_m;
    if (ragged) {
      block_m = a.block_m;
      grid_m = a.grid_m;
    } else {
      // 0: the dispatcher chooses (it knows which kernels apply)
      block_m = a.force_variant;
      grid_m = block_m ? ((a.M + block_m - 1) / block_m) * a.n_experts : 0;
    }
    if (a.x_dtype == TAMD_BF16) return dispatch_mm_bf16(a, block_m, grid_m, st);
    if (a.x_dtype == TAMD_F16) return dispatch_mm_f16(a, block_m, grid_m, st);
    if (a.x_dtype == TAMD_FP8_E5M2) return dispatch_mm_fp8e5m2(a, block_m, grid_m, st);
    return dispatch_mm_fp8e4m3(a, block_m, grid_m, st);
  }
  if ((a.x_dtype == TAMD_BF16 || a.x_dtype == TAMD_F16) && a.w_dtype == a.x_dtype) {
    // unquantised weights of the activations' type
    int block_m, grid_m;
    if (ragged) {
      block_m = a.block_m;
      grid_m = a.grid_m;
    } else {
      block_m = a.force_variant;
      grid_m = block_m ? ((a.M + block_m - 1) / block_m) * a.n_experts : 0;
    }
    if (a.x_dtype == TAMD_BF16) return dispatch_mm_w16_bf16(a, block_m, grid_m, st);
    return dispatch_mm_w16_f16(a, block_m, grid_m, st);
  }
  return TAMD_E_UNSUPPORTED;
}

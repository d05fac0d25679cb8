/*
 * triton_amd C ABI — MI355X (gfx950) kernels for the quantized-MoE hot path.
 *
 * The reference (facebookexperimental/triton, python/triton_kernels) has no FFI
 * on this path: its boundary is a set of Python callables that launch Triton
 * kernels on the caller's current stream.  Each entry point below replaces one
 * such launch site and is what a ctypes / cffi / pybind binding of that site
 * would bind.  File:line citations are relative to
 * python/triton_kernels/triton_kernels/ in the reference tree.
 *
 * Conventions
 *   - every function returns int: 0 = ok, < 0 = TAMD_E_* (invalid argument or
 *     unsupported combination, nothing was launched), > 0 = hipError_t;
 *   - all pointers are device pointers unless stated; buffers are owned by the
 *     caller; the library allocates nothing and never synchronises;
 *   - `stream` is a hipStream_t passed as void*; work is enqueued on it;
 *   - strides are in elements of the pointed-to type;
 *   - entry points are re-entrant and keep no mutable global state.
 */
#ifndef TRITON_AMD_H
#define TRITON_AMD_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TAMD_VERSION 1

/* error codes (negative) */
#define TAMD_E_INVALID (-1)     /* bad shape / stride / pointer / enum */
#define TAMD_E_UNSUPPORTED (-2) /* valid in the reference, not built here */
#define TAMD_E_ALIGNMENT (-3)   /* pointer or stride not aligned as the kernel needs */
#define TAMD_E_TOO_LARGE (-4)   /* problem exceeds a fixed capacity of the entry point (see its comment) */

/* element types */
#define TAMD_F32 0
#define TAMD_F16 1
#define TAMD_BF16 2
#define TAMD_FP8_E4M3 3 /* OCP e4m3fn */
#define TAMD_FP8_E5M2 4
#define TAMD_MXFP4 5    /* two e2m1 codes per byte, even index in the low nibble */

/* encodings of the weight scales (tamd_matmul_args.w_mx_layout) */
#define TAMD_SCALE_STRIDED 0
#define TAMD_SCALE_CDNA4 1
/* encodings of MXFP4 weight codes (tamd_matmul_args.w_layout) */
#define TAMD_W_STRIDED 0
#define TAMD_W_CDNA4_BLOCKS 1

/* dequant-scale rounding of downcast_to_mxfp (numerics_details/mxfp.py:17-22) */
#define TAMD_ROUND_UP 0
#define TAMD_ROUND_DOWN 1

int tamd_version(void);
const char *tamd_error_string(int code);

/*
 * downcast_to_mxfp: replaces the launch of _downcast_to_mxfp
 * (numerics_details/mxfp.py:70-85; kernel mxfp_details/_downcast_to_mxfp.py:33-215).
 *
 * src is viewed as [nb, L, nr]; quantisation runs along the middle axis in
 * groups of 32 (L % 32 == 0).  Either src_stride_l == 1 or src_stride_r == 1.
 * out_vals gets L/2 bytes (mxfp4) contiguous along the quantised axis for every
 * (b, r): byte j of run (b, r) holds codes 2j (low nibble) and 2j+1.
 * out_scales gets L/32 e8m0 bytes per (b, r), contiguous likewise.
 * out_dtype TAMD_FP8_E4M3 / TAMD_FP8_E5M2 (MXFP8: one byte per element, clamped to the finite range and rounded to
 * nearest even, mxfp.py:313-316) is built for src_stride_l == 1 only; other layouts return TAMD_E_UNSUPPORTED.
 */
int tamd_downcast_mxfp(const void *src, int src_dtype, int64_t nb, int64_t L, int64_t nr,
                       int64_t src_stride_b, int64_t src_stride_l, int64_t src_stride_r,
                       void *out_vals, int out_dtype, int64_t val_stride_b, int64_t val_stride_r,
                       uint8_t *out_scales, int64_t scale_stride_b, int64_t scale_stride_r,
                       int rounding_mode, void *stream);

/*
 * upcast_from_mxfp: replaces the launch of _upcast_from_mxfp
 * (numerics_details/mxfp.py:174-188; kernel mxfp_details/_upcast_from_mxfp.py:252-335).
 *
 * vals / scales are laid out as tamd_downcast_mxfp writes them (runs contiguous
 * along the quantised axis, strides for b and r given).  dst is [nb, L, nr] with
 * either dst_stride_l == 1 or dst_stride_r == 1.  A scale byte of 0xFF yields
 * NaN, 0x00 multiplies by +0.0; results are clamped to the finite range of
 * dst_dtype (F32 / F16 / BF16).  val_dtype TAMD_FP8_E4M3 / TAMD_FP8_E5M2 (one byte per element; e5m2
 * infinities pass through, mxfp.py:438-440) needs dst_stride_l == 1.
 */
int tamd_upcast_mxfp(const void *vals, int val_dtype, int64_t val_stride_b, int64_t val_stride_r,
                     const uint8_t *scales, int64_t scale_stride_b, int64_t scale_stride_r,
                     void *dst, int dst_dtype, int64_t nb, int64_t L, int64_t nr,
                     int64_t dst_stride_b, int64_t dst_stride_l, int64_t dst_stride_r, void *stream);

/*
 * MXFP4 activations of the matmul (matmul.py:131-136, 772-778: a_mx_scale with e2m1 values): the reference's kernel
 * loads the packed codes itself; here the rows are widened, exactly, to float8_e4m3fn (every e2m1 number is an e4m3
 * number) and run through the MXFP8 path of tamd_matmul with the same e8m0 scales.
 * src: rows x row_bytes packed bytes (two codes each, low nibble = even index), dst: rows x 2 * row_bytes bytes.
 */
int tamd_widen_mxfp4_rows(const uint8_t *src, int64_t rows, int64_t row_bytes, int64_t src_stride, uint8_t *dst,
                          int64_t dst_stride, void *stream);

/*
 * topk forward: replaces the launch of _topk_forward (topk.py:58-67; kernel
 * topk_details/_topk_forward.py:87-147).
 *
 * x [n_rows_total, n_cols] (row stride x_stride, unit column stride), dtype
 * F32 / F16 / BF16.  For rows < n_rows: picks the k largest entries (ties: lower
 * column first), orders them by value descending, optionally replaces the
 * values by their softmax over the k picked (float32 arithmetic), writes
 * y_vals [.,k] (x dtype), y_indx [.,k] int16 and the bit matrix words
 * bits[t*bits_stride_row + w*bits_stride_word], w < ceil(n_cols/32).
 * With use_provided_indx != 0, y_indx is an input and only values / bits are made.
 * Limits: n_cols < 32768, 1 <= k <= min(n_cols, 64).
 */
int tamd_topk_forward(const void *x, int x_dtype, int64_t x_stride, int n_rows, int n_cols, int k,
                      int apply_softmax, int use_provided_indx, void *y_vals, int16_t *y_indx,
                      int64_t y_stride, uint32_t *bits, int64_t bits_stride_row,
                      int64_t bits_stride_word, void *stream);

/*
 * bitmatrix metadata: replaces sum_bitmatrix_rows + _bitmatrix_metadata_compute_stage1/2
 * (tensor_details/bitmatrix.py:110-150).
 *
 * indx: n_indx expert ids (int16 or int32 chosen by indx_is_int16), -1 = skip.
 * Outputs: col_sum int32 [n_cols]; col_sorted_indx int32 [n_indx] = positions of
 * indx ordered by expert id (stable), padded with -1; row_sorted_indx int32
 * [n_indx] = rank of each position in that order (-1 for skipped).
 * workspace: int32 scratch of tamd_bitmatrix_metadata_workspace(n_indx, n_cols)
 * elements.  Limit: n_cols <= 16384.
 */
int64_t tamd_bitmatrix_metadata_workspace(int64_t n_indx, int n_cols);
int tamd_bitmatrix_metadata(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols,
                            int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                            int32_t *workspace, void *stream);

/*
 * ragged tensor metadata: replaces _ragged_tensor_metadata_memset + _compute
 * (tensor_details/ragged_tensor.py:183-210).
 *
 * slice_sizes int32 [n_slices].  offs: int32 [6, offs_pitch]; row 0 = slice_offs
 * ([0]+cumsum), rows 1..5 = block_offs for block sizes 16,32,64,128,256, each
 * n_slices+1 long.  schedule: int32 [5, sched_pitch]; entry j of row b is
 * (block<<16)|slice for the j-th block of size 16<<b, -1 for j beyond the last
 * block, for j < max_n_blocks.
 */
int tamd_ragged_metadata(const int32_t *slice_sizes, int n_slices, int32_t *offs, int64_t offs_pitch,
                         int32_t *schedule, int64_t sched_pitch, int max_n_blocks, void *stream);

/*
 * fused routing metadata (no single counterpart; equals bitmatrix metadata
 * followed by ragged metadata on its col_sum, the composition of
 * tests/test_distributed.py:201-208) plus gather_indx = col_sorted_indx / k.
 */
int tamd_routing_metadata(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols, int k,
                          int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                          int32_t *gather_indx, int32_t *offs, int64_t offs_pitch, int32_t *schedule,
                          int64_t sched_pitch, int max_n_blocks, int32_t *workspace, void *stream);

/*
 * The whole routing step in one call: tamd_topk_forward (softmax over the k picked, indices chosen here) followed by
 * tamd_routing_metadata on its indices -- the composition of tests/test_distributed.py:201-208 as one entry point,
 * so that a binding pays for one foreign call per batch.  Arguments as in the two functions; y_indx is [n_rows, k]
 * with unit stride along k.
 */
int tamd_routing(const void *logits, int dtype, int64_t stride, int n_rows, int n_cols, int k, void *y_vals,
                 int16_t *y_indx, uint32_t *bits, int64_t bits_stride_row, int64_t bits_stride_word, int32_t *col_sum,
                 int32_t *col_sorted_indx, int32_t *row_sorted_indx, int32_t *gather_indx, int32_t *offs,
                 int64_t offs_pitch, int32_t *schedule, int64_t sched_pitch, int max_n_blocks, int32_t *workspace,
                 void *stream);

/*
 * tamd_routing_metadata for callers that cannot allocate (code under HIP graph capture, serving loops and
 * harnesses that forbid hipMalloc).  No counterpart in the reference, where every workspace is a torch allocation
 * made per call.  Same arguments and results as tamd_routing_metadata without `workspace`: the intermediate
 * tables live in a fixed 4 MiB array inside the library's code object (one copy per GPU, held until the process
 * ends).  Calls no allocating routine.  Problems whose workspace
 * (tamd_bitmatrix_metadata_workspace(n_indx, n_cols) int32 elements) exceeds
 * tamd_routing_metadata_static_max_workspace() elements return TAMD_E_TOO_LARGE and launch nothing.  All calls on
 * one GPU share that array: calls that overlap in time on the same GPU (different streams or threads) race; calls
 * on one stream are ordered and safe.  Nothing in the array has to start at zero (every entry a launch reads is
 * written earlier by the same call).
 * One-time host-side set-up per device (the array's address by hipGetSymbolAddress, the raised dynamic-LDS limits of
 * three kernels by hipFuncSetAttribute) happens on a device's first call, or ahead of time in
 * tamd_routing_metadata_static_init() with that device current: a caller that records a graph calls init, or makes
 * one ordinary call, before the capture begins.
 */
int tamd_routing_metadata_static_init(void);
int64_t tamd_routing_metadata_static_max_workspace(void);
int tamd_routing_metadata_static(const void *indx, int indx_is_int16, int64_t n_indx, int n_cols, int k,
                                 int32_t *col_sum, int32_t *col_sorted_indx, int32_t *row_sorted_indx,
                                 int32_t *gather_indx, int32_t *offs, int64_t offs_pitch, int32_t *schedule,
                                 int64_t sched_pitch, int max_n_blocks, void *stream);

/* activation fused into the matmul epilogue (matmul.py:40-43, swiglu_details/_swiglu.py:55-70) */
#define TAMD_ACT_NONE 0
#define TAMD_ACT_SWIGLU 1

/*
 * Grouped / dense matmul: replaces the launch of _matmul (matmul.py:642-709;
 * kernel matmul_details/_matmul.py:43-669).  The struct mirrors that kernel's
 * argument list.
 *
 *   y[dst(r), :] = act((x[src(r), :] . deq(w[e])) * x_scale * w_scale
 *                      + bias[e, :] * beta[r]) * out_alpha) * gamma[r]
 *
 * for every expert e and row r of its slice; src(r) = gather_indx[r] or r,
 * dst(r) = scatter_indx[r] (-1 drops the row) or r.
 */
typedef struct tamd_matmul_args {
  /* activations: [M_x, K], unit stride along K */
  const void *x;
  int x_dtype; /* TAMD_BF16 / TAMD_F16 / TAMD_FP8_E4M3 / TAMD_FP8_E5M2 */
  int64_t x_stride_m;
  const float *x_scale; /* per-tensor flex scale (device scalar) or NULL */
  /* weights: n_experts x [K, N]; MXFP4: packed bytes, K/2 bytes contiguous per column.  TAMD_BF16 / TAMD_F16
   * weights must have the activations' type, unit stride along K or along N, and K % 8 == 0 (N % 8 == 0 too when
   * N is the contiguous axis) */
  const void *w;
  int w_dtype; /* TAMD_MXFP4 / TAMD_BF16 / TAMD_F16 */
  int64_t w_stride_e, w_stride_k, w_stride_n; /* in storage elements (bytes for MXFP4) */
  const float *w_scale;                       /* per-tensor flex scale or NULL */
  const uint8_t *w_mx_scale;                  /* e8m0 [E, K/32, N] or NULL; see w_mx_layout */
  int64_t w_mx_stride_e, w_mx_stride_k, w_mx_stride_n;
  /* bias [E, N] (unit stride along N) or NULL */
  const void *bias;
  int bias_dtype; /* TAMD_F32 / TAMD_BF16 / TAMD_F16 */
  int64_t bias_stride_e;
  /* per expert-sorted-row factors, float32, or NULL */
  const float *betas;
  const float *gammas;
  float out_alpha; /* 1.0 when unused */
  /* output [rows_out, N_out], unit stride along N */
  void *y;
  int y_dtype; /* TAMD_BF16 / TAMD_F16 / TAMD_F32 / TAMD_FP8_E4M3 / TAMD_FP8_E5M2 */
  int64_t y_stride_m;
  /* problem */
  int M; /* rows to compute (len(gather_indx) or rows of x); per expert if not ragged */
  int N, K;
  int n_experts;          /* slices of w */
  const int32_t *gather_indx;  /* [M] or NULL */
  const int32_t *scatter_indx; /* [M] or NULL */
  /* ragged-M metadata (all NULL for a dense / batched problem) */
  const int32_t *slice_sizes;    /* [n_experts] */
  const int32_t *slice_offs;     /* [n_experts+1] */
  const int32_t *block_offs;     /* [n_experts+1] for block_m */
  const int32_t *block_schedule; /* [grid_m] for block_m */
  int block_m;                   /* 16..256: the block size block_offs / block_schedule were built for */
  int grid_m;                    /* upper bound on row blocks (RaggedTensorMetadata.n_blocks) */
  /* batched (non ragged, n_experts > 1): strides between batches */
  int64_t x_stride_z, y_stride_z;
  /* epilogue */
  int activation; /* TAMD_ACT_* */
  float act_alpha, act_limit;
  int act_has_limit;
  /* tuning overrides (0 = heuristic) */
  int force_variant;
  /* rows of x addressable through gather_indx (0 = M); x_rows * x_stride_m must stay below 2^30 elements */
  int64_t x_rows;
  /* flexpoint output (numerics_details/flexpoint.py:137-188, float_to_flex / update_scale): the result is
   * multiplied by 1 / *y_expected_scale before the cast (and clamped to the finite range of y_dtype when
   * y_saturate_inf); max|result| / max_finite(y_dtype) + 1e-30 is folded into *y_actual_scale by atomic max
   * (NaN counts as +inf).  Either pointer may be NULL.  y_dtype may then also be TAMD_FP8_E4M3 / TAMD_FP8_E5M2. */
  const float *y_expected_scale;
  float *y_actual_scale;
  int y_saturate_inf;
  /* encoding of w_mx_scale: TAMD_SCALE_STRIDED (strides above) or TAMD_SCALE_CDNA4, the pre-shuffled storage of
   * tensor_details/layout_details/cdna4_scale.py:32-68 (per expert: ceil(N/32) blocks of ceil(K/256)*8*32 bytes,
   * 16-byte aligned; only w_mx_stride_e is used) */
  int w_mx_layout;
  /* microscaled activations (MXFP8: x_dtype TAMD_FP8_E4M3 with one e8m0 byte per 32 elements of a row, the
   * a_mx_scale of matmul.py:131-136): [x_rows, K/32] bytes, unit stride along K/32, indexed by the same (gathered)
   * row as x; NULL = no block scales.  x_mx_stride_z is the batch pitch. */
  const uint8_t *x_mx_scale;
  int64_t x_mx_stride_m, x_mx_stride_z;
  /* MXFP8 output (the quantising epilogue _quantize_mxfp8_fn, mxfp_details/_downcast_to_mxfp.py:218-220): with
   * y_dtype TAMD_FP8_E4M3 the result is quantised per 32 consecutive output columns of a row exactly as
   * tamd_downcast_mxfp (ROUND_UP) would quantise the float32 result; the e8m0 bytes go to
   * y_mx_scale[row, column / 32] (rows placed like the rows of y).  NULL = plain output. */
  uint8_t *y_mx_scale;
  int64_t y_mx_stride_m, y_mx_stride_z;
  /* encoding of MXFP4 w: TAMD_W_STRIDED (w_stride_* above: K/2 bytes contiguous per column) or TAMD_W_CDNA4_BLOCKS,
   * this library's own layout (no counterpart in the reference, whose AMD path keeps the strided one;
   * tensor_details/layout.py CDNA4MXValueLayout): per expert ceil(N/64) strips x ceil(K/128) stages of 4 KB blocks,
   * K and N padded with zero codes; in a block, column 2c + f of the strip is position 32 f + c (64 bytes), its
   * 16-byte part p in slot p ^ ((c >> 2) & 3) ^ 2 f.  Only w_stride_e is used (bytes); w 16-byte aligned. */
  int w_layout;
} tamd_matmul_args;

int tamd_matmul(const tamd_matmul_args *args, void *stream);

/*
 * reduce over the middle axis: replaces the launch of _reduce_forward
 * (reduce.py:813; API reduce.py:1135-1157) for the sum / mask / scale case.
 * x [S0, R, S1] -> y [S0, S1], y = sum_r mask * scale * x in float32, cast to
 * y_dtype.  mask (uint8 / bool, nonzero = keep) and scale (float32) are optional
 * and indexed with their own strides (0 broadcasts).
 */
int tamd_reduce(const void *x, int x_dtype, int64_t S0, int64_t R, int64_t S1, int64_t xs0, int64_t xsr,
                int64_t xs1, const uint8_t *mask, int64_t ms0, int64_t msr, int64_t ms1,
                const float *scale, int64_t ss0, int64_t ssr, int64_t ss1, void *y, int y_dtype,
                int64_t ys0, int64_t ys1, void *stream);

/*
 * General reduction over the middle axis: replaces the launch of _reduce_forward with all of its optional operands
 * (reduce.py:375-492 kernel body, :818-957 host, API :1135-1157).  x [S0, R, S1] -> y [S0, S1 / n] where n = 1
 * without post-processing and 2 with one of the pairwise functions below.
 *
 *   acc[s0, c] = sum_r mask * (x * 2^(x_mx_scale - 127) * *x_flex_scale * scale)       float32, r in index order; the
 *                first term starts the sum when R <= 8 (reduce.py:137, 467-470: a column of -0.0 stays -0.0), longer
 *                axes start from +0.0; a term with a scale is fma(x, scale, +0.0) (reduce.py:466)
 *   o          = postprocess(acc) * *x_global_scale
 *   flexpoint output (no y_mx_scale): *y_actual_scale <- max(*y_actual_scale, max|o| / max_finite(y_dtype) + 1e-30)
 *                                     by atomic max; o / *y_expected_scale, clamped to y_dtype's finite range when
 *                                     y_saturate_inf; cast (numerics_details/flexpoint.py:137-188)
 *   MXFP8 output (y_mx_scale given):  o / *y_expected_scale quantised per 32 output columns exactly as
 *                                     tamd_downcast_mxfp (ROUND_UP, float8_e4m3fn values) quantises float32 input
 * x_dtype / y_dtype: F32, F16, BF16, FP8_E4M3, FP8_E5M2.  x_mx_scale: e8m0 bytes, one per 32 columns of S1, indexed
 * [s0, r, c / 32] with its own strides.  mask (nonzero = keep) and scale (float32) are indexed with their own
 * strides (0 broadcasts).  Every pointer but x and y may be NULL.
 */
#define TAMD_PP_NONE 0
#define TAMD_PP_SWIGLU 1          /* o[j] = swiglu(acc[2j], acc[2j+1]; alpha = pp_arg0, limit = pp_arg1 if pp_has_arg1) */
#define TAMD_PP_PLUS_A_PAIRSUM 2  /* o[j] = (acc[2j] + pp_arg0) + (acc[2j+1] + pp_arg0): tests/test_reduce.py:35-38 */
typedef struct tamd_reduce_args {
  const void *x;
  int x_dtype;
  int64_t S0, R, S1;
  int64_t xs0, xsr, xs1;
  const uint8_t *x_mx_scale;
  int64_t xms0, xmsr, xms1;
  const float *x_flex_scale;
  const float *x_global_scale;
  const uint8_t *mask;
  int64_t ms0, msr, ms1;
  const float *scale;
  int64_t ss0, ssr, ss1;
  int postprocess; /* TAMD_PP_* */
  float pp_arg0, pp_arg1;
  int pp_has_arg1;
  void *y;
  int y_dtype;
  int64_t ys0, ys1;
  const float *y_expected_scale;
  float *y_actual_scale;
  int y_saturate_inf;
  uint8_t *y_mx_scale; /* [S0, ceil(S1 / n / 32)] */
  int64_t yms0, yms1;
  /* optional device scalar (reduce.py:550-555 of the reference, `unpadded_batch_size`): only rows s0 < *it are
   * reduced and written; the rest of y (and of y_mx_scale) is left as it is */
  const int32_t *unpadded_batch_size;
} tamd_reduce_args;

int tamd_reduce_ex(const tamd_reduce_args *args, void *stream);

/*
 * standalone interleaved SwiGLU: replaces the launch of _swiglu (swiglu.py:52-76).
 * a [M, 2*N_out] -> out [M, N_out].
 */
int tamd_swiglu(const void *a, int dtype, int64_t M, int64_t N_out, int64_t a_stride_m, void *out,
                int64_t out_stride_m, float alpha, float limit, int has_limit, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* TRITON_AMD_H */

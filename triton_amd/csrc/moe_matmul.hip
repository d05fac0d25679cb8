// Grouped (ragged-M) / dense matmul for gfx950: 16-bit activations x MXFP4 weights.
//
//   y[dst(r), :] = act(((x[src(r), :] . deq(w[e])) * sx * sw + bias[e, :] * beta[r]) * alpha) * gamma[r]
//
// (matmul_details/_matmul.py:43-669 of the reference; epilogue order :540-559.)
//
// Work decomposition
//   workgroup (4 waves) = one BLOCK_M x BLOCK_N output tile of one expert, taken from
//     the ragged block schedule ((block << 16) | expert, -1 = padding);
//   wave w owns the 16*NF columns [w*16*NF, (w+1)*16*NF) of the tile and ALL its rows:
//     the MXFP4 weights of those columns go HBM -> registers (one 128-bit load = 32
//     consecutive K of one column = one e8m0 group), are expanded to bf16/f16 in
//     registers with v_cvt_scalef32_pk_*_fp4 and feed v_mfma_f32_16x16x32 as the B
//     operand, so every weight byte is fetched and converted once per workgroup;
//   the activation rows (gathered) are staged through LDS, double buffered, 128 K
//     per stage, 16-byte chunks XOR-swizzled by row so that the MFMA A-operand reads
//     (16 rows x one chunk per quarter-wave) hit distinct banks.
//
// K order inside a 128-K stage: lane group g = lane/16 holds K [32g, 32g+32) of its
// column; MFMA step s consumes elements [8s, 8s+8) of every group, for A and B alike.
#include "common.h"

namespace tamd {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 f16x8_t __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

constexpr int KB = 128;            // K per pipeline stage
constexpr int ROW_BYTES = KB * 2;  // LDS bytes per activation row per stage

template <int XDT>
struct Mma;
template <>
struct Mma<TAMD_BF16> {
  typedef bf16x8_t frag_t;
  static TAMD_DEVICE frag_t expand(uint32_t codes, float scale) {
    bf16x2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 0);
    bf16x2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 1);
    bf16x2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 2);
    bf16x2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(codes, scale, 3);
    return frag_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  }
  static TAMD_DEVICE f32x4_t mma(frag_t a, frag_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
template <>
struct Mma<TAMD_F16> {
  typedef f16x8_t frag_t;
  static TAMD_DEVICE frag_t expand(uint32_t codes, float scale) {
    f16x2_t p0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 0);
    f16x2_t p1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 1);
    f16x2_t p2 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 2);
    f16x2_t p3 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(codes, scale, 3);
    return frag_t{p0[0], p0[1], p1[0], p1[1], p2[0], p2[1], p3[0], p3[1]};
  }
  static TAMD_DEVICE f32x4_t mma(frag_t a, frag_t b, f32x4_t c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};

TAMD_DEVICE float load_any_f32(const void *p, int dt, int64_t i) {
  if (dt == TAMD_F32) return ((const float *)p)[i];
  if (dt == TAMD_BF16) return bf16_bits_to_f32(((const uint16_t *)p)[i]);
  return f16_bits_to_f32(((const uint16_t *)p)[i]);
}

TAMD_DEVICE void store_any(void *p, int dt, int64_t i, float v) {
  if (dt == TAMD_F32) ((float *)p)[i] = v;
  else if (dt == TAMD_BF16) ((uint16_t *)p)[i] = (uint16_t)f32_to_bf16_bits(v);
  else ((uint16_t *)p)[i] = (uint16_t)f32_to_f16_bits(v);
}

TAMD_DEVICE float swiglu_epi(float g, float l, float alpha, float limit, bool has_limit) {
  if (has_limit) {
    g = __builtin_fminf(g, limit);
    l = __builtin_fminf(__builtin_fmaxf(l, -limit), limit);
  }
  float s = g / (1.0f + expf(-alpha * g));
  return __builtin_fmaf(s, l, s);
}

// Tile coordinates of a workgroup.
struct Tile {
  int expert;     // weight slice
  int z;          // batch index (dense batched) else 0
  int start_m;    // first expert-sorted row of the slice
  int off_m;      // first row of the tile inside the slice
  int rows;       // valid rows in the tile (1..BLOCK_M)
  int slice_rows; // rows of the slice
  int n0;         // first column of the tile
};

template <int BLOCK_M, int BLOCK_N>
TAMD_DEVICE bool locate_tile(const tamd_matmul_args &a, int grid_n, int64_t grid_total, Tile &t) {
  // XCD-aware remap: hardware deals workgroups round-robin to the 8 XCDs; give each
  // XCD a contiguous range of tiles so neighbours (same expert, adjacent columns)
  // share one L2.
  const int64_t per_xcd = (grid_total + 7) / 8;
  int64_t pid = (int64_t)(blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (pid >= grid_total) return false;
  int pid_m = (int)(pid / grid_n);
  int pid_n = (int)(pid - (int64_t)pid_m * grid_n);
  t.n0 = pid_n * BLOCK_N;
  t.z = 0;
  if (a.block_schedule) {
    int sched = a.block_schedule[pid_m];
    if (sched == -1) return false;
    t.expert = sched & 0xFFFF;
    int blk = sched >> 16;
    t.slice_rows = a.slice_sizes[t.expert];
    t.start_m = a.slice_offs[t.expert];
    t.off_m = blk * BLOCK_M;
  } else {
    int bm = (a.M + BLOCK_M - 1) / BLOCK_M;
    int z = pid_m / bm;
    t.expert = z;
    t.z = z;
    t.slice_rows = a.M;
    t.start_m = 0;
    t.off_m = (pid_m - z * bm) * BLOCK_M;
  }
  t.rows = t.slice_rows - t.off_m;
  if (t.rows > BLOCK_M) t.rows = BLOCK_M;
  return t.rows > 0;
}

// MF: 16-row fragments per tile (BLOCK_M = 16*MF); NF: 16-column fragments per wave.
template <int XDT, int MF, int NF, int ACT>
__global__ __launch_bounds__(256) void mm_x16_mxfp4_kernel(tamd_matmul_args a, int grid_n, int64_t grid_total) {
  typedef Mma<XDT> M;
  typedef typename M::frag_t frag_t;
  constexpr int BLOCK_M = 16 * MF;
  constexpr int BLOCK_N = 64 * NF;
  __shared__ __attribute__((aligned(16))) uint8_t lds[2][BLOCK_M * ROW_BYTES];

  Tile t;
  if (!locate_tile<BLOCK_M, BLOCK_N>(a, grid_n, grid_total, t)) return;
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int cidx = lane % 16, g = lane / 16;
  const int nfr = (t.rows + 15) / 16;  // active row fragments (wave uniform)
  const int K = a.K, N = a.N;

  // ---- activation staging: thread -> (row tid/16 of every fragment, chunk tid%16)
  const int a_chunk = tid % 16, a_row = tid / 16;
  const uint8_t *a_ptr[MF];
#pragma unroll
  for (int i = 0; i < MF; ++i) {
    int r = i * 16 + a_row;
    int rr = t.off_m + (r < t.rows ? r : t.rows - 1);
    int64_t src = a.gather_indx ? (int64_t)a.gather_indx[t.start_m + rr] : (int64_t)(t.start_m + rr);
    a_ptr[i] = (const uint8_t *)a.x + ((int64_t)t.z * a.x_stride_z + src * a.x_stride_m) * 2 + a_chunk * 16;
  }
  // ---- weight columns of this lane
  const uint8_t *w_ptr[NF];
  const uint8_t *s_ptr[NF];
  int col[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    col[f] = t.n0 + wave * (16 * NF) + cidx * NF + f;
    int cc = col[f] < N ? col[f] : N - 1;
    w_ptr[f] = (const uint8_t *)a.w + (int64_t)t.expert * a.w_stride_e + (int64_t)cc * a.w_stride_n + g * 16;
    s_ptr[f] = a.w_mx_scale + (int64_t)t.expert * a.w_mx_stride_e + (int64_t)cc * a.w_mx_stride_n + g;
  }

  f32x4_t acc[MF][NF];
#pragma unroll
  for (int i = 0; i < MF; ++i)
#pragma unroll
    for (int f = 0; f < NF; ++f) acc[i][f] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  uint4 a_stage[MF];
  uint4 b_raw[NF];
  uint32_t b_scale[NF];

  auto fetch = [&](int kb) {
    const bool a_ok = kb + a_chunk * 8 < K;
#pragma unroll
    for (int i = 0; i < MF; ++i) {
      if (i < nfr) a_stage[i] = a_ok ? *(const uint4 *)(a_ptr[i] + (int64_t)kb * 2) : make_uint4(0, 0, 0, 0);
    }
    const bool b_ok = kb + g * 32 < K;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      b_raw[f] = b_ok ? *(const uint4 *)(w_ptr[f] + (kb >> 1)) : make_uint4(0, 0, 0, 0);
      b_scale[f] = b_ok ? (uint32_t)s_ptr[f][kb >> 5] : 0u;
    }
  };

  const int n_kb = (K + KB - 1) / KB;
  fetch(0);
  for (int it = 0; it < n_kb; ++it) {
    uint8_t *buf = lds[it & 1];
#pragma unroll
    for (int i = 0; i < MF; ++i) {
      if (i < nfr) {
        int r = i * 16 + a_row;
        *(uint4 *)(buf + r * ROW_BYTES + ((a_chunk ^ (r & 15)) * 16)) = a_stage[i];
      }
    }
    uint4 b_cur[NF];
    float sc_cur[NF];
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      b_cur[f] = b_raw[f];
      sc_cur[f] = bits_to_f32(b_scale[f] << 23);
    }
    __syncthreads();
    if (it + 1 < n_kb) fetch((it + 1) * KB);
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      frag_t af[MF];
#pragma unroll
      for (int i = 0; i < MF; ++i) {
        if (i < nfr) {
          int r = i * 16 + cidx;
          af[i] = *(const frag_t *)(buf + r * ROW_BYTES + (((g * 4 + s) ^ (r & 15)) * 16));
        }
      }
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        uint32_t codes = s == 0 ? b_cur[f].x : (s == 1 ? b_cur[f].y : (s == 2 ? b_cur[f].z : b_cur[f].w));
        frag_t bf = M::expand(codes, sc_cur[f]);
#pragma unroll
        for (int i = 0; i < MF; ++i) {
          if (i < nfr) acc[i][f] = M::mma(af[i], bf, acc[i][f]);
        }
      }
    }
  }

  // ---- epilogue
  float flex = 1.0f;
  if (a.x_scale) flex *= *a.x_scale;
  if (a.w_scale) flex *= *a.w_scale;
  float bias[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f)
    bias[f] = (a.bias && col[f] < N) ? load_any_f32(a.bias, a.bias_dtype, (int64_t)t.expert * a.bias_stride_e + col[f])
                                     : 0.f;
  constexpr int NO = ACT == TAMD_ACT_SWIGLU ? NF / 2 : NF;  // outputs per lane per row
  const int n_out = ACT == TAMD_ACT_SWIGLU ? N / 2 : N;
  const int out_col0 = ACT == TAMD_ACT_SWIGLU ? (t.n0 + wave * (16 * NF) + cidx * NF) / 2
                                              : (t.n0 + wave * (16 * NF) + cidx * NF);
  const bool has_limit = a.act_has_limit != 0;
#pragma unroll
  for (int i = 0; i < MF; ++i) {
    if (i >= nfr) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int r = i * 16 + g * 4 + j;
      if (r >= t.rows) continue;
      const int erow = t.start_m + t.off_m + r;  // expert-sorted row
      int64_t dst = erow;
      if (a.scatter_indx) {
        dst = a.scatter_indx[erow];
        if (dst < 0) continue;
      }
      const float beta = a.betas ? a.betas[erow] : 1.0f;
      const float gamma = a.gammas ? a.gammas[erow] : 1.0f;
      float v[NF];
#pragma unroll
      for (int f = 0; f < NF; ++f) v[f] = (acc[i][f][j] * flex + bias[f] * beta) * a.out_alpha;
      float o[NO];
      if constexpr (ACT == TAMD_ACT_SWIGLU) {
#pragma unroll
        for (int p = 0; p < NO; ++p) o[p] = swiglu_epi(v[2 * p], v[2 * p + 1], a.act_alpha, a.act_limit, has_limit);
      } else {
#pragma unroll
        for (int p = 0; p < NO; ++p) o[p] = v[p];
      }
      const int64_t base = (int64_t)t.z * a.y_stride_z + dst * a.y_stride_m;
      uint16_t *y16 = (uint16_t *)a.y + base + out_col0;
      if (NO == 4 && a.y_dtype != TAMD_F32 && out_col0 + NO <= n_out && ((uintptr_t)y16 & 7) == 0) {
        uint32_t lo, hi;
        if (a.y_dtype == TAMD_BF16) {
          lo = f32_to_bf16_bits(o[0] * gamma) | (f32_to_bf16_bits(o[1 % NO] * gamma) << 16);
          hi = f32_to_bf16_bits(o[2 % NO] * gamma) | (f32_to_bf16_bits(o[3 % NO] * gamma) << 16);
        } else {
          lo = f32_to_f16_bits(o[0] * gamma) | (f32_to_f16_bits(o[1 % NO] * gamma) << 16);
          hi = f32_to_f16_bits(o[2 % NO] * gamma) | (f32_to_f16_bits(o[3 % NO] * gamma) << 16);
        }
        *(uint2 *)y16 = make_uint2(lo, hi);
      } else if (NO == 2 && a.y_dtype != TAMD_F32 && out_col0 + NO <= n_out && ((uintptr_t)y16 & 3) == 0) {
        uint32_t lo;
        if (a.y_dtype == TAMD_BF16)
          lo = f32_to_bf16_bits(o[0] * gamma) | (f32_to_bf16_bits(o[1 % NO] * gamma) << 16);
        else
          lo = f32_to_f16_bits(o[0] * gamma) | (f32_to_f16_bits(o[1 % NO] * gamma) << 16);
        *(uint32_t *)y16 = lo;
      } else {
#pragma unroll
        for (int p = 0; p < NO; ++p)
          if (out_col0 + p < n_out) store_any(a.y, a.y_dtype, base + out_col0 + p, o[p] * gamma);
      }
    }
  }
}

template <int XDT, int MF, int NF>
int launch_x16(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  constexpr int BLOCK_N = 64 * NF;
  int grid_n = (a.N + BLOCK_N - 1) / BLOCK_N;
  int64_t total = (int64_t)grid_m * grid_n;
  if (total <= 0) return 0;
  int64_t launch = ((total + 7) / 8) * 8;
  if (launch > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
  if (a.activation == TAMD_ACT_SWIGLU)
    mm_x16_mxfp4_kernel<XDT, MF, NF, TAMD_ACT_SWIGLU><<<dim3((unsigned)launch), 256, 0, st>>>(a, grid_n, total);
  else
    mm_x16_mxfp4_kernel<XDT, MF, NF, TAMD_ACT_NONE><<<dim3((unsigned)launch), 256, 0, st>>>(a, grid_n, total);
  return launch_status();
}

template <int XDT>
int dispatch_x16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  switch (block_m) {
    case 16: return launch_x16<XDT, 1, 4>(a, grid_m, st);
    case 32: return launch_x16<XDT, 2, 4>(a, grid_m, st);
    case 64: return launch_x16<XDT, 4, 4>(a, grid_m, st);
    case 128: return launch_x16<XDT, 8, 4>(a, grid_m, st);
    default: return TAMD_E_UNSUPPORTED;
  }
}

}  // namespace tamd

using namespace tamd;

extern "C" int tamd_matmul(const tamd_matmul_args *args, void *stream) {
  if (!args) return TAMD_E_INVALID;
  const tamd_matmul_args &a = *args;
  if (a.M < 0 || a.N < 0 || a.K < 0 || a.n_experts < 1) return TAMD_E_INVALID;
  if (a.M == 0 || a.N == 0) return 0;
  if (!a.x || !a.w || !a.y) return TAMD_E_INVALID;
  if (a.activation != TAMD_ACT_NONE && a.activation != TAMD_ACT_SWIGLU) return TAMD_E_INVALID;
  if (a.activation == TAMD_ACT_SWIGLU && (a.N % 2) != 0) return TAMD_E_INVALID;
  if (a.y_dtype != TAMD_BF16 && a.y_dtype != TAMD_F16 && a.y_dtype != TAMD_F32) return TAMD_E_INVALID;
  if (a.bias && a.bias_dtype != TAMD_F32 && a.bias_dtype != TAMD_BF16 && a.bias_dtype != TAMD_F16)
    return TAMD_E_INVALID;
  const bool ragged = a.block_schedule != nullptr;
  if (ragged && (!a.slice_sizes || !a.slice_offs || a.grid_m < 0)) return TAMD_E_INVALID;
  hipStream_t st = (hipStream_t)stream;

  if (a.w_dtype == TAMD_MXFP4 && (a.x_dtype == TAMD_BF16 || a.x_dtype == TAMD_F16)) {
    if (!a.w_mx_scale) return TAMD_E_INVALID;
    if (a.K % 32 != 0) return TAMD_E_INVALID;
    // weights / scales must be contiguous along K ("column-major" mxfp weights)
    if (a.w_stride_k != 1 || a.w_mx_stride_k != 1) return TAMD_E_UNSUPPORTED;
    if (!aligned(a.w, 16) || a.w_stride_n % 16 != 0 || a.w_stride_e % 16 != 0) return TAMD_E_ALIGNMENT;
    if (!aligned(a.x, 16) || (a.x_stride_m * 2) % 16 != 0 || (a.x_stride_z * 2) % 16 != 0) return TAMD_E_ALIGNMENT;
    int block_m, grid_m;
    if (ragged) {
      block_m = a.block_m;
      grid_m = a.grid_m;
    } else {
      block_m = a.force_variant ? a.force_variant : (a.M <= 16 ? 16 : a.M <= 32 ? 32 : a.M <= 64 ? 64 : 128);
      grid_m = ((a.M + block_m - 1) / block_m) * a.n_experts;
    }
    if (a.x_dtype == TAMD_BF16) return dispatch_x16<TAMD_BF16>(a, block_m, grid_m, st);
    return dispatch_x16<TAMD_F16>(a, block_m, grid_m, st);
  }
  return TAMD_E_UNSUPPORTED;
}

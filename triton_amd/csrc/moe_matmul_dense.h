// Grouped / dense matmul with unquantised 16-bit weights (bf16 x bf16, f16 x f16): the gate matmul and
// every caller of `matmul` that passes plain weights.  Same tile decomposition, activation staging and
// epilogue as the MXFP4 kernel of moe_matmul_impl.h; only the weight path differs:
//
//   * K-contiguous weights (w_stride_k == 1, the layout of the quantised weights): a stage holds
//     [256 columns][64 K] = 128 bytes per column, copied by DMA exactly like activation rows and read
//     as 16-byte MFMA fragments;
//   * N-contiguous weights (w_stride_n == 1, the usual row-major [K, N]): a stage holds
//     [64 K][256 columns] as it lies in memory (512 bytes per K row); a lane gathers the 8 K values of
//     its column with 2-byte LDS reads.  The MFMA wants K-contiguous operands on both sides, so one of
//     the two has to be transposed somewhere; doing it on the LDS read costs no extra pass.
//
// One workgroup per CU (three 32 KB weight stages); not a tuned kernel -- the unquantised
// products on this path are small next to the expert matmuls.
#pragma once
#include "moe_matmul_impl.h"

namespace tamd {

constexpr int W16_STAGE = 256 * 128;  // bytes of one weight stage in either layout

template <int XDT, int NFR, int LDS_ROWS, int ACT, bool WKC>
TAMD_DEVICE void run_tile_w16(const tamd_matmul_args &a, const Tile &t, uint8_t *lds) {
  typedef Mma<XDT> M;
  typedef typename M::frag_t frag_t;
  constexpr int KA = 64;
  constexpr int A_STAGE = LDS_ROWS * A_ROW_BYTES;
  constexpr uint32_t kOob = 0x7FFFFFFFu;
  const int tid = threadIdx.x;
  const int wave = tid / kWave, lane = tid % kWave;
  const int c32 = lane % 32, h = lane / 32;
  const int K = a.K, N = a.N;

  const v4i_t rx = make_rsrc((const uint8_t *)a.x + (int64_t)t.z * a.x_stride_z * 2, kOob);
  // the descriptor ends with the expert's weights: a copy that starts inside and runs past the end
  // (partial last chunk of columns) delivers zeros for the part outside
  const int64_t w_span = (WKC ? (int64_t)N * a.w_stride_n : (int64_t)K * a.w_stride_k) * 2;
  const v4i_t rw = make_rsrc((const uint8_t *)a.w + (int64_t)t.expert * a.w_stride_e * 2, (uint32_t)w_span);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  constexpr int RING = 3;  // stages: one consumed, two in flight (the K loop of a small tile is latency bound)
  const uint32_t lds_b = lds_base + RING * A_STAGE;

  // ---- activation DMA (as in run_tile): lane -> (row 8w + lane/8, slot lane%8)
  const int a_rin = wave * 8 + lane / 8;
  const int a_chunk = (lane % 8) ^ ((a_rin >> 1) & 7);
  uint32_t a_off[NFR];
#pragma unroll
  for (int i = 0; i < NFR; ++i) {
    const int r = i * 32 + a_rin;
    const int rr = t.off_m + (r < t.rows ? r : t.rows - 1);
    const uint32_t src = a.gather_indx ? (uint32_t)a.gather_indx[t.start_m + rr] : (uint32_t)(t.start_m + rr);
    a_off[i] = src * (uint32_t)(a.x_stride_m * 2) + a_chunk * 16;
  }
  // ---- weight DMA: 8 instructions per wave and stage
  uint32_t w_off[8];
  int w_chunk[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    if constexpr (WKC) {
      // LDS row p = wave*64 + j*8 + lane/8 holds tile column wave*64 + 2*(q%32) + q/32 (q = p%64) so that a lane's
      // two fragments are a gate / linear pair; 16-byte chunks swizzled like activation rows
      const int q = j * 8 + lane / 8;
      const int col = t.n0 + wave * 64 + 2 * (q % 32) + q / 32;
      w_chunk[j] = (lane % 8) ^ (((wave * 64 + q) >> 1) & 7);
      w_off[j] = col < N ? (uint32_t)col * (uint32_t)(a.w_stride_n * 2) + w_chunk[j] * 16 : kOob;
    } else {
      // K rows 16w + 2j, 16w + 2j + 1 of the stage, 32 chunks of 8 columns each
      const int col = t.n0 + 8 * (lane % 32);
      w_chunk[j] = wave * 16 + 2 * j + lane / 32;  // K row inside the stage
      // N is a multiple of 8 here; the lane's half (lane/32) of the K row pair goes into the vector offset, the
      // pair's first row into the wave-uniform scalar offset
      w_off[j] = col + 8 <= N ? (uint32_t)col * 2u + (uint32_t)(lane / 32) * (uint32_t)(a.w_stride_k * 2) : kOob;
    }
  }

  f32x16_t acc[NFR][NF];
#pragma unroll
  for (int i = 0; i < NFR; ++i)
#pragma unroll
    for (int f = 0; f < NF; ++f)
#pragma unroll
      for (int j = 0; j < 16; ++j) acc[i][f][j] = 0.f;

  const int n_k = (K + KA - 1) / KA;
  auto issue = [&](int it, int slot) {  // clamped: past the end the last stage is copied again (never read)
    it = it < n_k ? it : n_k - 1;
    const int kb = it * KA;
    const uint32_t akill = kb + a_chunk * 8 < K ? 0u : kOob;
    const uint32_t sa = lds_base + slot * A_STAGE + wave * 8 * A_ROW_BYTES;
#pragma unroll
    for (int i = 0; i < NFR; ++i) dma16(rx, sa + i * 32 * A_ROW_BYTES, a_off[i] | akill, kb * 2);
    const uint32_t sb = lds_b + slot * W16_STAGE;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      if constexpr (WKC) {
        const uint32_t kill = kb + w_chunk[j] * 8 < K ? 0u : kOob;
        dma16(rw, sb + (wave * 64 + j * 8) * 128, w_off[j] | kill, kb * 2);
      } else {
        const int k = kb + w_chunk[j];
        const uint32_t kill = k < K ? 0u : kOob;
        dma16(rw, sb + (wave * 16 + 2 * j) * 512, w_off[j] | kill,
              (uint32_t)((int64_t)(kb + wave * 16 + 2 * j) * a.w_stride_k * 2));
      }
    }
  };

  auto compute = [&](int slot) {
    const uint8_t *abuf = lds + slot * A_STAGE;
    const uint8_t *bbuf = lds + RING * A_STAGE + slot * W16_STAGE;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      frag_t af[NFR];
      const int aslot = (h * 4 + s) ^ ((c32 >> 1) & 7);
#pragma unroll
      for (int i = 0; i < NFR; ++i) af[i] = *(const frag_t *)(abuf + (i * 32 + c32) * A_ROW_BYTES + aslot * 16);
#pragma unroll
      for (int f = 0; f < NF; ++f) {
        frag_t bf;
        if constexpr (WKC) {
          const int p = wave * 64 + f * 32 + c32;
          bf = *(const frag_t *)(bbuf + p * 128 + (((h * 4 + s) ^ ((p >> 1) & 7)) * 16));
        } else {
          const uint16_t *colp = (const uint16_t *)bbuf + (wave * 64 + c32 * NF + f);
          uint32_t w[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int k = (h * 4 + s) * 8 + 2 * e;
            w[e] = (uint32_t)colp[k * 256] | ((uint32_t)colp[(k + 1) * 256] << 16);
          }
          bf = __builtin_bit_cast(frag_t, make_uint4(w[0], w[1], w[2], w[3]));
        }
#pragma unroll
        for (int i = 0; i < NFR; ++i) acc[i][f] = M::mma(af[i], bf, acc[i][f]);
      }
    }
  };

  issue(0, 0);
  issue(1, 1);
  int rd = 0;  // ring slot of the stage being consumed (stage it lives in slot it % 3)
  for (int it = 0; it < n_k; ++it) {
    wait_vmcnt<NFR + 8>();  // copies complete in order: all but the NFR + 8 of stage it + 1 have landed
    __syncthreads();        // stage `it` is visible; everyone is done with the slot stage it + 2 goes to
    issue(it + 2, rd == 0 ? 2 : rd - 1);
    compute(rd);
    rd = rd == 2 ? 0 : rd + 1;
  }
  wait_dma();
  tile_epilogue<NFR, ACT, XDT, false>(a, t, acc, lds);
}

template <int XDT, int BM, int ACT, bool WKC>
__global__ __launch_bounds__(256, 1) void mm_x16_w16_kernel(tamd_matmul_args a, int grid_n, int64_t grid_total) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr int MF = BM <= 32 ? 1 : BM / 32;
  Tile t;
  if (!locate_tile<BM, 0>(a, grid_n, grid_total, 1, t)) return;
  const int nfr = (t.rows + 31) / 32;
#define TAMD_CASE(n)                                                            \
  case n:                                                                       \
    if constexpr (n <= MF) run_tile_w16<XDT, n, 32 * MF, ACT, WKC>(a, t, lds);  \
    break;
  switch (nfr) { TAMD_CASE(1) TAMD_CASE(2) TAMD_CASE(3) TAMD_CASE(4) }
#undef TAMD_CASE
}

template <int XDT, int BM, int ACT, bool WKC>
int launch_w16(const tamd_matmul_args &a, int grid_m, hipStream_t st) {
  constexpr int MF = BM <= 32 ? 1 : BM / 32;
  constexpr int LDS_ROWS = 32 * MF;
  constexpr int PIPE = 3 * LDS_ROWS * A_ROW_BYTES + 3 * W16_STAGE;
  static_assert(PIPE <= 160 * 1024, "one workgroup per CU");
  constexpr int OUT_BYTES = LDS_ROWS * 256 * 2;
  const int grid_n = (a.N + BLOCK_N - 1) / BLOCK_N;
  const int64_t total = (int64_t)grid_m * grid_n;
  if (total <= 0) return 0;
  const int64_t launch = ((total + 7) / 8) * 8;
  if (launch > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
  auto kern = mm_x16_w16_kernel<XDT, BM, ACT, WKC>;
  if (int rc = raise_lds_limit_once((const void *)kern)) return rc;
  kern<<<dim3((unsigned)launch), 256, PIPE > OUT_BYTES ? PIPE : OUT_BYTES, st>>>(a, grid_n, total);
  return launch_status();
}

// ---------------------------------------------------------------------------
// Narrow outputs (N <= 128: the gate matmul, tokens x d_model times d_model x n_experts): one dense product whose
// weights are small and whose activations are read once.  The tiled kernel above would give such a problem a
// handful of half-empty 256-column tiles with a long, latency-bound K loop each.  Here a workgroup owns 16 rows x
// 64 columns and its four waves split K: wave w takes the 64-K blocks w, w + 4, ...  Both operands are
// K-contiguous; a block is 16 + 64 lines of 128 bytes, copied by DMA whole lines at a time (8 lanes per line)
// into a ring of three stages that belongs to the wave alone -- so the loop has no barrier: a wave waits for its
// own copies, reads v_mfma_f32_16x16x32 operands (lane (c = lane % 16, g = lane / 16): K values 8g .. 8g+7 of
// row / column c; 16-byte chunks swizzled by the line index) and requests the block two ahead.  The four partial
// sums meet in LDS; bias, scales and the cast follow.
// ---------------------------------------------------------------------------
typedef float f32x4s_t __attribute__((ext_vector_type(4)));
template <int XDT>
TAMD_DEVICE f32x4s_t mma16x16x32(uint4 a, uint4 b, f32x4s_t c) {
  if constexpr (XDT == TAMD_BF16)
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

constexpr int SKINNY_COLS = 64;                     // columns of a workgroup
constexpr int SKINNY_PITCH = 68;                    // floats per row of a partial sum in LDS (padded)
constexpr int SKINNY_STAGE = (16 + 64) * 128;       // bytes of one 64-K block: 16 rows, then 64 columns
constexpr int SKINNY_RING = 3;
constexpr int SKINNY_LDS = 4 * SKINNY_RING * SKINNY_STAGE + 4 * 16 * SKINNY_PITCH * 4;

template <int XDT>
__global__ __launch_bounds__(256) void mm_skinny16_kernel(tamd_matmul_args a) {
  extern __shared__ __attribute__((aligned(16))) uint8_t lds[];
  constexpr uint32_t kOob = 0x7FFFFFFFu;
  float *red = (float *)(lds + 4 * SKINNY_RING * SKINNY_STAGE);
  const int tid = threadIdx.x;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave), lane = tid % kWave;
  const int c = lane % 16, g = lane / 16;
  const int M = a.M, N = a.N, K = a.K;
  const int row0 = blockIdx.x * 16, col0 = blockIdx.y * SKINNY_COLS;
  const v4i_t rx = make_rsrc(a.x, kOob), rw = make_rsrc(a.w, kOob);
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t *)lds;
  const uint32_t ring = lds_base + wave * SKINNY_RING * SKINNY_STAGE;
  const uint8_t *ringp = lds + wave * SKINNY_RING * SKINNY_STAGE;
  // copy instruction i moves lines 8i .. 8i+7 of a stage: lane -> (line 8i + lane / 8, 16-byte slot lane % 8), the
  // slot holding chunk slot ^ (line % 8) of the line.  Rows past M and columns past N repeat the last one (their
  // results are not stored); chunks past K are not read (zeros).
  const int slot = lane % 8;
  uint32_t src_off[10];
  int src_chunk[10];
#pragma unroll
  for (int i = 0; i < 10; ++i) {
    const int line = (i < 2 ? i : i - 2) * 8 + lane / 8;
    src_chunk[i] = slot ^ (line & 7);
    if (i < 2) {
      const int row = row0 + line < M ? row0 + line : M - 1;
      src_off[i] = (uint32_t)((int64_t)row * a.x_stride_m * 2) + src_chunk[i] * 16;
    } else {
      const int col = col0 + line < N ? col0 + line : N - 1;
      src_off[i] = (uint32_t)((int64_t)col * a.w_stride_n * 2) + src_chunk[i] * 16;
    }
  }
  const int n_blocks = (K + 63) / 64;
  auto issue = [&](int kb, int st) {  // block kb (may lie past the end: nothing is read) into stage st
    const uint32_t dst = ring + st * SKINNY_STAGE;
#pragma unroll
    for (int i = 0; i < 10; ++i) {
      const uint32_t kill = kb * 64 + src_chunk[i] * 8 < K ? 0u : kOob;
      dma16(i < 2 ? rx : rw, dst + i * 1024, src_off[i] | kill, (uint32_t)kb * 128u);
    }
  };
  f32x4s_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = f32x4s_t{0.f, 0.f, 0.f, 0.f};
  issue(wave, 0);
  issue(wave + 4, 1);
  int st = 0;
#pragma unroll 1
  for (int kb = wave; kb < n_blocks; kb += 4) {
    wait_vmcnt<10>();  // copies complete in order: all but the newest block's ten have landed
    const uint8_t *sp = ringp + st * SKINNY_STAGE;
    uint4 av[2], bv[2][4];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      av[t] = *(const uint4 *)(sp + c * 128 + (((t * 4 + g) ^ (c & 7)) * 16));
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int line = j * 16 + c;
        bv[t][j] = *(const uint4 *)(sp + 2048 + line * 128 + (((t * 4 + g) ^ (line & 7)) * 16));
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // operands are in registers: the stage two ahead may reuse ...
    const int nst = st == 0 ? 2 : st - 1;                // ... the stage read one iteration ago
    issue(kb + 8, nst);
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = mma16x16x32<XDT>(av[t], bv[t][j], acc[j]);
    st = st == 2 ? 0 : st + 1;
  }
  wait_dma();
  // element i of fragment j is row 4g + i, column 16j + c
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * 16 + g * 4 + i) * SKINNY_PITCH + j * 16 + c] = acc[j][i];
  __syncthreads();
  // thread -> row tid / 16, four columns
  const int r = tid / 16, cq = (tid % 16) * 4;
  if (row0 + r >= M) return;
  float flex = 1.0f;
  if (a.x_scale) flex *= *a.x_scale;
  if (a.w_scale) flex *= *a.w_scale;
  float o[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int idx = r * SKINNY_PITCH + cq + e;
    const float v = (red[idx] + red[16 * SKINNY_PITCH + idx]) + (red[32 * SKINNY_PITCH + idx] + red[48 * SKINNY_PITCH + idx]);
    const int col = col0 + cq + e;
    const float b = (a.bias && col < N) ? load_any_f32(a.bias, a.bias_dtype, col) : 0.f;
    o[e] = (v * flex + b) * a.out_alpha;
  }
  const int64_t base = (int64_t)(row0 + r) * a.y_stride_m + col0 + cq;
  if (a.y_dtype == TAMD_F32) {
    float *yp = (float *)a.y + base;
    if (col0 + cq + 4 <= N && ((uintptr_t)yp & 15) == 0) *(float4 *)yp = make_float4(o[0], o[1], o[2], o[3]);
    else
      for (int e = 0; e < 4 && col0 + cq + e < N; ++e) yp[e] = o[e];
  } else {
    uint16_t *yp = (uint16_t *)a.y + base;
    uint32_t h[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) h[e] = a.y_dtype == TAMD_BF16 ? f32_to_bf16_bits(o[e]) : f32_to_f16_bits(o[e]);
    if (col0 + cq + 4 <= N && ((uintptr_t)yp & 7) == 0) *(uint2 *)yp = make_uint2(h[0] | (h[1] << 16), h[2] | (h[3] << 16));
    else
      for (int e = 0; e < 4 && col0 + cq + e < N; ++e) yp[e] = (uint16_t)h[e];
  }
}

// Whether the narrow kernel covers the problem: one dense product (no ragged / batched / gathered rows, no per-row
// factors, no activation, no flexpoint or microscaled output), K-contiguous weights, N <= 128, both operands
// addressable with 32-bit byte offsets.
inline bool skinny16_applicable(const tamd_matmul_args &a) {
  if (a.N > 128 || a.N < 1 || a.M < 1 || a.n_experts != 1 || a.w_stride_k != 1 || a.K % 8 != 0) return false;
  if (a.block_schedule || a.slice_sizes || a.gather_indx || a.scatter_indx || a.betas || a.gammas) return false;
  if (a.activation != TAMD_ACT_NONE || a.y_expected_scale || a.y_actual_scale || a.y_mx_scale || a.x_mx_scale) return false;
  if (a.y_dtype != a.x_dtype && a.y_dtype != TAMD_F32) return false;
  if (a.force_variant != 0) return false;
  if (!aligned(a.w, 16) || (a.w_stride_n * 2) % 16 != 0 || !aligned(a.x, 16) || (a.x_stride_m * 2) % 16 != 0) return false;
  if (a.x_stride_m < 0 || a.w_stride_n < 0) return false;
  const int64_t lim = 0x7FFFFF00;
  if (((int64_t)a.M * a.x_stride_m + a.K) * 2 >= lim || ((int64_t)a.N * a.w_stride_n + a.K) * 2 >= lim) return false;
  return true;
}

template <int XDT>
int launch_skinny16(const tamd_matmul_args &a, hipStream_t st) {
  const int64_t gm = ((int64_t)a.M + 15) / 16;
  if (gm > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
  auto kern = mm_skinny16_kernel<XDT>;
  if (int rc = raise_lds_limit_once((const void *)kern)) return rc;
  kern<<<dim3((unsigned)gm, (unsigned)((a.N + SKINNY_COLS - 1) / SKINNY_COLS)), 256, SKINNY_LDS, st>>>(a);
  return launch_status();
}

// 16-bit activations x 16-bit weights of the same type.  Returns TAMD_E_UNSUPPORTED / _ALIGNMENT for layouts
// the kernel does not cover.
template <int XDT>
int dispatch_w16(const tamd_matmul_args &a, int block_m, int grid_m, hipStream_t st) {
  if (skinny16_applicable(a)) return launch_skinny16<XDT>(a, st);
  dense_grid(a, block_m, grid_m);
  const bool kc = a.w_stride_k == 1, nc = a.w_stride_n == 1;
  if (!kc && !nc) return TAMD_E_UNSUPPORTED;
  if (a.K % 8 != 0) return TAMD_E_UNSUPPORTED;  // whole 16-byte chunks along K
  if (!kc && a.N % 8 != 0) return TAMD_E_UNSUPPORTED;  // whole 16-byte chunks along N
  const int64_t pitch = kc ? a.w_stride_n : a.w_stride_k;
  if (!aligned(a.w, 16) || (pitch * 2) % 16 != 0 || (a.w_stride_e * 2) % 16 != 0) return TAMD_E_ALIGNMENT;
  if (!aligned(a.x, 16) || (a.x_stride_m * 2) % 16 != 0 || (a.x_stride_z * 2) % 16 != 0) return TAMD_E_ALIGNMENT;
  const int64_t x_rows = a.x_rows > 0 ? a.x_rows : a.M;
  const int64_t w_span = (kc ? (int64_t)a.N * a.w_stride_n : (int64_t)a.K * a.w_stride_k) * 2;
  if (x_rows * a.x_stride_m * 2 >= (int64_t)0x7FFFFF00 || w_span >= (int64_t)0x7FFFFF00) return TAMD_E_UNSUPPORTED;
  const bool sw = a.activation == TAMD_ACT_SWIGLU;
#define TAMD_W16(BMV)                                                                                           \
  case BMV:                                                                                                     \
    if (kc) return sw ? launch_w16<XDT, BMV, TAMD_ACT_SWIGLU, true>(a, grid_m, st)                               \
                      : launch_w16<XDT, BMV, TAMD_ACT_NONE, true>(a, grid_m, st);                                 \
    return sw ? launch_w16<XDT, BMV, TAMD_ACT_SWIGLU, false>(a, grid_m, st)                                      \
              : launch_w16<XDT, BMV, TAMD_ACT_NONE, false>(a, grid_m, st);
  switch (block_m) {
    TAMD_W16(16) TAMD_W16(32) TAMD_W16(64) TAMD_W16(128)
    default: return TAMD_E_UNSUPPORTED;
  }
#undef TAMD_W16
}

}  // namespace tamd

// MXFP4 / MXFP8 quantise / dequantise for gfx950.  Bandwidth kernels: 128-bit global
// accesses, one 32-element group handled by 4 lanes (quantised axis contiguous)
// or by one lane per column set (quantised axis strided, i.e. the weight layout: tiles
// of 16 or 32 groups x 128 or 256 columns that pass through LDS).
//
// Arithmetic follows numerics_details/mxfp.py:212-363 and :384-449 of the
// reference: scale = 2^ceil(log2(max/6)) taken from the float32 bit pattern,
// q = x * (1/scale), round-to-nearest-even onto {0,.5,1,1.5,2,3,4,6}, saturate.
#include "common.h"
#include <type_traits>

namespace tamd {

// Two e2m1 codes (q0 in the low nibble) by the hardware conversion: round to nearest even onto the e2m1 grid,
// saturating at 6 (v_cvt_scalef32_pk_fp4_f32 with a unit scale).  NaN has no e2m1 code: it becomes the largest
// magnitude with the sign bit of the NaN's pattern.
TAMD_DEVICE uint32_t e2m1_pair(float q0, float q1) {
  uint32_t c = (uint32_t)__builtin_amdgcn_cvt_scalef32_pk_fp4_f32(0u, q0, q1, 1.0f, 0) & 0xFFu;
  if (q0 != q0) c = (c & 0xF0u) | 7u | ((f32_to_bits(q0) >> 28) & 8u);
  if (q1 != q1) c = (c & 0x0Fu) | ((7u | ((f32_to_bits(q1) >> 28) & 8u)) << 4);
  return c;
}

// The same conversion with the division by the group's scale (a power of two, `ds`) done by the instruction:
// writes the code pair of (a / ds, b / ds) into byte BS of `old`.  Exact wherever a / ds is: callers keep to
// scales whose reciprocal is a normal float and to groups without NaN.
template <int BS>
TAMD_DEVICE uint32_t e2m1_pair_scaled(uint32_t old, float a, float b, float ds) {
  return (uint32_t)__builtin_amdgcn_cvt_scalef32_pk_fp4_f32(old, a, b, ds, BS);
}
// 8 e2m1 codes of one column (rows l0 .. l0+7, v[i] = row l0 + i) -> one 32-bit word
TAMD_DEVICE uint32_t e2m1_word_scaled(const float (&v)[8], float ds) {
  uint32_t w = 0;
  w = e2m1_pair_scaled<0>(w, v[0], v[1], ds);
  w = e2m1_pair_scaled<1>(w, v[2], v[3], ds);
  w = e2m1_pair_scaled<2>(w, v[4], v[5], ds);
  w = e2m1_pair_scaled<3>(w, v[6], v[7], ds);
  return w;
}

// 16-byte accesses to memory that is touched once (non-temporal).  Measured on the two tile kernels below: the
// quantiser is fastest with non-temporal loads of its source and ordinary stores of the codes (110 us; 130 with
// ordinary loads), the dequantiser with ordinary loads of the codes and non-temporal stores of its rows (61 us; 67 with
// ordinary stores, 71 with both non-temporal).
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
TAMD_DEVICE uint4 load_once(const void *p) {
  u32x4_t q = __builtin_nontemporal_load((const u32x4_t *)p);
  return make_uint4(q.x, q.y, q.z, q.w);
}
TAMD_DEVICE void store_once(void *p, uint4 v) {
  __builtin_nontemporal_store(u32x4_t{v.x, v.y, v.z, v.w}, (u32x4_t *)p);
}
// the same as ordinary accesses; through the vector type so that they stay one 16-byte instruction (a 16-byte access
// through a pointer derived from char * is split into four 4-byte ones otherwise, a quarter of the bandwidth)
TAMD_DEVICE uint4 load16(const void *p) {
  u32x4_t q = *(const u32x4_t *)p;
  return make_uint4(q.x, q.y, q.z, q.w);
}
TAMD_DEVICE void store16(void *p, uint4 v) { *(u32x4_t *)p = u32x4_t{v.x, v.y, v.z, v.w}; }

// Value kinds of a microscaled tensor: e2m1 codes (two per byte), or fp8 bytes.  Largest magnitude and
// largest power of two of each (mxfp.py:206-209, mxfp_details/_downcast_to_mxfp.py:24-31).
constexpr int QK_E2M1 = 0, QK_E4M3 = 1, QK_E5M2 = 2;
template <int QK>
constexpr float kMaxQ = QK == QK_E2M1 ? 6.0f : (QK == QK_E4M3 ? 448.0f : 57344.0f);
template <int QK>
constexpr float kInvPow2Q = QK == QK_E2M1 ? 0.25f : (QK == QK_E4M3 ? 1.0f / 256.0f : 1.0f / 32768.0f);

// Returns the multiplier 1/scale and writes the e8m0 byte.
template <int QK = QK_E2M1>
TAMD_DEVICE float group_scale(float gmax, int mode, uint32_t &scale_byte) {
  uint32_t sb;
  if (mode == TAMD_ROUND_UP) {
    sb = (f32_to_bits(gmax / kMaxQ<QK>) + 0x007FFFFFu) & 0x7F800000u;
  } else {
    sb = f32_to_bits(gmax * kInvPow2Q<QK>) & 0x7F800000u;
  }
  scale_byte = sb >> 23;
  float ds = bits_to_f32(sb);
  return ds == 0.f ? 0.f : 1.0f / ds;
}

TAMD_DEVICE float e2m1_value(uint32_t code) {
  uint32_t m = code & 7u;
  uint32_t bits = m < 2u ? (m ? 0x3F000000u : 0u) : ((((m >> 1) + 126u) << 23) | ((m & 1u) << 22));
  return bits_to_f32(bits | ((code & 8u) << 28));
}

// q (already multiplied by 1/scale) -> fp8 byte: clamp to the finite range, round to nearest even (mxfp.py:313-316)
template <int QK>
TAMD_DEVICE uint32_t fp8_code(float q) {
  if (q != q) return 0x7Fu;
  const float c = __builtin_fminf(__builtin_fmaxf(q, -kMaxQ<QK>), kMaxQ<QK>);
  if constexpr (QK == QK_E4M3) return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false) & 0xFFu;
  return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(c, c, 0, false) & 0xFFu;
}
template <int QK>
TAMD_DEVICE float fp8_value(uint32_t byte) {
  if constexpr (QK == QK_E4M3) return __builtin_amdgcn_cvt_f32_fp8((int)byte, 0);
  return __builtin_amdgcn_cvt_f32_bf8((int)byte, 0);
}

template <int DT>
constexpr float kMaxFinite =
    DT == TAMD_F32 ? 3.4028234663852886e+38f : (DT == TAMD_BF16 ? 3.3895313892515355e+38f : 65504.f);

template <int DT, int QK = QK_E2M1>
TAMD_DEVICE float dequant_one(uint32_t code, float mult, bool is_nan) {
  float v = (QK == QK_E2M1 ? e2m1_value(code) : fp8_value<QK>(code)) * mult;
  constexpr float mf = kMaxFinite<DT>;
  v = v != v ? v : __builtin_fminf(__builtin_fmaxf(v, -mf), mf);
  // e5m2 has infinities: they pass through whatever the scale is (mxfp.py:438-440 of the reference)
  if (QK == QK_E5M2 && (code & 0x7Fu) == 0x7Cu) v = bits_to_f32(0x7F800000u | ((code & 0x80u) << 24));
  return is_nan ? bits_to_f32(0x7FC00000u) : v;
}

template <int DT>
TAMD_DEVICE uint32_t pack2(float a, float b) {
  if constexpr (DT == TAMD_BF16) return f32_to_bf16_bits(a) | (f32_to_bf16_bits(b) << 16);
  return f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
}

// ---------------------------------------------------------------------------
// downcast, quantised axis contiguous in the source: 4 lanes x 8 elements per group
// ---------------------------------------------------------------------------
template <int DT, bool VEC, int QK>
__global__ __launch_bounds__(256) void downcast_rows_kernel(
    const void *__restrict__ src, int64_t n_groups_total, int64_t G, int64_t nr, int64_t ssb, int64_t ssr,
    uint8_t *__restrict__ vals, int64_t vsb, int64_t vsr, uint8_t *__restrict__ scales, int64_t csb,
    int64_t csr, int mode) {
  int64_t gid = (int64_t)blockIdx.x * 64 + (threadIdx.x >> 2);
  int sub = threadIdx.x & 3;
  bool live = gid < n_groups_total;
  int64_t gg = live ? gid : 0;
  int64_t run = gg / G, g = gg - run * G;
  int64_t b = run / nr, r = run - b * nr;
  int64_t off = b * ssb + r * ssr + g * 32 + sub * 8;
  float v[8];
  if constexpr (VEC && DT == TAMD_F32) {
    const float4 *p = (const float4 *)((const float *)src + off);
    float4 a = p[0], c = p[1];
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = c.x; v[5] = c.y; v[6] = c.z; v[7] = c.w;
  } else if constexpr (VEC) {
    uint4 a = *(const uint4 *)((const uint16_t *)src + off);
    uint32_t w[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if constexpr (DT == TAMD_BF16) {
        v[2 * j] = bf16_bits_to_f32(w[j] & 0xFFFFu);
        v[2 * j + 1] = bf16_bits_to_f32(w[j] >> 16);
      } else {
        v[2 * j] = f16_bits_to_f32(w[j] & 0xFFFFu);
        v[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
      }
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = load_as_f32<DT>(src, off + j);
  }
  float m = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j) m = __builtin_fmaxf(m, __builtin_fabsf(v[j]));
  m = __builtin_fmaxf(m, __shfl_xor(m, 1));
  m = __builtin_fmaxf(m, __shfl_xor(m, 2));
  uint32_t sbyte;
  float qs = group_scale<QK>(m, mode, sbyte);
  if constexpr (QK == QK_E2M1) {
    uint32_t packed = 0;
#pragma unroll
    for (int j = 0; j < 8; j += 2) packed |= e2m1_pair(v[j] * qs, v[j + 1] * qs) << (4 * j);
    if (!live) return;
    *(uint32_t *)(vals + b * vsb + r * vsr + g * 16 + sub * 4) = packed;
  } else {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      lo |= fp8_code<QK>(v[j] * qs) << (8 * j);
      hi |= fp8_code<QK>(v[4 + j] * qs) << (8 * j);
    }
    if (!live) return;
    *(uint2 *)(vals + b * vsb + r * vsr + g * 32 + sub * 8) = make_uint2(lo, hi);
  }
  if (sub == 0) scales[b * csb + r * csr + g] = (uint8_t)sbyte;
}

// ---------------------------------------------------------------------------
// downcast, source contiguous along r (quantised axis strided), any alignment: a thread owns one column and
// walks the 32 rows of one group.  The aligned case has the tile kernel below.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void downcast_cols_kernel(
    const void *__restrict__ src, int64_t nb, int64_t G, int64_t nr, int64_t ssb, int64_t ssl,
    uint8_t *__restrict__ vals, int64_t vsb, int64_t vsr, uint8_t *__restrict__ scales, int64_t csb,
    int64_t csr, int mode) {
  // a workgroup covers 8 consecutive groups of 32 columns: the 8 lanes that share a column write 8 x 16
  // consecutive bytes of its codes (one 128-byte line) and 8 consecutive scale bytes.  The grid is
  // ceil(nr / 32) * ceil(G / 8) * nb workgroups (launch_downcast).
  int64_t blocks_r = (nr + 31) / 32;
  int64_t g_chunks = (G + 7) / 8;
  int64_t bid = blockIdx.x;
  int64_t br = bid % blocks_r;
  int64_t t = bid / blocks_r;
  int64_t g = (t % g_chunks) * 8 + threadIdx.x % 8;
  int64_t b = t / g_chunks;
  int64_t r0 = br * 32 + threadIdx.x / 8;
  if (r0 >= nr || g >= G || b >= nb) return;
  constexpr int ES = DT == TAMD_F32 ? 4 : 2;
  const char *base = (const char *)src + (b * ssb + g * 32 * ssl + r0) * ES;
  float mx = 0.f;
  float v[32];
#pragma unroll
  for (int l = 0; l < 32; ++l) {
    v[l] = load_as_f32<DT>(base, l * ssl);
    mx = __builtin_fmaxf(mx, __builtin_fabsf(v[l]));
  }
  uint32_t sbyte;
  float qs = group_scale(mx, mode, sbyte);
  uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
  for (int l = 0; l < 32; l += 2) w[l >> 3] |= e2m1_pair(v[l] * qs, v[l + 1] * qs) << (4 * (l & 7));
  *(uint4 *)(vals + b * vsb + r0 * vsr + g * 16) = make_uint4(w[0], w[1], w[2], w[3]);
  scales[b * csb + r0 * csr + g] = (uint8_t)sbyte;
}

// ---------------------------------------------------------------------------
// downcast, source contiguous along r, 16-byte aligned: a workgroup quantises a tile of GT groups x 32*NV
// columns.  A load instruction of a wave reads 512 contiguous bytes of two source rows (a thread keeps the 32
// rows of its NV columns in registers, as above); the codes pass through LDS so that they leave as GT x 16
// contiguous bytes per column.  The source is read once: its loads are non-temporal.
// ---------------------------------------------------------------------------
// groups per tile: 64 KiB of codes in LDS either way
template <int DT>
constexpr int kTileGroups = DT == TAMD_F32 ? 32 : 16;
template <int DT>
constexpr int kTileCols = 32 * (DT == TAMD_F32 ? 4 : 8);
template <int DT>
constexpr size_t kTileLds = (size_t)kTileCols<DT> * kTileGroups<DT> * 17;

template <int DT>
__global__ __launch_bounds__(256) void downcast_cols_tile_kernel(
    const void *__restrict__ src, int64_t nb, int64_t G, int64_t nr, int64_t ssb, int64_t ssl,
    uint8_t *__restrict__ vals, int64_t vsb, int64_t vsr, uint8_t *__restrict__ scales, int64_t csb,
    int64_t csr, int mode) {
  constexpr int ES = DT == TAMD_F32 ? 4 : 2;
  constexpr int NV = 16 / ES;
  constexpr int GT = kTileGroups<DT>;
  constexpr int CW = kTileCols<DT>;
  // s_codes[column][slot]: slot = group ^ (column / NV) % 8 keeps both the writes (two groups, 32 column sets
  // per wave) and the reads (GT groups of 256 / GT columns per workgroup) spread over the banks
  extern __shared__ uint4 s_tile[];
  uint4 *s_codes = s_tile;
  uint8_t *s_sc = (uint8_t *)(s_tile + CW * GT);
  const int64_t tiles_r = (nr + CW - 1) / CW;
  const int64_t g_chunks = (G + GT - 1) / GT;
  const int64_t bid = blockIdx.x;
  const int64_t br = bid % tiles_r;
  const int64_t t = bid / tiles_r;
  const int64_t gc = t % g_chunks;
  const int64_t b = t / g_chunks;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int cs = lane % 32;  // the thread's column set
  const int64_t col0 = br * CW + cs * NV;
#pragma unroll 1
  for (int pass = 0; pass < GT / 8; ++pass) {
    const int gl = pass * 8 + wave * 2 + lane / 32;
    const int64_t g = gc * GT + gl;
    if (g >= G || col0 >= nr) continue;
    const char *base = (const char *)src + (b * ssb + g * 32 * ssl + col0) * ES;
    uint4 raw[32];
#pragma unroll
    for (int l = 0; l < 32; ++l) raw[l] = load_once(base + (int64_t)l * ssl * ES);
    auto elem = [&](int l, int c) -> float {
      const uint4 &q = raw[l];
      uint32_t w[4] = {q.x, q.y, q.z, q.w};
      if constexpr (DT == TAMD_F32) return bits_to_f32(w[c]);
      uint32_t h = (c & 1) ? (w[c >> 1] >> 16) : (w[c >> 1] & 0xFFFFu);
      if constexpr (DT == TAMD_BF16) return bf16_bits_to_f32(h);
      return f16_bits_to_f32(h);
    };
    float mx[NV];
#pragma unroll
    for (int c = 0; c < NV; ++c) mx[c] = 0.f;
#pragma unroll
    for (int l = 0; l < 32; ++l)
#pragma unroll
      for (int c = 0; c < NV; ++c) mx[c] = __builtin_fmaxf(mx[c], __builtin_fabsf(elem(l, c)));
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      bool has_nan = false;
#pragma unroll
      for (int l = 0; l < 32; l += 2) has_nan |= __builtin_isunordered(elem(l, c), elem(l + 1, c));
      uint32_t sbyte;
      float qs = group_scale(mx[c], mode, sbyte);
      uint32_t w[4] = {0, 0, 0, 0};
      if (!has_nan && sbyte - 2u <= 251u) {
        // the usual case: the instruction divides by the scale and packs, 1.5 operations per element
        const float ds = bits_to_f32(sbyte << 23);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float v[8] = {elem(8 * j, c),     elem(8 * j + 1, c), elem(8 * j + 2, c), elem(8 * j + 3, c),
                              elem(8 * j + 4, c), elem(8 * j + 5, c), elem(8 * j + 6, c), elem(8 * j + 7, c)};
          w[j] = e2m1_word_scaled(v, ds);
        }
      } else {
#pragma unroll
        for (int l = 0; l < 32; l += 2)
          w[l >> 3] |= e2m1_pair(elem(l, c) * qs, elem(l + 1, c) * qs) << (4 * (l & 7));
      }
      const int cl = cs * NV + c;
      s_codes[cl * GT + (gl ^ (cs & 7))] = make_uint4(w[0], w[1], w[2], w[3]);
      s_sc[cl * GT + gl] = (uint8_t)sbyte;
    }
  }
  __syncthreads();
  const int64_t n_g = G - gc * GT < GT ? G - gc * GT : GT;
  const int64_t n_c = nr - br * CW < CW ? nr - br * CW : CW;
  uint8_t *vbase = vals + b * vsb + br * CW * vsr + gc * GT * 16;
  uint8_t *sbase = scales + b * csb + br * CW * csr + gc * GT;
  const int part = threadIdx.x % GT;
  if (part < n_g) {
#pragma unroll 4
    for (int c = threadIdx.x / GT; c < n_c; c += 256 / GT) {
      store16(vbase + (int64_t)c * vsr + part * 16, s_codes[c * GT + (part ^ ((c / NV) & 7))]);
      sbase[(int64_t)c * csr + part] = s_sc[c * GT + part];
    }
  }
}

// ---------------------------------------------------------------------------
// upcast, destination contiguous along the quantised axis
// ---------------------------------------------------------------------------
template <int DT, int QK>
__global__ __launch_bounds__(256) void upcast_rows_kernel(
    const uint8_t *__restrict__ vals, int64_t vsb, int64_t vsr, const uint8_t *__restrict__ scales,
    int64_t csb, int64_t csr, void *__restrict__ dst, int64_t n_groups_total, int64_t G, int64_t nr,
    int64_t dsb, int64_t dsr, int vec_ok) {
  int64_t gid = (int64_t)blockIdx.x * 64 + (threadIdx.x >> 2);
  int sub = threadIdx.x & 3;
  if (gid >= n_groups_total) return;
  int64_t run = gid / G, g = gid - run * G;
  int64_t b = run / nr, r = run - b * nr;
  uint32_t s = scales[b * csb + r * csr + g];
  float mult = bits_to_f32(s << 23);
  bool is_nan = s == 0xFFu;
  float o[8];
  if constexpr (QK == QK_E2M1) {
    uint32_t packed = *(const uint32_t *)(vals + b * vsb + r * vsr + g * 16 + sub * 4);
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = dequant_one<DT>((packed >> (4 * j)) & 0xFu, mult, is_nan);
  } else {
    const uint2 w = *(const uint2 *)(vals + b * vsb + r * vsr + g * 32 + sub * 8);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      o[j] = dequant_one<DT, QK>((w.x >> (8 * j)) & 0xFFu, mult, is_nan);
      o[4 + j] = dequant_one<DT, QK>((w.y >> (8 * j)) & 0xFFu, mult, is_nan);
    }
  }
  int64_t off = b * dsb + r * dsr + g * 32 + sub * 8;
  if (vec_ok) {
    if constexpr (DT == TAMD_F32) {
      float4 *p = (float4 *)((float *)dst + off);
      p[0] = make_float4(o[0], o[1], o[2], o[3]);
      p[1] = make_float4(o[4], o[5], o[6], o[7]);
    } else {
      *(uint4 *)((uint16_t *)dst + off) =
          make_uint4(pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3]), pack2<DT>(o[4], o[5]), pack2<DT>(o[6], o[7]));
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) store_from_f32<DT>(dst, off + j, o[j]);
  }
}

// ---------------------------------------------------------------------------
// upcast, destination contiguous along r, any alignment: a thread owns one column of one group.  The aligned
// case has the tile kernel below.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void upcast_cols_kernel(
    const uint8_t *__restrict__ vals, int64_t vsb, int64_t vsr, const uint8_t *__restrict__ scales,
    int64_t csb, int64_t csr, void *__restrict__ dst, int64_t nb, int64_t G, int64_t nr, int64_t dsb,
    int64_t dsl) {
  // a workgroup covers 8 consecutive groups of 32 columns: the 8 lanes that share a column read 8 x 16
  // consecutive bytes of its codes (one 128-byte line) and 8 consecutive scale bytes.  The grid is
  // ceil(nr / 32) * ceil(G / 8) * nb workgroups (launch_upcast).
  int64_t blocks_r = (nr + 31) / 32;
  int64_t g_chunks = (G + 7) / 8;
  int64_t bid = blockIdx.x;
  int64_t br = bid % blocks_r;
  int64_t t = bid / blocks_r;
  int64_t g = (t % g_chunks) * 8 + threadIdx.x % 8;
  int64_t b = t / g_chunks;
  int64_t r0 = br * 32 + threadIdx.x / 8;
  if (r0 >= nr || g >= G || b >= nb) return;
  const uint4 code = *(const uint4 *)(vals + b * vsb + r0 * vsr + g * 16);
  const uint32_t s = scales[b * csb + r0 * csr + g];
  const float mult = bits_to_f32(s << 23);
  const bool isn = s == 0xFFu;
  constexpr int ES = DT == TAMD_F32 ? 4 : 2;
  char *base = (char *)dst + (b * dsb + g * 32 * dsl + r0) * ES;
  const uint32_t w[4] = {code.x, code.y, code.z, code.w};
#pragma unroll
  for (int l = 0; l < 32; ++l)
    store_from_f32<DT>(base + (int64_t)l * dsl * ES, 0, dequant_one<DT>((w[l >> 3] >> (4 * (l & 7))) & 0xFu, mult, isn));
}

// Scale bytes for which 0.5 * 2^(s-127) and 6 * 2^(s-127) are normal numbers of the destination type: there the
// product needs neither the clamp to the largest finite value nor any care about denormals.
template <int DT>
constexpr uint32_t kFastLo = DT == TAMD_F16 ? 127u - 13u : 3u;
template <int DT>
constexpr uint32_t kFastHi = DT == TAMD_F16 ? 127u + 13u : 252u;

// Rows l and l+1 (the code pairs in byte BS of w[c]) of a thread's 16 / sizeof(element) columns, dequantised by the
// conversion instruction and stored as two 16-byte pieces `pitch` bytes apart.
template <int DT, int BS>
TAMD_DEVICE void upcast_rows2_regs(const uint32_t *w, const float *mult, uint4 &r0, uint4 &r1) {
  if constexpr (DT == TAMD_F32) {
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    f32x2_t v[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) v[c] = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(w[c], mult[c], BS);
    r0 = make_uint4(f32_to_bits(v[0].x), f32_to_bits(v[1].x), f32_to_bits(v[2].x), f32_to_bits(v[3].x));
    r1 = make_uint4(f32_to_bits(v[0].y), f32_to_bits(v[1].y), f32_to_bits(v[2].y), f32_to_bits(v[3].y));
  } else {
    uint32_t u[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) {
      if constexpr (DT == TAMD_BF16) {
        typedef __bf16 bf16x2v_t __attribute__((ext_vector_type(2)));
        bf16x2v_t t = __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w[c], mult[c], BS);
        u[c] = __builtin_bit_cast(uint32_t, t);
      } else {
        typedef _Float16 f16x2v_t __attribute__((ext_vector_type(2)));
        f16x2v_t t = __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(w[c], mult[c], BS);
        u[c] = __builtin_bit_cast(uint32_t, t);
      }
    }
    // u[c] = (row l, row l+1) of column c; a stored word is (column 2i, column 2i+1) of one row
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[i] = __builtin_amdgcn_perm(u[2 * i + 1], u[2 * i], 0x05040100u);
      hi[i] = __builtin_amdgcn_perm(u[2 * i + 1], u[2 * i], 0x07060302u);
    }
    r0 = make_uint4(lo[0], lo[1], lo[2], lo[3]);
    r1 = make_uint4(hi[0], hi[1], hi[2], hi[3]);
  }
}
template <int DT, int BS>
TAMD_DEVICE void upcast_rows2(const uint32_t *w, const float *mult, char *p, int64_t pitch) {
  uint4 r0, r1;
  upcast_rows2_regs<DT, BS>(w, mult, r0, r1);
  store_once(p, r0);
  store_once(p + pitch, r1);
}

// ---------------------------------------------------------------------------
// upcast, destination contiguous along r, 16-byte aligned: the mirror image of downcast_cols_tile_kernel.  The
// codes and scales of a tile of GT groups x 32*NV columns come in as GT x 16 contiguous bytes per column, pass
// through LDS, and a store instruction of a wave writes 512 contiguous bytes of two destination rows.
// ---------------------------------------------------------------------------
template <int DT>
__global__ __launch_bounds__(256) void upcast_cols_tile_kernel(
    const uint8_t *__restrict__ vals, int64_t vsb, int64_t vsr, const uint8_t *__restrict__ scales,
    int64_t csb, int64_t csr, void *__restrict__ dst, int64_t nb, int64_t G, int64_t nr, int64_t dsb,
    int64_t dsl) {
  constexpr int ES = DT == TAMD_F32 ? 4 : 2;
  constexpr int NV = 16 / ES;
  constexpr int GT = kTileGroups<DT>;
  constexpr int CW = kTileCols<DT>;
  extern __shared__ uint4 s_tile[];
  uint4 *s_codes = s_tile;
  uint8_t *s_sc = (uint8_t *)(s_tile + CW * GT);
  const int64_t tiles_r = (nr + CW - 1) / CW;
  const int64_t g_chunks = (G + GT - 1) / GT;
  const int64_t bid = blockIdx.x;
  const int64_t br = bid % tiles_r;
  const int64_t t = bid / tiles_r;
  const int64_t gc = t % g_chunks;
  const int64_t b = t / g_chunks;
  const int64_t n_g = G - gc * GT < GT ? G - gc * GT : GT;
  const int64_t n_c = nr - br * CW < CW ? nr - br * CW : CW;
  const uint8_t *vbase = vals + b * vsb + br * CW * vsr + gc * GT * 16;
  const uint8_t *sbase = scales + b * csb + br * CW * csr + gc * GT;
  const int part = threadIdx.x % GT;
  if (part < n_g) {
#pragma unroll 4
    for (int c = threadIdx.x / GT; c < n_c; c += 256 / GT) {
      s_codes[c * GT + (part ^ ((c / NV) & 7))] = load16(vbase + (int64_t)c * vsr + part * 16);
      s_sc[c * GT + part] = sbase[(int64_t)c * csr + part];
    }
  }
  __syncthreads();
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int cs = lane % 32;
  const int64_t col0 = br * CW + cs * NV;
#pragma unroll 1
  for (int pass = 0; pass < GT / 8; ++pass) {
    const int gl = pass * 8 + wave * 2 + lane / 32;
    const int64_t g = gc * GT + gl;
    if (g >= G || col0 >= nr) continue;
    uint4 code[NV];
    float mult[NV];
    bool isn[NV];
    bool fast = true;
#pragma unroll
    for (int c = 0; c < NV; ++c) {
      const int cl = cs * NV + c;
      code[c] = s_codes[cl * GT + (gl ^ (cs & 7))];
      uint32_t s = s_sc[cl * GT + gl];
      mult[c] = bits_to_f32(s << 23);
      isn[c] = s == 0xFFu;
      fast &= s - kFastLo<DT> <= kFastHi<DT> - kFastLo<DT>;
    }
    char *base = (char *)dst + (b * dsb + g * 32 * dsl + col0) * ES;
    if (fast) {
      // the usual case: every product code * scale is a normal number of the destination type, and the
      // conversion instruction yields it for two rows of a column at once
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint32_t w[NV];
#pragma unroll
        for (int c = 0; c < NV; ++c) w[c] = j == 0 ? code[c].x : (j == 1 ? code[c].y : (j == 2 ? code[c].z : code[c].w));
        upcast_rows2<DT, 0>(w, mult, base + (int64_t)(8 * j + 0) * dsl * ES, dsl * ES);
        upcast_rows2<DT, 1>(w, mult, base + (int64_t)(8 * j + 2) * dsl * ES, dsl * ES);
        upcast_rows2<DT, 2>(w, mult, base + (int64_t)(8 * j + 4) * dsl * ES, dsl * ES);
        upcast_rows2<DT, 3>(w, mult, base + (int64_t)(8 * j + 6) * dsl * ES, dsl * ES);
      }
      continue;
    }
#pragma unroll
    for (int l = 0; l < 32; ++l) {
      float o[NV];
#pragma unroll
      for (int c = 0; c < NV; ++c) {
        uint32_t w[4] = {code[c].x, code[c].y, code[c].z, code[c].w};
        o[c] = dequant_one<DT>((w[l >> 3] >> (4 * (l & 7))) & 0xFu, mult[c], isn[c]);
      }
      char *p = base + (int64_t)l * dsl * ES;
      if constexpr (DT == TAMD_F32) {
        store_once(p, make_uint4(f32_to_bits(o[0]), f32_to_bits(o[1]), f32_to_bits(o[2]), f32_to_bits(o[3])));
      } else {
        store_once(p, make_uint4(pack2<DT>(o[0], o[1]), pack2<DT>(o[2], o[3]), pack2<DT>(o[4], o[5]),
                                 pack2<DT>(o[6], o[7])));
      }
    }
  }
}

template <int DT, int QK>
int launch_downcast(const void *src, int64_t nb, int64_t L, int64_t nr, int64_t ssb, int64_t ssl, int64_t ssr,
                    uint8_t *vals, int64_t vsb, int64_t vsr, uint8_t *scales, int64_t csb, int64_t csr,
                    int mode, hipStream_t st) {
  const int64_t G = L / 32;
  constexpr int ES = DT == TAMD_F32 ? 4 : 2;
  if (ssl == 1) {
    int64_t total = nb * nr * G;
    bool vec = aligned(src, 16) && (ssb * ES) % 16 == 0 && (ssr * ES) % 16 == 0;
    int64_t blocks = (total + 63) / 64;
    if (blocks > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
    if (vec)
      downcast_rows_kernel<DT, true, QK><<<dim3((unsigned)blocks), 256, 0, st>>>(src, total, G, nr, ssb, ssr, vals,
                                                                            vsb, vsr, scales, csb, csr, mode);
    else
      downcast_rows_kernel<DT, false, QK><<<dim3((unsigned)blocks), 256, 0, st>>>(src, total, G, nr, ssb, ssr, vals,
                                                                             vsb, vsr, scales, csb, csr, mode);
    return launch_status();
  }
  if (ssr != 1) return TAMD_E_INVALID;
  if constexpr (QK != QK_E2M1) return TAMD_E_UNSUPPORTED;  // fp8 values: quantised axis contiguous only
  constexpr int NV = 16 / ES;
  bool vec = nr % NV == 0 && aligned(src, 16) && (ssb * ES) % 16 == 0 && (ssl * ES) % 16 == 0;
  if (vec) {
    constexpr int CW = kTileCols<DT>, GT = kTileGroups<DT>;
    int64_t blocks = ((nr + CW - 1) / CW) * ((G + GT - 1) / GT) * nb;
    if (blocks > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
    if (int rc = raise_lds_limit_once((const void *)downcast_cols_tile_kernel<DT>)) return rc;
    downcast_cols_tile_kernel<DT><<<dim3((unsigned)blocks), 256, kTileLds<DT>, st>>>(src, nb, G, nr, ssb, ssl, vals, vsb, vsr,
                                                                         scales, csb, csr, mode);
  } else {
    int64_t blocks = ((nr + 31) / 32) * ((G + 7) / 8) * nb;
    if (blocks > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
    downcast_cols_kernel<DT><<<dim3((unsigned)blocks), 256, 0, st>>>(src, nb, G, nr, ssb, ssl, vals, vsb, vsr,
                                                                       scales, csb, csr, mode);
  }
  return launch_status();
}

template <int DT, int QK>
int launch_upcast(const uint8_t *vals, int64_t vsb, int64_t vsr, const uint8_t *scales, int64_t csb, int64_t csr,
                  void *dst, int64_t nb, int64_t L, int64_t nr, int64_t dsb, int64_t dsl, int64_t dsr,
                  hipStream_t st) {
  const int64_t G = L / 32;
  constexpr int ES = DT == TAMD_F32 ? 4 : 2;
  if (dsl == 1) {
    int64_t total = nb * nr * G;
    int vec = aligned(dst, 16) && (dsb * ES) % 16 == 0 && (dsr * ES) % 16 == 0;
    int64_t blocks = (total + 63) / 64;
    if (blocks > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
    upcast_rows_kernel<DT, QK><<<dim3((unsigned)blocks), 256, 0, st>>>(vals, vsb, vsr, scales, csb, csr, dst, total, G,
                                                                  nr, dsb, dsr, vec);
    return launch_status();
  }
  if (dsr != 1) return TAMD_E_INVALID;
  if constexpr (QK != QK_E2M1) return TAMD_E_UNSUPPORTED;  // fp8 values: quantised axis contiguous only
  constexpr int NV = 16 / ES;
  bool vec = nr % NV == 0 && aligned(dst, 16) && (dsb * ES) % 16 == 0 && (dsl * ES) % 16 == 0;
  if (vec) {
    constexpr int CW = kTileCols<DT>, GT = kTileGroups<DT>;
    int64_t blocks = ((nr + CW - 1) / CW) * ((G + GT - 1) / GT) * nb;
    if (blocks > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
    if (int rc = raise_lds_limit_once((const void *)upcast_cols_tile_kernel<DT>)) return rc;
    upcast_cols_tile_kernel<DT><<<dim3((unsigned)blocks), 256, kTileLds<DT>, st>>>(vals, vsb, vsr, scales, csb, csr, dst, nb, G,
                                                                       nr, dsb, dsl);
  } else {
    int64_t blocks = ((nr + 31) / 32) * ((G + 7) / 8) * nb;
    if (blocks > 0x7FFFFFFF) return TAMD_E_UNSUPPORTED;
    upcast_cols_kernel<DT><<<dim3((unsigned)blocks), 256, 0, st>>>(vals, vsb, vsr, scales, csb, csr, dst, nb, G,
                                                                     nr, dsb, dsl);
  }
  return launch_status();
}

// e2m1 codes -> float8_e4m3fn bytes, exactly: every e2m1 number (0, .5, 1, 1.5, 2, 3, 4, 6 and their negatives) is an
// e4m3 number.  A thread widens 16 packed bytes (32 codes, low nibble first) of a row to 32 bytes.
__global__ __launch_bounds__(256) void widen_e2m1_rows_kernel(const uint8_t *__restrict__ src, int64_t rows, int64_t row_bytes,
                                                              int64_t src_stride, uint8_t *__restrict__ dst, int64_t dst_stride,
                                                              int vec) {
  // magnitudes 0..7 as e4m3 bytes, one table entry per byte of two 32-bit words
  constexpr uint32_t kLo = 0x3C383000u, kHi = 0x4C484440u;  // {0x00, 0x30, 0x38, 0x3C}, {0x40, 0x44, 0x48, 0x4C}
  auto widen = [&](uint32_t code) -> uint32_t {              // one nibble -> one byte
    const uint32_t mag = code & 7u;
    const uint32_t tab = mag < 4u ? kLo : kHi;
    return ((tab >> (8 * (mag & 3u))) & 0xFFu) | ((code & 8u) << 4);
  };
  auto widen4 = [&](uint32_t two_bytes) -> uint32_t {        // four nibbles (16 bits) -> four bytes
    return widen(two_bytes) | (widen(two_bytes >> 4) << 8) | (widen(two_bytes >> 8) << 16) | (widen(two_bytes >> 12) << 24);
  };
  const int64_t chunks = (row_bytes + 15) / 16, total = rows * chunks;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t r = i / chunks, c = (i - r * chunks) * 16;
    const uint8_t *sp = src + r * src_stride + c;
    uint8_t *dp = dst + r * dst_stride + 2 * c;
    if (vec && c + 16 <= row_bytes) {
      const uint4 q = *(const uint4 *)sp;
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
      uint32_t o[8];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        o[2 * j] = widen4(w[j] & 0xFFFFu);
        o[2 * j + 1] = widen4(w[j] >> 16);
      }
      *(uint4 *)dp = make_uint4(o[0], o[1], o[2], o[3]);
      *(uint4 *)(dp + 16) = make_uint4(o[4], o[5], o[6], o[7]);
    } else {
      for (int64_t b = 0; b < 16 && c + b < row_bytes; ++b) {
        const uint32_t v = sp[b];
        dp[2 * b] = (uint8_t)widen(v);
        dp[2 * b + 1] = (uint8_t)widen(v >> 4);
      }
    }
  }
}

}  // namespace tamd

using namespace tamd;

extern "C" int tamd_widen_mxfp4_rows(const uint8_t *src, int64_t rows, int64_t row_bytes, int64_t src_stride, uint8_t *dst,
                                     int64_t dst_stride, void *stream) {
  if (rows < 0 || row_bytes < 0) return TAMD_E_INVALID;
  if (rows == 0 || row_bytes == 0) return 0;
  if (!src || !dst) return TAMD_E_INVALID;
  const int vec = aligned(src, 16) && aligned(dst, 16) && src_stride % 16 == 0 && dst_stride % 16 == 0;
  int64_t blocks = (rows * ((row_bytes + 15) / 16) + 255) / 256;
  blocks = blocks > 65536 * 16 ? 65536 * 16 : blocks;
  widen_e2m1_rows_kernel<<<dim3((unsigned)blocks), 256, 0, (hipStream_t)stream>>>(src, rows, row_bytes, src_stride, dst,
                                                                                 dst_stride, vec);
  return launch_status();
}

extern "C" int tamd_downcast_mxfp(const void *src, int src_dtype, int64_t nb, int64_t L, int64_t nr,
                                  int64_t src_stride_b, int64_t src_stride_l, int64_t src_stride_r,
                                  void *out_vals, int out_dtype, int64_t val_stride_b, int64_t val_stride_r,
                                  uint8_t *out_scales, int64_t scale_stride_b, int64_t scale_stride_r,
                                  int rounding_mode, void *stream) {
  if (nb < 0 || L < 0 || nr < 0 || L % 32 != 0) return TAMD_E_INVALID;
  if (rounding_mode != TAMD_ROUND_UP && rounding_mode != TAMD_ROUND_DOWN) return TAMD_E_INVALID;
  if (out_dtype != TAMD_MXFP4 && out_dtype != TAMD_FP8_E4M3 && out_dtype != TAMD_FP8_E5M2) return TAMD_E_INVALID;
  if (nb == 0 || L == 0 || nr == 0) return 0;
  if (!src || !out_vals || !out_scales) return TAMD_E_INVALID;
  if (!aligned(out_vals, 16) || val_stride_b % 16 != 0 || val_stride_r % 16 != 0) return TAMD_E_ALIGNMENT;
  hipStream_t st = (hipStream_t)stream;
  uint8_t *v = (uint8_t *)out_vals;
#define TAMD_DOWN(DT, QK)                                                                                          \
  return launch_downcast<DT, QK>(src, nb, L, nr, src_stride_b, src_stride_l, src_stride_r, v, val_stride_b,          \
                                 val_stride_r, out_scales, scale_stride_b, scale_stride_r, rounding_mode, st)
#define TAMD_DOWN_SRC(QK)                      \
  switch (src_dtype) {                         \
    case TAMD_F32: TAMD_DOWN(TAMD_F32, QK);    \
    case TAMD_BF16: TAMD_DOWN(TAMD_BF16, QK);  \
    case TAMD_F16: TAMD_DOWN(TAMD_F16, QK);    \
    default: return TAMD_E_INVALID;            \
  }
  if (out_dtype == TAMD_MXFP4) TAMD_DOWN_SRC(QK_E2M1)
  if (out_dtype == TAMD_FP8_E4M3) TAMD_DOWN_SRC(QK_E4M3)
  TAMD_DOWN_SRC(QK_E5M2)
#undef TAMD_DOWN_SRC
#undef TAMD_DOWN
}

extern "C" int tamd_upcast_mxfp(const void *vals, int val_dtype, int64_t val_stride_b, int64_t val_stride_r,
                                const uint8_t *scales, int64_t scale_stride_b, int64_t scale_stride_r, void *dst,
                                int dst_dtype, int64_t nb, int64_t L, int64_t nr, int64_t dst_stride_b,
                                int64_t dst_stride_l, int64_t dst_stride_r, void *stream) {
  if (nb < 0 || L < 0 || nr < 0 || L % 32 != 0) return TAMD_E_INVALID;
  if (val_dtype != TAMD_MXFP4 && val_dtype != TAMD_FP8_E4M3 && val_dtype != TAMD_FP8_E5M2) return TAMD_E_INVALID;
  if (nb == 0 || L == 0 || nr == 0) return 0;
  if (!vals || !scales || !dst) return TAMD_E_INVALID;
  if (!aligned(vals, 16) || val_stride_b % 16 != 0 || val_stride_r % 16 != 0) return TAMD_E_ALIGNMENT;
  hipStream_t st = (hipStream_t)stream;
  const uint8_t *v = (const uint8_t *)vals;
#define TAMD_UP(DT, QK)                                                                                              \
  return launch_upcast<DT, QK>(v, val_stride_b, val_stride_r, scales, scale_stride_b, scale_stride_r, dst, nb, L, nr, \
                               dst_stride_b, dst_stride_l, dst_stride_r, st)
#define TAMD_UP_DST(QK)                      \
  switch (dst_dtype) {                       \
    case TAMD_F32: TAMD_UP(TAMD_F32, QK);    \
    case TAMD_BF16: TAMD_UP(TAMD_BF16, QK);  \
    case TAMD_F16: TAMD_UP(TAMD_F16, QK);    \
    default: return TAMD_E_INVALID;          \
  }
  if (val_dtype == TAMD_MXFP4) TAMD_UP_DST(QK_E2M1)
  if (val_dtype == TAMD_FP8_E4M3) TAMD_UP_DST(QK_E4M3)
  TAMD_UP_DST(QK_E5M2)
#undef TAMD_UP_DST
#undef TAMD_UP
}

// Bandwidth kernels next to the matmul: the top-k combine (sum over the middle
// axis with optional mask / scale) and the standalone interleaved SwiGLU.
#include "common.h"
#include <type_traits>

namespace tamd {

// swiglu_details/_swiglu.py:55-65: gate clamped from above, linear clamped to
// [-limit, limit], s = g / (1 + exp(-alpha g)), out = fma(s, l, s).
TAMD_DEVICE float swiglu_f32(float g, float l, float alpha, float limit, bool has_limit) {
  if (has_limit) {
    g = __builtin_fminf(g, limit);
    l = __builtin_fminf(__builtin_fmaxf(l, -limit), limit);
  }
  float s = g / (1.0f + expf(-alpha * g));
  return __builtin_fmaf(s, l, s);
}

template <int DT>
__global__ __launch_bounds__(256) void swiglu_kernel(const void *__restrict__ a, int64_t M, int64_t N,
                                                     int64_t a_stride, void *__restrict__ out, int64_t o_stride,
                                                     float alpha, float limit, int has_limit) {
  int64_t total = M * N;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    int64_t m = i / N, n = i - m * N;
    float g = load_as_f32<DT>(a, m * a_stride + 2 * n);
    float l = load_as_f32<DT>(a, m * a_stride + 2 * n + 1);
    store_from_f32<DT>(out, m * o_stride + n, swiglu_f32(g, l, alpha, limit, has_limit != 0));
  }
}

// Four outputs (eight interleaved inputs) per thread: rows and pitches aligned so that a thread's inputs are one or
// two 16-byte loads and its outputs one 8- or 16-byte store.
template <int DT>
__global__ __launch_bounds__(256) void swiglu_vec4_kernel(const void *__restrict__ a, int64_t M, int64_t N,
                                                          int64_t a_stride, void *__restrict__ out, int64_t o_stride,
                                                          float alpha, float limit, int has_limit) {
  const int64_t nq = N / 4, total = M * nq;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t m = i / nq, n = (i - m * nq) * 4;
    float v[8];
    if constexpr (DT == TAMD_F32) {
      const float4 lo = *(const float4 *)((const float *)a + m * a_stride + 2 * n);
      const float4 hi = *(const float4 *)((const float *)a + m * a_stride + 2 * n + 4);
      v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4] = hi.x, v[5] = hi.y, v[6] = hi.z, v[7] = hi.w;
    } else {
      const uint4 q = *(const uint4 *)((const uint16_t *)a + m * a_stride + 2 * n);
      const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        v[2 * j] = DT == TAMD_BF16 ? bf16_bits_to_f32(w[j] & 0xFFFFu) : f16_bits_to_f32(w[j] & 0xFFFFu);
        v[2 * j + 1] = DT == TAMD_BF16 ? bf16_bits_to_f32(w[j] >> 16) : f16_bits_to_f32(w[j] >> 16);
      }
    }
    float o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) o[j] = swiglu_f32(v[2 * j], v[2 * j + 1], alpha, limit, has_limit != 0);
    if constexpr (DT == TAMD_F32) {
      *(float4 *)((float *)out + m * o_stride + n) = make_float4(o[0], o[1], o[2], o[3]);
    } else {
      uint32_t w[2];
#pragma unroll
      for (int j = 0; j < 2; ++j)
        w[j] = DT == TAMD_BF16 ? ((f32_to_bf16_bits(o[2 * j]) & 0xFFFFu) | (f32_to_bf16_bits(o[2 * j + 1]) << 16))
                               : ((f32_to_f16_bits(o[2 * j]) & 0xFFFFu) | (f32_to_f16_bits(o[2 * j + 1]) << 16));
      *(uint2 *)((uint16_t *)out + m * o_stride + n) = make_uint2(w[0], w[1]);
    }
  }
}

// x [S0, R, S1] -> y [S0, S1].  VEC elements of the inner axis per thread when
// the inner stride is 1 and everything is 16-byte aligned.
template <int XDT, int YDT, int VEC>
__global__ __launch_bounds__(256) void reduce_kernel(const void *__restrict__ x, int64_t S0, int64_t R, int64_t S1,
                                                     int64_t xs0, int64_t xsr, int64_t xs1,
                                                     const uint8_t *__restrict__ mask, int64_t ms0, int64_t msr,
                                                     int64_t ms1, const float *__restrict__ scale, int64_t ss0,
                                                     int64_t ssr, int64_t ss1, void *__restrict__ y, int64_t ys0,
                                                     int64_t ys1) {
  const int64_t nv = (S1 + VEC - 1) / VEC;
  const int64_t total = S0 * nv;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
    const int64_t s0 = total <= 0x7FFFFFFF ? (int64_t)((uint32_t)i / (uint32_t)nv) : i / nv, c0 = (i - s0 * nv) * VEC;
    // the first term starts the sum when the axis has at most 8 entries (reduce.py:137, 467-470 of the reference: a
    // column of -0.0 stays -0.0), which is what a start from -0.0 does; longer axes start from +0.0
    const float acc0 = (R > 0 && R <= 8) ? -0.0f : 0.0f;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = acc0;
    int64_t r = 0;
    if constexpr (VEC == 8) {
      // plain sums (no mask, no scale: the top-k combine) fetch four rows at a time so that their loads overlap;
      // the additions keep the order r = 0, 1, 2, ...
      if (!scale && !mask) {
        const uint16_t *xp = (const uint16_t *)x + s0 * xs0 + c0;
        for (; r + 4 <= R; r += 4) {
          uint4 q[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) q[u] = *(const uint4 *)(xp + (r + u) * xsr);
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const uint32_t w[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
              if constexpr (XDT == TAMD_BF16) {
                acc[2 * j] += bf16_bits_to_f32(w[j] & 0xFFFFu);
                acc[2 * j + 1] += bf16_bits_to_f32(w[j] >> 16);
              } else {
                acc[2 * j] += f16_bits_to_f32(w[j] & 0xFFFFu);
                acc[2 * j + 1] += f16_bits_to_f32(w[j] >> 16);
              }
            }
          }
        }
      }
    }
    for (; r < R; ++r) {
      float v[VEC];
      if constexpr (VEC == 1) {
        v[0] = load_as_f32<XDT>(x, s0 * xs0 + r * xsr + c0 * xs1);
      } else if constexpr (XDT == TAMD_F32) {
        float4 q = *(const float4 *)((const float *)x + s0 * xs0 + r * xsr + c0);
        v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
      } else {
        uint4 q = *(const uint4 *)((const uint16_t *)x + s0 * xs0 + r * xsr + c0);
        uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          if constexpr (XDT == TAMD_BF16) {
            v[2 * j] = bf16_bits_to_f32(w[j] & 0xFFFFu);
            v[2 * j + 1] = bf16_bits_to_f32(w[j] >> 16);
          } else {
            v[2 * j] = f16_bits_to_f32(w[j] & 0xFFFFu);
            v[2 * j + 1] = f16_bits_to_f32(w[j] >> 16);
          }
        }
      }
#pragma unroll
      for (int j = 0; j < VEC; ++j) {
        float t = v[j];
        if (scale) t = __builtin_fmaf(t, scale[s0 * ss0 + r * ssr + (c0 + j) * ss1], 0.0f);  // reduce.py:466
        if (mask && !mask[s0 * ms0 + r * msr + (c0 + j) * ms1]) t = 0.f;
        acc[j] += t;
      }
    }
    if constexpr (VEC > 1) {
      // the vector form has S1 % VEC == 0: with a dense, aligned output row the VEC results leave as 16-byte stores
      // (element-wise 2-byte stores at a 16-byte lane pitch use an eighth of every write they cause)
      constexpr int YS = YDT == TAMD_F32 ? 4 : 2;
      uint8_t *yp = (uint8_t *)y + (s0 * ys0 + c0) * YS;
      constexpr int ALIGN = VEC * YS < 16 ? VEC * YS : 16;
      if (ys1 == 1 && (((uintptr_t)yp) & (ALIGN - 1)) == 0) {
        if constexpr (YDT == TAMD_F32) {
#pragma unroll
          for (int j = 0; j < VEC; j += 4) *(float4 *)(yp + j * 4) = make_float4(acc[j], acc[j + 1], acc[j + 2], acc[j + 3]);
        } else {
          uint32_t w[VEC / 2];
#pragma unroll
          for (int j = 0; j < VEC / 2; ++j) {
            if constexpr (YDT == TAMD_BF16) w[j] = (f32_to_bf16_bits(acc[2 * j]) & 0xFFFFu) | (f32_to_bf16_bits(acc[2 * j + 1]) << 16);
            else w[j] = (f32_to_f16_bits(acc[2 * j]) & 0xFFFFu) | (f32_to_f16_bits(acc[2 * j + 1]) << 16);
          }
          if constexpr (VEC == 8) *(uint4 *)yp = make_uint4(w[0], w[1], w[2], w[3]);
          else *(uint2 *)yp = make_uint2(w[0], w[1]);
        }
        continue;
      }
    }
#pragma unroll
    for (int j = 0; j < VEC; ++j)
      if (c0 + j < S1) store_from_f32<YDT>(y, s0 * ys0 + (c0 + j) * ys1, acc[j]);
  }
}

template <int XDT, int YDT>
int launch_reduce(const void *x, int64_t S0, int64_t R, int64_t S1, int64_t xs0, int64_t xsr, int64_t xs1,
                  const uint8_t *mask, int64_t ms0, int64_t msr, int64_t ms1, const float *scale, int64_t ss0,
                  int64_t ssr, int64_t ss1, void *y, int64_t ys0, int64_t ys1, hipStream_t st) {
  constexpr int ES = XDT == TAMD_F32 ? 4 : 2;
  constexpr int NV = 16 / ES;
  bool vec = xs1 == 1 && S1 % NV == 0 && aligned(x, 16) && (xs0 * ES) % 16 == 0 && (xsr * ES) % 16 == 0;
  int64_t work = S0 * (vec ? S1 / NV : S1);
  int64_t blocks = (work + 255) / 256;
  if (blocks > 65536 * 16) blocks = 65536 * 16;
  if (blocks < 1) blocks = 1;
  if (vec)
    reduce_kernel<XDT, YDT, NV><<<dim3((unsigned)blocks), 256, 0, st>>>(x, S0, R, S1, xs0, xsr, xs1, mask, ms0, msr,
                                                                       ms1, scale, ss0, ssr, ss1, y, ys0, ys1);
  else
    reduce_kernel<XDT, YDT, 1><<<dim3((unsigned)blocks), 256, 0, st>>>(x, S0, R, S1, xs0, xsr, xs1, mask, ms0, msr,
                                                                      ms1, scale, ss0, ssr, ss1, y, ys0, ys1);
  return launch_status();
}


// ---------------------------------------------------------------------------------------------------------------------
// The general reduction (reduce.py:375-492 of the reference, _reduce_forward_inner): every operand optional.
//   t_r  = x[s0, r, c] (* 2^(e-127) of its 32-column group) * x_flex_scale * scale[s0, r, c], 0 where the mask is 0
//   acc  = sum_r t_r                      float32, in index order
//   o    = postprocess(acc)               none; SwiGLU of (gate, linear) column pairs; (pair + a) sums
//   o   *= x_global_scale
//   then either  flexpoint:  actual_scale <- max(actual_scale, max|o| / max_finite(y) + 1e-30); o /= expected_scale
//                            (clamped to the finite range of y when saturating), cast to y's type
//        or      MXFP8:      o /= expected_scale; per 32 output columns: scale = 2^ceil(log2(max|o| / 448)), values
//                            o / scale as float8_e4m3fn (what tamd_downcast_mxfp makes of the same float32 numbers).
// A thread owns PV consecutive input columns of one row s0 (PV = 8: vector loads when the layout allows; PV = RN: one
// output per thread for narrow or strided inner axes).  The threads of a row are padded to a multiple of the threads
// of a 32-column output group, so that a group's maximum is a shuffle over neighbouring lanes of one wave.
// ---------------------------------------------------------------------------------------------------------------------
TAMD_DEVICE float load_elem_f32(const void *p, int dt, int64_t i) {
  switch (dt) {
    case TAMD_F32: return ((const float *)p)[i];
    case TAMD_BF16: return bf16_bits_to_f32(((const uint16_t *)p)[i]);
    case TAMD_F16: return f16_bits_to_f32(((const uint16_t *)p)[i]);
    case TAMD_FP8_E4M3: return __builtin_amdgcn_cvt_f32_fp8((int)((const uint8_t *)p)[i], 0);
    default: return __builtin_amdgcn_cvt_f32_bf8((int)((const uint8_t *)p)[i], 0);
  }
}

TAMD_DEVICE uint32_t narrow_bits(float v, int dt) {  // 8- or 16-bit output types
  return dt == TAMD_BF16 ? (f32_to_bf16_bits(v) & 0xFFFFu) : (dt == TAMD_F16 ? (f32_to_f16_bits(v) & 0xFFFFu) : f32_to_fp8_bits(v, dt));
}

// LEAN: plain sums of dense, aligned rows (no mask, no per-element or block scales, no pairwise post-processing, no
// flexpoint or MXFP8 output; the scalar input scales may be there) -- what the top-k combine of fp8 rows is.  Only
// the vector paths are compiled, which takes the kernel from 143 to about half as many registers: it is bound by
// the loads it has in flight, i.e. by how many of its waves fit a CU.
template <int PV, int RN, bool LEAN = false>
__global__ __launch_bounds__(256) void reduce_ex_kernel(tamd_reduce_args a, int64_t threads_per_row, int vec_in, int vec_out) {
  constexpr int NO = PV / RN;                         // outputs per thread
  constexpr int TPG = 32 / NO > 0 ? 32 / NO : 1;      // threads of one 32-column output group
  const int64_t S1 = a.S1, Y_S1 = S1 / RN;
  // rows past the device-side count are neither reduced nor written (reduce.py:550-555)
  int64_t rows = a.S0;
  if (a.unpadded_batch_size) {
    const int64_t u = *a.unpadded_batch_size;
    rows = u < 0 ? 0 : (u < rows ? u : rows);
  }
  const int64_t total = rows * threads_per_row;
  const int xsz = a.x_dtype == TAMD_F32 ? 4 : (is_fp8_type(a.x_dtype) ? 1 : 2);
  const int ysz = a.y_dtype == TAMD_F32 ? 4 : (is_fp8_type(a.y_dtype) ? 1 : 2);
  const float flex_in = a.x_flex_scale ? *a.x_flex_scale : 1.0f;
  const float global = a.x_global_scale ? *a.x_global_scale : 1.0f;
  const float inv_expected = a.y_expected_scale ? 1.0f / *a.y_expected_scale : 1.0f;
  const float out_max = max_finite_of(a.y_dtype);
  const bool clamp_out = a.y_expected_scale != nullptr && a.y_saturate_inf != 0 && a.y_mx_scale == nullptr;
  uint32_t amax = 0;
  for (int64_t base = (int64_t)blockIdx.x * 256; base < total; base += (int64_t)gridDim.x * 256) {
    const int64_t i = base + threadIdx.x;
    const bool live = i < total;
    // (a 64-bit division costs about a hundred instructions per thread; the index usually fits 32 bits)
    const int64_t s0 = !live ? 0 : (total <= 0x7FFFFFFF ? (int64_t)((uint32_t)i / (uint32_t)threads_per_row) : i / threads_per_row);
    const int64_t c0 = live ? (i - s0 * threads_per_row) * PV : S1;  // c0 >= S1: a padding thread of the row
    // the first term starts the sum when the axis has at most 8 entries (reduce.py:137, 467-470: a column of -0.0
    // stays -0.0), which is what a start from -0.0 does; longer axes start from +0.0
    const float acc0 = (a.R > 0 && a.R <= 8) ? -0.0f : 0.0f;
    float acc[PV];
#pragma unroll
    for (int j = 0; j < PV; ++j) acc[j] = acc0;
    if (c0 < S1) {
      // PV values of row r of the reduced axis
      auto load_row = [&](int64_t r, float (&v)[PV]) {
        const int64_t xo = s0 * a.xs0 + r * a.xsr;
        if (LEAN || (PV == 8 && vec_in)) {  // unit inner stride, 8 columns inside S1, 8-element alignment of every row
          if (xsz == 4) {
            const float4 lo = *(const float4 *)((const float *)a.x + xo + c0), hi = *(const float4 *)((const float *)a.x + xo + c0 + 4);
            v[0] = lo.x, v[1] = lo.y, v[2] = lo.z, v[3] = lo.w, v[4 % PV] = hi.x, v[5 % PV] = hi.y, v[6 % PV] = hi.z, v[7 % PV] = hi.w;
          } else if (xsz == 2) {
            const uint4 q = *(const uint4 *)((const uint16_t *)a.x + xo + c0);
            const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
            for (int j = 0; j < PV / 2; ++j) {
              v[2 * j] = a.x_dtype == TAMD_BF16 ? bf16_bits_to_f32(w[j] & 0xFFFFu) : f16_bits_to_f32(w[j] & 0xFFFFu);
              v[2 * j + 1] = a.x_dtype == TAMD_BF16 ? bf16_bits_to_f32(w[j] >> 16) : f16_bits_to_f32(w[j] >> 16);
            }
          } else {
            const uint2 q = *(const uint2 *)((const uint8_t *)a.x + xo + c0);
#pragma unroll
            for (int j = 0; j < PV; ++j) {
              const int b = (int)(((j < 4 ? q.x : q.y) >> (8 * (j & 3))) & 0xFFu);
              v[j] = a.x_dtype == TAMD_FP8_E4M3 ? __builtin_amdgcn_cvt_f32_fp8(b, 0) : __builtin_amdgcn_cvt_f32_bf8(b, 0);
            }
          }
        } else {
#pragma unroll
          for (int j = 0; j < PV; ++j) v[j] = c0 + j < S1 ? load_elem_f32(a.x, a.x_dtype, xo + (c0 + j) * a.xs1) : 0.f;
        }
      };
      int64_t r = 0;
      if (LEAN || (PV == 8 && vec_in && !a.x_mx_scale && !a.scale && !a.mask)) {
        // plain sums (the top-k combine): four rows are fetched together -- raw loads first, conversions after, with
        // the element size fixed outside so that no branch separates the loads -- and added in the order r = 0, 1, ...
        auto batches = [&](auto xs_tag) {
          constexpr int XS = decltype(xs_tag)::value;
          constexpr int NQ = XS == 4 ? 2 : 1;
          for (; r + 4 <= a.R; r += 4) {
            uint4 q[4][NQ];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              const uint8_t *src = (const uint8_t *)a.x + (s0 * a.xs0 + (r + u) * a.xsr + c0) * XS;
              if constexpr (XS == 1) {
                const uint2 h = *(const uint2 *)src;
                q[u][0] = make_uint4(h.x, h.y, 0, 0);
              } else {
#pragma unroll
                for (int n = 0; n < NQ; ++n) q[u][n] = *(const uint4 *)(src + 16 * n);
              }
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
              float v[8];
              if constexpr (XS == 4) {
                v[0] = bits_to_f32(q[u][0].x), v[1] = bits_to_f32(q[u][0].y), v[2] = bits_to_f32(q[u][0].z), v[3] = bits_to_f32(q[u][0].w);
                v[4] = bits_to_f32(q[u][NQ - 1].x), v[5] = bits_to_f32(q[u][NQ - 1].y), v[6] = bits_to_f32(q[u][NQ - 1].z), v[7] = bits_to_f32(q[u][NQ - 1].w);
              } else if constexpr (XS == 2) {
                const uint32_t w[4] = {q[u][0].x, q[u][0].y, q[u][0].z, q[u][0].w};
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                  v[2 * j] = a.x_dtype == TAMD_BF16 ? bf16_bits_to_f32(w[j] & 0xFFFFu) : f16_bits_to_f32(w[j] & 0xFFFFu);
                  v[2 * j + 1] = a.x_dtype == TAMD_BF16 ? bf16_bits_to_f32(w[j] >> 16) : f16_bits_to_f32(w[j] >> 16);
                }
              } else {
                // two values per conversion instruction (the pair is picked by an immediate)
                typedef float f32x2_t __attribute__((ext_vector_type(2)));
                const int w0 = (int)q[u][0].x, w1 = (int)q[u][0].y;
                f32x2_t p[4];
                if (a.x_dtype == TAMD_FP8_E4M3) {
                  p[0] = __builtin_amdgcn_cvt_pk_f32_fp8(w0, false), p[1] = __builtin_amdgcn_cvt_pk_f32_fp8(w0, true);
                  p[2] = __builtin_amdgcn_cvt_pk_f32_fp8(w1, false), p[3] = __builtin_amdgcn_cvt_pk_f32_fp8(w1, true);
                } else {
                  p[0] = __builtin_amdgcn_cvt_pk_f32_bf8(w0, false), p[1] = __builtin_amdgcn_cvt_pk_f32_bf8(w0, true);
                  p[2] = __builtin_amdgcn_cvt_pk_f32_bf8(w1, false), p[3] = __builtin_amdgcn_cvt_pk_f32_bf8(w1, true);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) v[2 * j] = p[j][0], v[2 * j + 1] = p[j][1];
              }
#pragma unroll
              for (int j = 0; j < PV; ++j) acc[j] += v[j % 8] * flex_in;
            }
          }
        };
        if (xsz == 1) batches(std::integral_constant<int, 1>{});
        else if (xsz == 2) batches(std::integral_constant<int, 2>{});
        else batches(std::integral_constant<int, 4>{});
      }
      for (; r < a.R; ++r) {
        float v[PV];
        load_row(r, v);
        if constexpr (LEAN) {
#pragma unroll
          for (int j = 0; j < PV; ++j) acc[j] += v[j] * flex_in;
          continue;
        }
#pragma unroll
        for (int j = 0; j < PV; ++j) {
          const int64_t c = c0 + j;
          float t = v[j];
          if (a.x_mx_scale) {
            const uint32_t e = c < S1 ? a.x_mx_scale[s0 * a.xms0 + r * a.xmsr + (c / 32) * a.xms1] : 127u;
            t *= bits_to_f32(e << 23);
          }
          t *= flex_in;
          if (a.scale && c < S1) t = __builtin_fmaf(t, a.scale[s0 * a.ss0 + r * a.ssr + c * a.ss1], 0.0f);  // reduce.py:466
          if (a.mask && c < S1 && !a.mask[s0 * a.ms0 + r * a.msr + c * a.ms1]) t = 0.f;
          acc[j] += c < S1 ? t : 0.f;
        }
      }
    }
    // ---- post-processing over groups of RN columns
    float o[NO];
#pragma unroll
    for (int j = 0; j < NO; ++j) {
      if constexpr (RN == 1) o[j] = acc[j];
      else if (a.postprocess == TAMD_PP_SWIGLU) o[j] = swiglu_f32(acc[2 * j], acc[2 * j + 1], a.pp_arg0, a.pp_arg1, a.pp_has_arg1 != 0);
      else o[j] = (acc[2 * j] + a.pp_arg0) + (acc[2 * j + 1] + a.pp_arg0);
      o[j] *= global;
    }
    const int64_t oc0 = c0 / RN;  // first output column
    if constexpr (LEAN) {
      // nothing between the sums and the store
    } else if (a.y_mx_scale) {
      // MXFP8: the group's threads are TPG neighbouring lanes (rows are padded to whole groups of threads)
      float m = 0.f;
#pragma unroll
      for (int j = 0; j < NO; ++j) {
        o[j] *= inv_expected;
        m = __builtin_fmaxf(m, oc0 + j < Y_S1 ? __builtin_fabsf(o[j]) : 0.f);
      }
#pragma unroll
      for (int sh = TPG / 2; sh > 0; sh >>= 1) m = __builtin_fmaxf(m, __shfl_xor(m, sh));
      const uint32_t sb = (f32_to_bits(m / 448.0f) + 0x007FFFFFu) & 0x7F800000u;
      const float ds = bits_to_f32(sb);
      const float qs = ds == 0.f ? 0.f : 1.0f / ds;
#pragma unroll
      for (int j = 0; j < NO; ++j) {
        const float q = o[j] * qs;
        o[j] = q != q ? q : __builtin_fminf(__builtin_fmaxf(q, -448.0f), 448.0f);
      }
      if (oc0 < Y_S1 && (threadIdx.x & (TPG - 1)) == 0) a.y_mx_scale[s0 * a.yms0 + (oc0 / 32) * a.yms1] = (uint8_t)(sb >> 23);
    } else {
      if (a.y_actual_scale) {
#pragma unroll
        for (int j = 0; j < NO; ++j)
          if (oc0 + j < Y_S1) amax = absmax_bits(amax, o[j]);
      }
#pragma unroll
      for (int j = 0; j < NO; ++j) {
        o[j] *= inv_expected;
        if (clamp_out) o[j] = __builtin_fminf(__builtin_fmaxf(o[j], -out_max), out_max);
      }
    }
    if (oc0 >= Y_S1) continue;
    // ---- store: NO outputs, as one or two vector stores when the row is dense and aligned
    if (LEAN || (NO > 1 && vec_out && oc0 + NO <= Y_S1)) {
      uint8_t *yp = (uint8_t *)a.y + (s0 * a.ys0 + oc0) * ysz;
      if (ysz == 4) {
#pragma unroll
        for (int j = 0; j < NO; j += 4) *(float4 *)(yp + j * 4) = make_float4(o[j], o[(j + 1) % NO], o[(j + 2) % NO], o[(j + 3) % NO]);
      } else if (ysz == 2) {
        uint32_t w[NO / 2 > 0 ? NO / 2 : 1];
#pragma unroll
        for (int j = 0; j < NO / 2; ++j) w[j] = narrow_bits(o[2 * j], a.y_dtype) | (narrow_bits(o[2 * j + 1], a.y_dtype) << 16);
        if constexpr (NO == 8) *(uint4 *)yp = make_uint4(w[0], w[1], w[2], w[3]);
        else if constexpr (NO == 4) *(uint2 *)yp = make_uint2(w[0], w[1]);
        else *(uint32_t *)yp = w[0];
      } else {
        uint32_t w[NO / 4 > 0 ? NO / 4 : 1];
#pragma unroll
        for (int j = 0; j < NO / 4; ++j)
          w[j] = narrow_bits(o[4 * j], a.y_dtype) | (narrow_bits(o[4 * j + 1], a.y_dtype) << 8) |
                 (narrow_bits(o[4 * j + 2], a.y_dtype) << 16) | (narrow_bits(o[4 * j + 3], a.y_dtype) << 24);
        if constexpr (NO == 8) *(uint2 *)yp = make_uint2(w[0], w[1]);
        else if constexpr (NO == 4) *(uint32_t *)yp = w[0];
        else {
#pragma unroll
          for (int j = 0; j < NO; ++j) yp[j] = (uint8_t)narrow_bits(o[j], a.y_dtype);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < NO; ++j) {
        if (oc0 + j >= Y_S1) break;
        const int64_t yi = s0 * a.ys0 + (oc0 + j) * a.ys1;
        if (ysz == 4) ((float *)a.y)[yi] = o[j];
        else if (ysz == 2) ((uint16_t *)a.y)[yi] = (uint16_t)narrow_bits(o[j], a.y_dtype);
        else ((uint8_t *)a.y)[yi] = (uint8_t)narrow_bits(o[j], a.y_dtype);
      }
    }
  }
  if (!LEAN && a.y_actual_scale && !a.y_mx_scale) {
    // wave maximum, then one atomic per wave; positive floats order like their bit patterns, NaN counts as +inf
#pragma unroll
    for (int sh = 32; sh > 0; sh >>= 1) {
      const uint32_t other = (uint32_t)__shfl_xor((int)amax, sh);
      amax = other > amax ? other : amax;
    }
    if (threadIdx.x % kWave == 0) {
      amax = amax < 0x7F800000u ? amax : 0x7F800000u;
      atomicMax((unsigned int *)a.y_actual_scale, f32_to_bits(__builtin_fmaf(bits_to_f32(amax), 1.0f / out_max, 1.0e-30f)));
    }
  }
}

template <int PV, int RN, bool LEAN = false>
int launch_reduce_ex(const tamd_reduce_args &a, int vec_in, int vec_out, hipStream_t st) {
  constexpr int NO = PV / RN;
  constexpr int TPG = 32 / NO > 0 ? 32 / NO : 1;
  int64_t tpr = (a.S1 + PV - 1) / PV;
  if (a.y_mx_scale) tpr = (tpr + TPG - 1) / TPG * TPG;
  const int64_t total = a.S0 * tpr;
  int64_t blocks = (total + 255) / 256;
  blocks = blocks > 65536 * 16 ? 65536 * 16 : (blocks < 1 ? 1 : blocks);
  reduce_ex_kernel<PV, RN, LEAN><<<dim3((unsigned)blocks), 256, 0, st>>>(a, tpr, vec_in, vec_out);
  return launch_status();
}

}  // namespace tamd

using namespace tamd;

extern "C" int tamd_reduce(const void *x, int x_dtype, int64_t S0, int64_t R, int64_t S1, int64_t xs0, int64_t xsr,
                           int64_t xs1, const uint8_t *mask, int64_t ms0, int64_t msr, int64_t ms1,
                           const float *scale, int64_t ss0, int64_t ssr, int64_t ss1, void *y, int y_dtype,
                           int64_t ys0, int64_t ys1, void *stream) {
  if (S0 < 0 || R < 0 || S1 < 0) return TAMD_E_INVALID;
  if (S0 == 0 || S1 == 0) return 0;
  if (!y || (R > 0 && !x)) return TAMD_E_INVALID;
  hipStream_t st = (hipStream_t)stream;
#define TAMD_RED(XD, YD)                                                                                          \
  return launch_reduce<XD, YD>(x, S0, R, S1, xs0, xsr, xs1, mask, ms0, msr, ms1, scale, ss0, ssr, ss1, y, ys0, ys1, \
                               st)
  if (x_dtype == TAMD_BF16 && y_dtype == TAMD_BF16) TAMD_RED(TAMD_BF16, TAMD_BF16);
  if (x_dtype == TAMD_BF16 && y_dtype == TAMD_F32) TAMD_RED(TAMD_BF16, TAMD_F32);
  if (x_dtype == TAMD_F16 && y_dtype == TAMD_F16) TAMD_RED(TAMD_F16, TAMD_F16);
  if (x_dtype == TAMD_F16 && y_dtype == TAMD_F32) TAMD_RED(TAMD_F16, TAMD_F32);
  if (x_dtype == TAMD_F32 && y_dtype == TAMD_F32) TAMD_RED(TAMD_F32, TAMD_F32);
  if (x_dtype == TAMD_F32 && y_dtype == TAMD_BF16) TAMD_RED(TAMD_F32, TAMD_BF16);
  if (x_dtype == TAMD_F32 && y_dtype == TAMD_F16) TAMD_RED(TAMD_F32, TAMD_F16);
#undef TAMD_RED
  return TAMD_E_UNSUPPORTED;
}

extern "C" int tamd_swiglu(const void *a, int dtype, int64_t M, int64_t N_out, int64_t a_stride_m, void *out,
                           int64_t out_stride_m, float alpha, float limit, int has_limit, void *stream) {
  if (M < 0 || N_out < 0) return TAMD_E_INVALID;
  if (M == 0 || N_out == 0) return 0;
  if (!a || !out) return TAMD_E_INVALID;
  hipStream_t st = (hipStream_t)stream;
  const int esz = dtype == TAMD_F32 ? 4 : 2;
  if (N_out % 4 == 0 && aligned(a, 16) && aligned(out, 16) && (a_stride_m * esz) % 16 == 0 && (out_stride_m * esz) % 16 == 0 &&
      (dtype == TAMD_F32 || dtype == TAMD_BF16 || dtype == TAMD_F16)) {
    int64_t vblocks = (M * (N_out / 4) + 255) / 256;
    if (vblocks > 256 * 64) vblocks = 256 * 64;
    if (dtype == TAMD_F32)
      swiglu_vec4_kernel<TAMD_F32><<<dim3((unsigned)vblocks), 256, 0, st>>>(a, M, N_out, a_stride_m, out, out_stride_m, alpha, limit, has_limit);
    else if (dtype == TAMD_BF16)
      swiglu_vec4_kernel<TAMD_BF16><<<dim3((unsigned)vblocks), 256, 0, st>>>(a, M, N_out, a_stride_m, out, out_stride_m, alpha, limit, has_limit);
    else
      swiglu_vec4_kernel<TAMD_F16><<<dim3((unsigned)vblocks), 256, 0, st>>>(a, M, N_out, a_stride_m, out, out_stride_m, alpha, limit, has_limit);
    return launch_status();
  }
  int64_t blocks = (M * N_out + 255) / 256;
  if (blocks > 256 * 32) blocks = 256 * 32;
  switch (dtype) {
    case TAMD_F32:
      swiglu_kernel<TAMD_F32><<<dim3((unsigned)blocks), 256, 0, st>>>(a, M, N_out, a_stride_m, out, out_stride_m,
                                                                     alpha, limit, has_limit);
      break;
    case TAMD_BF16:
      swiglu_kernel<TAMD_BF16><<<dim3((unsigned)blocks), 256, 0, st>>>(a, M, N_out, a_stride_m, out, out_stride_m,
                                                                      alpha, limit, has_limit);
      break;
    case TAMD_F16:
      swiglu_kernel<TAMD_F16><<<dim3((unsigned)blocks), 256, 0, st>>>(a, M, N_out, a_stride_m, out, out_stride_m,
                                                                     alpha, limit, has_limit);
      break;
    default:
      return TAMD_E_INVALID;
  }
  return launch_status();
}

extern "C" int tamd_reduce_ex(const tamd_reduce_args *args, void *stream) {
  if (!args) return TAMD_E_INVALID;
  tamd_reduce_args a = *args;
  if (a.S0 < 0 || a.R < 0 || a.S1 < 0) return TAMD_E_INVALID;
  const int rn = a.postprocess == TAMD_PP_NONE ? 1 : 2;
  if (a.postprocess != TAMD_PP_NONE && a.postprocess != TAMD_PP_SWIGLU && a.postprocess != TAMD_PP_PLUS_A_PAIRSUM) return TAMD_E_INVALID;
  if (a.S1 % rn != 0) return TAMD_E_INVALID;
  if (a.S0 == 0 || a.S1 == 0) return 0;
  if (!a.y || (a.R > 0 && !a.x)) return TAMD_E_INVALID;
  const bool x8 = is_fp8_type(a.x_dtype), y8 = is_fp8_type(a.y_dtype);
  if (a.x_dtype != TAMD_F32 && a.x_dtype != TAMD_F16 && a.x_dtype != TAMD_BF16 && !x8) return TAMD_E_INVALID;
  if (a.y_dtype != TAMD_F32 && a.y_dtype != TAMD_F16 && a.y_dtype != TAMD_BF16 && !y8) return TAMD_E_INVALID;
  if (a.y_mx_scale && (a.y_dtype != TAMD_FP8_E4M3 || a.y_actual_scale)) return TAMD_E_UNSUPPORTED;
  hipStream_t st = (hipStream_t)stream;
  const int xsz = a.x_dtype == TAMD_F32 ? 4 : (x8 ? 1 : 2), ysz = a.y_dtype == TAMD_F32 ? 4 : (y8 ? 1 : 2);
  // eight columns per thread when the inner axis is dense, long enough and every row starts on an 8-element boundary
  const bool wide = a.xs1 == 1 && a.S1 >= 64;
  const int vec_in = wide && a.S1 % 8 == 0 && aligned(a.x, 8 * xsz) && a.xs0 % 8 == 0 && a.xsr % 8 == 0;
  const int no = 8 / rn;
  const int vec_out = wide && a.ys1 == 1 && (a.S1 / rn) % no == 0 && aligned(a.y, no * ysz < 16 ? no * ysz : 16) &&
                      (a.ys0 * ysz) % (no * ysz < 16 ? no * ysz : 16) == 0;
  const bool lean = wide && rn == 1 && vec_in && vec_out && !a.mask && !a.scale && !a.x_mx_scale && !a.y_mx_scale &&
                    !a.y_expected_scale && !a.y_actual_scale && !a.unpadded_batch_size;
  if (lean) return launch_reduce_ex<8, 1, true>(a, vec_in, vec_out, st);
  if (wide) return rn == 1 ? launch_reduce_ex<8, 1>(a, vec_in, vec_out, st) : launch_reduce_ex<8, 2>(a, vec_in, vec_out, st);
  return rn == 1 ? launch_reduce_ex<1, 1>(a, 0, 0, st) : launch_reduce_ex<2, 2>(a, 0, 0, st);
}

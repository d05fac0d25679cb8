// Bandwidth kernels next to the matmul: the top-k combine (sum over the middle
// axis with optional mask / scale) and the standalone interleaved SwiGLU.
#include "common.h"

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
    const int64_t s0 = i / nv, c0 = (i - s0 * nv) * VEC;
    float acc[VEC];
#pragma unroll
    for (int j = 0; j < VEC; ++j) acc[j] = 0.f;
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
        if (scale) t *= scale[s0 * ss0 + r * ssr + (c0 + j) * ss1];
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

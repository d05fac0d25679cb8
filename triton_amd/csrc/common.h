// Shared device / host helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <atomic>
#include <mutex>
#include <unordered_set>

#include "../../include/triton_amd.h"

#define TAMD_DEVICE __device__ __forceinline__

namespace tamd {

constexpr int kWave = 64;

TAMD_DEVICE float bits_to_f32(uint32_t u) { return __builtin_bit_cast(float, u); }
TAMD_DEVICE uint32_t f32_to_bits(float f) { return __builtin_bit_cast(uint32_t, f); }

TAMD_DEVICE float bf16_bits_to_f32(uint32_t h) { return bits_to_f32(h << 16); }

// float32 -> bfloat16 bits, round to nearest even, NaN kept quiet (one v_cvt_pk_bf16_f32 on gfx950).
TAMD_DEVICE uint32_t f32_to_bf16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)f);
}

TAMD_DEVICE float f16_bits_to_f32(uint32_t h) {
  return (float)__builtin_bit_cast(_Float16, (uint16_t)h);
}
TAMD_DEVICE uint32_t f32_to_f16_bits(float f) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)f);
}

// float32 -> OCP e4m3fn byte, round to nearest even.  Magnitudes that round beyond 448 (>= 464) give the
// largest finite code when `saturate`, NaN otherwise (what a plain cast does); NaN stays NaN.
TAMD_DEVICE uint32_t f32_to_e4m3_bits(float f, bool saturate) {
  const uint32_t u = f32_to_bits(f), sign = (u >> 24) & 0x80u, mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return sign | 0x7Fu;
  if (mag >= 0x43E80000u) return sign | (saturate ? 0x7Eu : 0x7Fu);  // 464.0f
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f, f, 0, false) & 0xFFu;
}

// float32 -> OCP e5m2 byte, round to nearest even.  Magnitudes that round beyond 57344 (>= 61440) give infinity
// (or the largest finite code when saturating); NaN stays NaN.
TAMD_DEVICE uint32_t f32_to_e5m2_bits(float f, bool saturate) {
  const uint32_t u = f32_to_bits(f), sign = (u >> 24) & 0x80u, mag = u & 0x7FFFFFFFu;
  if (mag > 0x7F800000u) return sign | 0x7Fu;
  if (mag >= 0x47700000u) return sign | (saturate ? 0x7Bu : 0x7Cu);  // 61440.0f
  return (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(f, f, 0, false) & 0xFFu;
}
TAMD_DEVICE uint32_t f32_to_fp8_bits(float f, int dt) {
  return dt == TAMD_FP8_E5M2 ? f32_to_e5m2_bits(f, false) : f32_to_e4m3_bits(f, false);
}

// Largest finite value of an output type, and the running |x| maximum kept as float bits so that NaN
// (above +inf as an integer) survives the maximum (flexpoint.py:119-146 of the reference).
TAMD_DEVICE float max_finite_of(int dt) {
  return dt == TAMD_FP8_E4M3 ? 448.0f : dt == TAMD_FP8_E5M2 ? 57344.0f : (dt == TAMD_F16 ? 65504.0f : (dt == TAMD_BF16 ? 3.3895313892515355e38f : 3.4028234663852886e38f));
}
TAMD_DEVICE uint32_t absmax_bits(uint32_t run, float v) {
  const uint32_t b = f32_to_bits(v) & 0x7FFFFFFFu;
  return b > run ? b : run;
}

// OCP e4m3fn byte -> float32 (exact).
TAMD_DEVICE float e4m3_bits_to_f32(uint32_t b) {
  uint32_t s = (b & 0x80u) << 24;
  uint32_t e = (b >> 3) & 0xFu;
  uint32_t m = b & 7u;
  float mag;
  if (e == 0) {
    mag = (float)m * 0.001953125f;  // m * 2^-9
  } else if (e == 15 && m == 7) {
    mag = bits_to_f32(0x7FC00000u);
  } else {
    mag = bits_to_f32(((e + 120u) << 23) | (m << 20));
  }
  return bits_to_f32(f32_to_bits(mag) | s);
}

template <int DT>
TAMD_DEVICE float load_as_f32(const void *p, int64_t i) {
  if constexpr (DT == TAMD_F32) return ((const float *)p)[i];
  if constexpr (DT == TAMD_BF16) return bf16_bits_to_f32(((const uint16_t *)p)[i]);
  if constexpr (DT == TAMD_F16) return f16_bits_to_f32(((const uint16_t *)p)[i]);
  if constexpr (DT == TAMD_FP8_E4M3) return e4m3_bits_to_f32(((const uint8_t *)p)[i]);
  return 0.f;
}

template <int DT>
TAMD_DEVICE void store_from_f32(void *p, int64_t i, float v) {
  if constexpr (DT == TAMD_F32) ((float *)p)[i] = v;
  if constexpr (DT == TAMD_BF16) ((uint16_t *)p)[i] = (uint16_t)f32_to_bf16_bits(v);
  if constexpr (DT == TAMD_F16) ((uint16_t *)p)[i] = (uint16_t)f32_to_f16_bits(v);
}

__host__ __device__ inline bool is_fp8_type(int dt) { return dt == TAMD_FP8_E4M3 || dt == TAMD_FP8_E5M2; }

inline int dtype_size(int dt) {
  switch (dt) {
    case TAMD_F32: return 4;
    case TAMD_F16:
    case TAMD_BF16: return 2;
    case TAMD_FP8_E4M3:
    case TAMD_FP8_E5M2:
    case TAMD_MXFP4: return 1;
    default: return 0;
  }
}

inline bool aligned(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

// One-time set-up per kernel and device, kept out of the per-call path: raising a kernel's dynamic LDS limit (an
// attribute of the function in the device's loaded code object) and the device's CU count.  The only process-wide
// state of the library besides its code objects; values never change once set, so calls stay re-entrant.
inline int current_device(int &dev) {
  hipError_t e = hipGetDevice(&dev);
  return e == hipSuccess ? 0 : (int)e;
}

inline int raise_lds_limit_once(const void *kern) {
  static std::mutex mu;
  static std::unordered_set<uint64_t> done;
  int dev = 0;
  if (int rc = current_device(dev)) return rc;
  const uint64_t key = ((uint64_t)(uint32_t)dev << 48) ^ (uint64_t)(uintptr_t)kern;
  {
    std::lock_guard<std::mutex> lock(mu);
    if (done.count(key)) return 0;
  }
  hipError_t e = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e != hipSuccess) return (int)e;
  std::lock_guard<std::mutex> lock(mu);
  done.insert(key);
  return 0;
}

inline int cu_count(int &cus) {
  constexpr int kMaxDevices = 64;
  static std::atomic<int> cached[kMaxDevices];
  int dev = 0;
  if (int rc = current_device(dev)) return rc;
  if (dev >= 0 && dev < kMaxDevices) {
    cus = cached[dev].load(std::memory_order_relaxed);
    if (cus > 0) return 0;
  }
  hipError_t e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
  if (e != hipSuccess) return (int)e;
  if (dev >= 0 && dev < kMaxDevices) cached[dev].store(cus, std::memory_order_relaxed);
  return 0;
}

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : (int)e;
}

}  // namespace tamd

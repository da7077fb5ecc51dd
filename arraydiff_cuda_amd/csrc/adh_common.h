// Shared host/device helpers for the gfx950 kernels of the spatial-conv path.
#ifndef ADH_COMMON_H
#define ADH_COMMON_H

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "adh_capi.h"

namespace adh {

// Division of a 31-bit value by a launch-time constant with one mul_hi, one add and one
// shift (Granlund-Montgomery round-up method).  Exact for 0 <= n < 2^31.
struct FastDiv {
  uint32_t d, mul, shift;
  FastDiv() : d(1), mul(1), shift(0) {}
  explicit FastDiv(uint32_t div) : d(div ? div : 1) {
    shift = 0;
    while ((1ull << shift) < d) ++shift;
    mul = (uint32_t)(((1ull << 32) * ((1ull << shift) - d)) / d + 1);
  }
  __host__ __device__ __forceinline__ uint32_t div(uint32_t n) const {
#if defined(__HIP_DEVICE_COMPILE__)
    return (__umulhi(n, mul) + n) >> shift;
#else
    return (uint32_t)(((((uint64_t)n * mul) >> 32) + n) >> shift);
#endif
  }
  __host__ __device__ __forceinline__ void divmod(uint32_t n, uint32_t &q, uint32_t &r) const {
    q = div(n);
    r = n - q * d;
  }
};

__device__ __forceinline__ float bf16_bits_to_f32(uint16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round-to-nearest-even; NaN stays a quiet NaN
__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float elem_add(float a, float b) { return a + b; }
__device__ __forceinline__ uint16_t elem_add(uint16_t a, uint16_t b) {
  return f32_to_bf16_bits(bf16_bits_to_f32(a) + bf16_bits_to_f32(b));
}

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? ADH_OK : (int)e;
}

inline bool aligned_to(const void *p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

inline size_t dtype_size(int dtype) { return dtype == ADH_BF16 ? 2 : 4; }
inline bool dtype_ok(int dtype) { return dtype == ADH_F32 || dtype == ADH_BF16; }

}  // namespace adh

#endif

// Shared host/device helpers for the gfx950 kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include "../../include/dt_hip.h"

#define DT_EXPORT extern "C" __attribute__((visibility("default")))

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

namespace dt {

// True when the current device is a gfx950 part; cached per process.
bool device_ok();

inline hipStream_t as_stream(dt_stream s) { return reinterpret_cast<hipStream_t>(s); }

// Launch errors (bad configuration) surface here; execution errors are the
// stream owner's to observe.
inline dt_status launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? DT_OK : DT_INVALID;
}

__device__ __forceinline__ half_t bits_to_half(uint16_t b) {
  return __builtin_bit_cast(half_t, b);
}
__device__ __forceinline__ uint16_t half_to_bits(half_t h) {
  return __builtin_bit_cast(uint16_t, h);
}

#if defined(__HIPCC__)
// Combine the two half-waves (lanes l and l ^ 32 hold the same matrix column) without touching LDS:
// v_permlane32_swap of a register with a copy of itself leaves {low, low} and {high, high}.
__device__ __forceinline__ void halves32(float v, float& lo, float& hi) {
  uint32_t a = __builtin_bit_cast(uint32_t, v), b = a;
  asm volatile("" : "+v"(b));  // the swap needs two distinct registers
  auto r = __builtin_amdgcn_permlane32_swap(a, b, false, false);
  uint32_t x0 = r[0], x1 = r[1];
  // keeps the two results apart: without it the compiler has been seen to
  // combine r[0] with itself when both inputs carry the same value
  asm volatile("" : "+v"(x0), "+v"(x1));
  lo = __builtin_bit_cast(float, x0);
  hi = __builtin_bit_cast(float, x1);
}
__device__ __forceinline__ float max32(float v) {
  float lo, hi;
  halves32(v, lo, hi);
  return fmaxf(lo, hi);
}
__device__ __forceinline__ float sum32(float v) {
  float lo, hi;
  halves32(v, lo, hi);
  return lo + hi;
}
#endif

}  // namespace dt

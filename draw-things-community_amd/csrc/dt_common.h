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

}  // namespace dt

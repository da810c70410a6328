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

// DT_OK when the calling thread's current device is a gfx950 part (cached per device ordinal); DT_NO_KERNEL for any
// other architecture; DT_DEVICE_ERROR when the runtime already reports a fault (a kernel that faulted, a lost
// device or context: it is left in place for its owner to read, and nothing is enqueued on top of it).  A stale
// non-fatal code in the thread's error slot -- one that some earlier call already returned to its caller -- is
// cleared, so that launch_status() reads this entry point's own launch.
dt_status device_ready();

inline hipStream_t as_stream(dt_stream s) { return reinterpret_cast<hipStream_t>(s); }

// Result of the launch just made.  device_ready() has left the thread's error slot empty, so what
// hipGetLastError() returns here belongs to this launch: a configuration the device cannot run (grid, block, LDS or
// register budget, missing code object) is the library's own "no kernel for this request"; bad arguments are
// DT_INVALID; anything else (the device was lost, an asynchronous fault surfaced in between) is DT_DEVICE_ERROR.
inline dt_status launch_status() {
  const hipError_t e = hipGetLastError();
  switch (e) {
    case hipSuccess:
    case hipErrorNotReady: return DT_OK;  // (the answer of someone's stream or event query, not a failure)
    case hipErrorInvalidConfiguration:
    case hipErrorLaunchOutOfResources:
    case hipErrorInvalidDeviceFunction:
    case hipErrorNoBinaryForGpu:
    case hipErrorSharedObjectInitFailed: return DT_NO_KERNEL;
    case hipErrorInvalidValue:
    case hipErrorInvalidDevicePointer:
    case hipErrorInvalidResourceHandle: return DT_INVALID;
    case hipErrorOutOfMemory: return DT_OOM;
    default: return DT_DEVICE_ERROR;
  }
}

__device__ __forceinline__ half_t bits_to_half(uint16_t b) {
  return __builtin_bit_cast(half_t, b);
}
__device__ __forceinline__ uint16_t half_to_bits(half_t h) {
  return __builtin_bit_cast(uint16_t, h);
}

#if defined(__HIPCC__)
// fp32 -> fp16 -> fp32 as a rounding step of its own.  The empty asm keeps the compiler from folding the arithmetic
// that produced `v` and the conversion into one mixed-precision instruction (v_fma_mixlo_f16 rounds the exact
// product-sum to fp16 once; the op-by-op graph rounds it to fp32 first and to fp16 second, and the two differ by an
// ulp in about one result in 2^15).
__device__ __forceinline__ float round_f16(float v) {
  asm volatile("" : "+v"(v));
  return (float)(half_t)v;
}

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

// One wave-wide memory -> LDS transfer (global_load_lds_dwordx4): an active
// lane l's 16 bytes land at LDS byte address lds_base + 16 * l (lds_base
// wave-uniform).  Written as assembly on purpose: for the builtin the compiler
// marks a "flat access to both memories" as pending and from then on turns
// every s_waitcnt it inserts -- LDS counter included -- into a wait for zero
// until the transfer has landed, which serialises all LDS reads behind it.
// The caller publishes the data itself: s_waitcnt vmcnt(0) (the transfer
// counts as a vector memory load; loads return in order, so an outstanding
// transfer the compiler does not know of can only make one of its own vmcnt
// waits longer, never too short), then a workgroup barrier, before any wave
// reads the destination.  M0 is reserved by the compiler, which sets it anew before
// each of its own uses, so overwriting it here needs no clobber.
__device__ __forceinline__ uint32_t lds_address(const void* p) {
  return (uint32_t)(uintptr_t)(const __attribute__((address_space(3))) void*)p;
}
// source = uniform 64-bit base + 32-bit per-lane byte offset
__device__ __forceinline__ void load_to_lds_16(const void* gbase, uint32_t voff, uint32_t lds_base) {
  // the base must sit in scalar registers whatever the control flow around the call made of it
  const uint64_t gb = (uint64_t)(uintptr_t)gbase;
  // (the builtin returns a signed int: widen through uint32_t, or bit 31 of the low half smears over the high half)
  const uint64_t gu = (uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)gb) |
                      ((uint64_t)(uint32_t)__builtin_amdgcn_readfirstlane((uint32_t)(gb >> 32)) << 32);
  lds_base = (uint32_t)__builtin_amdgcn_readfirstlane(lds_base);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2"
      :
      : "s"(lds_base), "v"(voff), "s"(gu)
      : "memory");
}
// source = per-lane 64-bit address
__device__ __forceinline__ void load_to_lds_16(const void* gptr, uint32_t lds_base) {
  lds_base = __builtin_amdgcn_readfirstlane(lds_base);
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off"
      :
      : "s"(lds_base), "v"(gptr)
      : "memory");
}

}  // namespace dt

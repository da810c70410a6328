// K4: LayerNorm(elementwiseAffine: false) over the last axis of an fp32 residual
// stream followed by the adaLN modulation, fp16 out -- the op in front of every
// Dense of a DiT block.  HBM-bound: 4 bytes read and 2 written per element.
// One wave per row; the row stays in registers between the mean, the variance
// and the output pass, so memory is touched once.
#include "dt_common.h"

namespace dt {

__device__ __forceinline__ float wave_sum64(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

__device__ __forceinline__ float round16(float v) { return round_f16(v); }

// One normalised value through the modulation (sc, sh already widened to float).
//   DT_MOD_F16: fp16(fp16(fp16(n) * scale) + shift), scale and shift fp16
//   DT_MOD_F32: fp16(n * (scale + 1) + shift), scale and shift fp32
//   DT_MOD_AFFINE_F32: fp16(n * scale + shift), scale and shift fp32
template <int MOD>
__device__ __forceinline__ uint16_t modulate(float n, bool has_scale, float sc, bool has_shift, float sh) {
  if constexpr (MOD == DT_MOD_F16) {
    n = round16(n);
    if (has_scale) n = round16(n * sc);
    if (has_shift) n = round16(n + sh);
  } else {
    if (has_scale) n = n * (MOD == DT_MOD_F32 ? sc + 1.0f : sc);
    if (has_shift) n = n + sh;
  }
  return half_to_bits((half_t)n);
}

template <int MOD>
__device__ __forceinline__ float mod_at(const void* p, int64_t c) {
  if constexpr (MOD == DT_MOD_F16) return (float)bits_to_half(static_cast<const uint16_t*>(p)[c]);
  else return static_cast<const float*>(p)[c];
}
// four consecutive values starting at element c (c % 4 == 0, vector aligned)
template <int MOD>
__device__ __forceinline__ void mod_at4(const void* p, int c, float (&o)[4]) {
  if constexpr (MOD == DT_MOD_F16) {
    const uint2_t t = *reinterpret_cast<const uint2_t*>(static_cast<const uint16_t*>(p) + c);
    o[0] = (float)bits_to_half((uint16_t)t[0]); o[1] = (float)bits_to_half((uint16_t)(t[0] >> 16));
    o[2] = (float)bits_to_half((uint16_t)t[1]); o[3] = (float)bits_to_half((uint16_t)(t[1] >> 16));
  } else {
    const float4_t t = *reinterpret_cast<const float4_t*>(static_cast<const float*>(p) + c);
    o[0] = t[0]; o[1] = t[1]; o[2] = t[2]; o[3] = t[3];
  }
}

struct AdaLnArgs {
  const float* x;
  int64_t ldx;
  int64_t m, c;
  const void* scale;
  const void* shift;
  float eps;
  uint16_t* y;
  int64_t ldy;
};

// Rows of up to NV * 256 elements, C % 4 == 0, 16-byte aligned rows: lane l
// holds the float4 at element 256 i + 4 l of every 256-element chunk i.
template <int NV, int MOD>
__global__ void __launch_bounds__(256) adaln_rows_kernel(const AdaLnArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.m) return;
  const float* xr = a.x + row * a.ldx;
  uint16_t* yr = a.y + row * a.ldy;
  const int c = (int)a.c;
  float4_t v[NV];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = i * 256 + lane * 4;
    v[i] = float4_t{0.f, 0.f, 0.f, 0.f};
    if (e < c) v[i] = *reinterpret_cast<const float4_t*>(xr + e);
    s += (v[i][0] + v[i][1]) + (v[i][2] + v[i][3]);
  }
  const float mean = wave_sum64(s) / (float)c;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = i * 256 + lane * 4;
    if (e < c) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        v[i][j] -= mean;
        q += v[i][j] * v[i][j];
      }
    }
  }
  const float inv = 1.0f / sqrtf(wave_sum64(q) / (float)c + a.eps);
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = i * 256 + lane * 4;
    if (e < c) {
      uint16_t o[4];
      float sc[4] = {0.f, 0.f, 0.f, 0.f}, sh[4] = {0.f, 0.f, 0.f, 0.f};
      if (a.scale) mod_at4<MOD>(a.scale, e, sc);
      if (a.shift) mod_at4<MOD>(a.shift, e, sh);
#pragma unroll
      for (int j = 0; j < 4; j++)
        o[j] = modulate<MOD>(v[i][j] * inv, a.scale != nullptr, sc[j], a.shift != nullptr, sh[j]);
      *reinterpret_cast<uint2_t*>(yr + e) =
          uint2_t{(uint32_t)o[0] | ((uint32_t)o[1] << 16), (uint32_t)o[2] | ((uint32_t)o[3] << 16)};
    }
  }
}

// Any width and alignment: three passes over the row (it stays in cache), scalar accesses.
template <int MOD>
__global__ void __launch_bounds__(256) adaln_generic_kernel(const AdaLnArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.m) return;
  const float* xr = a.x + row * a.ldx;
  uint16_t* yr = a.y + row * a.ldy;
  float s = 0.f;
  for (int64_t e = lane; e < a.c; e += 64) s += xr[e];
  const float mean = wave_sum64(s) / (float)a.c;
  float q = 0.f;
  for (int64_t e = lane; e < a.c; e += 64) {
    const float d = xr[e] - mean;
    q += d * d;
  }
  const float inv = 1.0f / sqrtf(wave_sum64(q) / (float)a.c + a.eps);
  for (int64_t e = lane; e < a.c; e += 64)
    yr[e] = modulate<MOD>((xr[e] - mean) * inv, a.scale != nullptr, a.scale ? mod_at<MOD>(a.scale, e) : 0.f,
                          a.shift != nullptr, a.shift ? mod_at<MOD>(a.shift, e) : 0.f);
}

// fp16 rows with an elementwise affine weight and bias (fp16), fp16 out: lane l holds the 8 halfs at
// element 512 i + 8 l of every 512-element chunk i.  C % 8 == 0, 16-byte aligned rows, C <= NV * 512.
struct LayerNorm16Args {
  const uint16_t* x;
  int64_t ldx;
  int64_t m, c;
  const uint16_t* gamma;
  const uint16_t* beta;
  float eps;
  uint16_t* y;
  int64_t ldy;
};

__device__ __forceinline__ void unpack8(const uint4_t r, float (&o)[8]) {
#pragma unroll
  for (int q = 0; q < 4; q++) {
    o[2 * q] = (float)bits_to_half((uint16_t)r[q]);
    o[2 * q + 1] = (float)bits_to_half((uint16_t)(r[q] >> 16));
  }
}

template <int NV>
__global__ void __launch_bounds__(256) layernorm16_rows_kernel(const LayerNorm16Args a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.m) return;
  const uint16_t* xr = a.x + row * a.ldx;
  uint16_t* yr = a.y + row * a.ldy;
  const int c = (int)a.c;
  float v[NV][8];
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = i * 512 + lane * 8;
    uint4_t r = {0u, 0u, 0u, 0u};
    if (e < c) r = *reinterpret_cast<const uint4_t*>(xr + e);
    unpack8(r, v[i]);
#pragma unroll
    for (int j = 0; j < 8; j++) s += v[i][j];
  }
  const float mean = wave_sum64(s) / (float)c;
  float q = 0.f;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if (i * 512 + lane * 8 < c) {
#pragma unroll
      for (int j = 0; j < 8; j++) {
        v[i][j] -= mean;
        q += v[i][j] * v[i][j];
      }
    }
  }
  const float inv = 1.0f / sqrtf(wave_sum64(q) / (float)c + a.eps);
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int e = i * 512 + lane * 8;
    if (e < c) {
      float g[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f}, b[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (a.gamma) unpack8(*reinterpret_cast<const uint4_t*>(a.gamma + e), g);
      if (a.beta) unpack8(*reinterpret_cast<const uint4_t*>(a.beta + e), b);
      uint32_t o[4];
#pragma unroll
      for (int p = 0; p < 4; p++) {
        const uint16_t lo = half_to_bits((half_t)(v[i][2 * p] * inv * g[2 * p] + b[2 * p]));
        const uint16_t hi = half_to_bits((half_t)(v[i][2 * p + 1] * inv * g[2 * p + 1] + b[2 * p + 1]));
        o[p] = (uint32_t)lo | ((uint32_t)hi << 16);
      }
      *reinterpret_cast<uint4_t*>(yr + e) = uint4_t{o[0], o[1], o[2], o[3]};
    }
  }
}

// any width and alignment
__global__ void __launch_bounds__(256) layernorm16_generic_kernel(const LayerNorm16Args a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= a.m) return;
  const uint16_t* xr = a.x + row * a.ldx;
  uint16_t* yr = a.y + row * a.ldy;
  float s = 0.f;
  for (int64_t e = lane; e < a.c; e += 64) s += (float)bits_to_half(xr[e]);
  const float mean = wave_sum64(s) / (float)a.c;
  float q = 0.f;
  for (int64_t e = lane; e < a.c; e += 64) {
    const float d = (float)bits_to_half(xr[e]) - mean;
    q += d * d;
  }
  const float inv = 1.0f / sqrtf(wave_sum64(q) / (float)a.c + a.eps);
  for (int64_t e = lane; e < a.c; e += 64) {
    const float n = ((float)bits_to_half(xr[e]) - mean) * inv;
    const float g = a.gamma ? (float)bits_to_half(a.gamma[e]) : 1.f, b = a.beta ? (float)bits_to_half(a.beta[e]) : 0.f;
    yr[e] = half_to_bits((half_t)(n * g + b));
  }
}

template <int MOD>
static void launch_adaln(hipStream_t s, const AdaLnArgs& a, bool vec) {
  const dim3 grid((unsigned)((a.m + 3) / 4)), block(256);
  if (!vec || a.c > 32 * 256) {
    hipLaunchKernelGGL((adaln_generic_kernel<MOD>), grid, block, 0, s, a);
    return;
  }
  const int nv = (int)((a.c + 255) / 256);
  if (nv <= 4) hipLaunchKernelGGL((adaln_rows_kernel<4, MOD>), grid, block, 0, s, a);
  else if (nv <= 8) hipLaunchKernelGGL((adaln_rows_kernel<8, MOD>), grid, block, 0, s, a);
  else if (nv <= 12) hipLaunchKernelGGL((adaln_rows_kernel<12, MOD>), grid, block, 0, s, a);
  else if (nv <= 16) hipLaunchKernelGGL((adaln_rows_kernel<16, MOD>), grid, block, 0, s, a);
  else if (nv <= 20) hipLaunchKernelGGL((adaln_rows_kernel<20, MOD>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((adaln_rows_kernel<32, MOD>), grid, block, 0, s, a);
}

}  // namespace dt

DT_EXPORT dt_status dt_layernorm_modulate_f16(dt_stream stream, int64_t M, int64_t C, const float* X, int64_t ldx,
                                              const void* scale, const void* shift, int32_t mod, float eps,
                                              uint16_t* Y, int64_t ldy) {
  using namespace dt;
  if (M < 0 || C <= 0 || mod < DT_MOD_F16 || mod > DT_MOD_AFFINE_F32) return DT_INVALID;
  if (!(eps >= 0.f) || eps - eps != 0.f) return DT_INVALID;
  if (M == 0) return DT_OK;
  if (!X || !Y || ldx < C || ldy < C) return DT_INVALID;
  if ((reinterpret_cast<uintptr_t>(X) & 3) || (reinterpret_cast<uintptr_t>(Y) & 1)) return DT_INVALID;
  const uintptr_t vec_align = mod == DT_MOD_F16 ? 1 : 3;
  if ((reinterpret_cast<uintptr_t>(scale) & vec_align) || (reinterpret_cast<uintptr_t>(shift) & vec_align)) return DT_INVALID;
  if ((M + 3) / 4 > 0x7fffffff) return DT_NO_KERNEL;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  AdaLnArgs a{X, ldx, M, C, scale, shift, eps, Y, ldy};
  const bool vec = (C % 4 == 0) && (ldx % 4 == 0) && (ldy % 4 == 0) && (reinterpret_cast<uintptr_t>(X) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(Y) & 7) == 0 &&
                   (reinterpret_cast<uintptr_t>(scale) & (mod == DT_MOD_F16 ? 7 : 15)) == 0 &&
                   (reinterpret_cast<uintptr_t>(shift) & (mod == DT_MOD_F16 ? 7 : 15)) == 0;
  if (mod == DT_MOD_F16) launch_adaln<DT_MOD_F16>(as_stream(stream), a, vec);
  else if (mod == DT_MOD_F32) launch_adaln<DT_MOD_F32>(as_stream(stream), a, vec);
  else launch_adaln<DT_MOD_AFFINE_F32>(as_stream(stream), a, vec);
  return launch_status();
}

DT_EXPORT dt_status dt_layernorm_f16(dt_stream stream, int64_t M, int64_t C, const uint16_t* X, int64_t ldx,
                                     const uint16_t* gamma, const uint16_t* beta, float eps, uint16_t* Y, int64_t ldy) {
  using namespace dt;
  if (M < 0 || C <= 0) return DT_INVALID;
  if (!(eps >= 0.f) || eps - eps != 0.f) return DT_INVALID;
  if (M == 0) return DT_OK;
  if (!X || !Y || ldx < C || ldy < C) return DT_INVALID;
  if (((reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Y) | reinterpret_cast<uintptr_t>(gamma) |
        reinterpret_cast<uintptr_t>(beta)) & 1) != 0)
    return DT_INVALID;
  if ((M + 3) / 4 > 0x7fffffff) return DT_NO_KERNEL;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  const LayerNorm16Args a{X, ldx, M, C, gamma, beta, eps, Y, ldy};
  const bool vec = (C % 8 == 0) && (ldx % 8 == 0) && (ldy % 8 == 0) && C <= 8 * 512 &&
                   ((reinterpret_cast<uintptr_t>(X) | reinterpret_cast<uintptr_t>(Y) | reinterpret_cast<uintptr_t>(gamma) |
                     reinterpret_cast<uintptr_t>(beta)) & 15) == 0;
  const dim3 grid((unsigned)((M + 3) / 4)), block(256);
  hipStream_t s = as_stream(stream);
  if (!vec) hipLaunchKernelGGL(layernorm16_generic_kernel, grid, block, 0, s, a);
  else if (C <= 512) hipLaunchKernelGGL((layernorm16_rows_kernel<1>), grid, block, 0, s, a);
  else if (C <= 1024) hipLaunchKernelGGL((layernorm16_rows_kernel<2>), grid, block, 0, s, a);
  else if (C <= 2048) hipLaunchKernelGGL((layernorm16_rows_kernel<4>), grid, block, 0, s, a);
  else hipLaunchKernelGGL((layernorm16_rows_kernel<8>), grid, block, 0, s, a);
  return launch_status();
}


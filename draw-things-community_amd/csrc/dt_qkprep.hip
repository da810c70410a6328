// K2: RMSNorm (per head or per row) + RoPE complex multiply + optional scale
// on a [B, S, H, D] fp16 view.  HBM-bound: one read and one write per element.
// Rounds to fp16 after each of the three stages, as the op-by-op graph does.
#include "dt_common.h"
#include "dt_qkprep.h"

namespace dt {

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}

// normalise-rotate-scale one (re, im) pair that is already in registers
__device__ __forceinline__ uint32_t finish_pair(float a, float b, float inv, const uint16_t* gamma, int p,
                                                const uint16_t* rot_row, float post_scale) {
  if (gamma) {
    a = round_h(a * inv * (float)bits_to_half(gamma[p]));
    b = round_h(b * inv * (float)bits_to_half(gamma[p + 1]));
  }
  if (rot_row) {
    uint32_t r = *reinterpret_cast<const uint32_t*>(rot_row + p);
    float c = (float)bits_to_half((uint16_t)r), s = (float)bits_to_half((uint16_t)(r >> 16));
    float na = round_h(a * c - b * s);
    float nb = round_h(a * s + b * c);
    a = na;
    b = nb;
  }
  if (post_scale != 1.0f) {
    a = round_h(a * post_scale);
    b = round_h(b * post_scale);
  }
  return (uint32_t)half_to_bits((half_t)a) | ((uint32_t)half_to_bits((half_t)b) << 16);
}

// Per-head norm (or no norm), any even D <= 128 and 4-byte alignment: one wave per (b, s, h) row,
// lane p owns the complex pair (2p, 2p+1).
__global__ void __launch_bounds__(256) qk_prep_head_kernel(const QkPrepArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t wave = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  const int64_t rows = (int64_t)a.B * a.S * a.H;
  if (wave >= rows) return;
  const int h = (int)(wave % a.H);
  const int64_t bs = wave / a.H;
  const int64_t s = bs % a.S;
  const int64_t b = bs / a.S;
  const uint16_t* src = a.src + b * a.src_sb + s * a.src_ss + h * a.src_sh;
  uint16_t* dst = a.dst + b * a.dst_sb + s * a.dst_ss + h * a.dst_sh;
  const bool on = 2 * lane < a.D;
  float x0 = 0.f, x1 = 0.f;
  if (on) {
    uint32_t v = *reinterpret_cast<const uint32_t*>(src + 2 * lane);
    x0 = (float)bits_to_half((uint16_t)v);
    x1 = (float)bits_to_half((uint16_t)(v >> 16));
  }
  float inv = 1.f;
  if (a.gamma) {
    float ss = wave_sum(x0 * x0 + x1 * x1);
    inv = 1.0f / sqrtf(ss / (float)a.D + a.eps);
  }
  if (on) {
    const uint16_t* rot_row = a.rot ? a.rot + (a.rot_pos0 + s) * a.D : nullptr;
    *reinterpret_cast<uint32_t*>(dst + 2 * lane) = finish_pair(x0, x1, inv, a.gamma, 2 * lane, rot_row, a.post_scale);
  }
}

// Whole-row norm over H*D elements (stride_h == D): one workgroup per (b, s).
__global__ void __launch_bounds__(256) qk_prep_row_kernel(const QkPrepArgs a) {
  __shared__ float part[4];
  const int64_t bs = blockIdx.x;
  const int64_t s = bs % a.S;
  const int64_t b = bs / a.S;
  const int width = a.H * a.D;
  const uint16_t* src = a.src + b * a.src_sb + s * a.src_ss;
  uint16_t* dst = a.dst + b * a.dst_sb + s * a.dst_ss;
  float ss = 0.f;
  for (int p = 2 * threadIdx.x; p < width; p += 512) {
    uint32_t v = *reinterpret_cast<const uint32_t*>(src + p);
    float x0 = (float)bits_to_half((uint16_t)v), x1 = (float)bits_to_half((uint16_t)(v >> 16));
    ss += x0 * x0 + x1 * x1;
  }
  ss = wave_sum(ss);
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = ss;
  __syncthreads();
  ss = (part[0] + part[1]) + (part[2] + part[3]);
  const float inv = 1.0f / sqrtf(ss / (float)width + a.eps);
  const uint16_t* rot_row = a.rot ? a.rot + (a.rot_pos0 + s) * a.D : nullptr;
  for (int p = 2 * threadIdx.x; p < width; p += 512) {
    uint32_t v = *reinterpret_cast<const uint32_t*>(src + p);
    float x0 = (float)bits_to_half((uint16_t)v), x1 = (float)bits_to_half((uint16_t)(v >> 16));
    const int d = p % a.D;
    uint32_t out;
    // gamma is indexed over the whole row, the table over the head dimension
    if (a.gamma) {
      x0 = round_h(x0 * inv * (float)bits_to_half(a.gamma[p]));
      x1 = round_h(x1 * inv * (float)bits_to_half(a.gamma[p + 1]));
    }
    out = finish_pair(x0, x1, 1.f, nullptr, 0, rot_row ? rot_row + d : nullptr, a.post_scale);
    *reinterpret_cast<uint32_t*>(dst + p) = out;
  }
}

// ---- 16-byte forms ------------------------------------------------------------
// The same arithmetic with every access a whole 16-byte chunk (8 elements = 4 complex pairs): used when the
// head dimension is a multiple of 8 and every row, the table and the norm weight are 16-byte aligned.

// Per-head norm (or none): LPR = D / 8 lanes (a power of two) per (b, s, h) row, 256 / LPR rows per pass of a
// workgroup, kHeadPasses passes per thread with all their loads issued before the first use.
constexpr int kHeadPasses = 4;
template <int LPR>
__global__ void __launch_bounds__(256) qk_prep_head16_kernel(const QkPrepArgs a) {
  constexpr int RPP = 256 / LPR;  // rows per pass
  const int c = threadIdx.x % LPR;
  const int64_t rows = (int64_t)a.B * a.S * a.H;
  const int64_t row0 = (int64_t)blockIdx.x * (RPP * kHeadPasses) + threadIdx.x / LPR;
  uint4_t v[kHeadPasses], r[kHeadPasses] = {};
  uint16_t* dst[kHeadPasses];
  bool on[kHeadPasses];
  uint4_t g = {0, 0, 0, 0};
  if (a.gamma) g = *reinterpret_cast<const uint4_t*>(a.gamma + 8 * c);
#pragma unroll
  for (int i = 0; i < kHeadPasses; i++) {
    const int64_t row = row0 + i * RPP;
    on[i] = row < rows;
    const int64_t rc = on[i] ? row : rows - 1;
    const int h = (int)(rc % a.H);
    const int64_t bs = rc / a.H;
    const int64_t s = bs % a.S;
    const int64_t b = bs / a.S;
    v[i] = *reinterpret_cast<const uint4_t*>(a.src + b * a.src_sb + s * a.src_ss + h * a.src_sh + 8 * c);
    dst[i] = a.dst + b * a.dst_sb + s * a.dst_ss + h * a.dst_sh + 8 * c;
    if (a.rot) r[i] = *reinterpret_cast<const uint4_t*>(a.rot + (a.rot_pos0 + s) * a.D + 8 * c);
  }
#pragma unroll
  for (int i = 0; i < kHeadPasses; i++) {
    float x[8];
    unpack_chunk(v[i], x);
    float inv = 1.f;
    if (a.gamma) {
      float ss = 0.f;
#pragma unroll
      for (int e = 0; e < 8; e++) ss += x[e] * x[e];
#pragma unroll
      for (int off = LPR / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
      inv = 1.0f / sqrtf(ss / (float)a.D + a.eps);
    }
    const uint4_t out = finish_chunk(x, inv, a.gamma != nullptr, g, a.rot != nullptr, r[i], a.post_scale);
    if (on[i]) *reinterpret_cast<uint4_t*>(dst[i]) = out;
  }
}

// Whole-row norm over H * D <= 8192 elements: one wave per (b, s) row, the row held in registers between the
// sum of squares and the output -- one read, one write.
constexpr int kRowChunks = 16;  // 16-byte chunks per lane
__global__ void __launch_bounds__(256) qk_prep_row16_kernel(const QkPrepArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t bs = ((int64_t)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
  if (bs >= (int64_t)a.B * a.S) return;
  const int64_t s = bs % a.S;
  const int64_t b = bs / a.S;
  const int width = a.H * a.D;
  const int nc = width / 8;  // chunks in the row
  const uint16_t* src = a.src + b * a.src_sb + s * a.src_ss;
  uint16_t* dst = a.dst + b * a.dst_sb + s * a.dst_ss;
  uint4_t v[kRowChunks];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kRowChunks; i++) {
    const int ch = lane + 64 * i;
    v[i] = uint4_t{0, 0, 0, 0};
    if (ch < nc) v[i] = *reinterpret_cast<const uint4_t*>(src + 8 * ch);
  }
#pragma unroll
  for (int i = 0; i < kRowChunks; i++) {
    float x[8];
    unpack_chunk(v[i], x);
#pragma unroll
    for (int e = 0; e < 8; e++) ss += x[e] * x[e];
  }
  ss = wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)width + a.eps);
  const uint16_t* rot_row = a.rot ? a.rot + (a.rot_pos0 + s) * a.D : nullptr;
#pragma unroll
  for (int i = 0; i < kRowChunks; i++) {
    const int ch = lane + 64 * i;
    if (ch < nc) {
      float x[8];
      unpack_chunk(v[i], x);
      // the norm weight is indexed over the whole row, the table over the head dimension
      const uint4_t g = *reinterpret_cast<const uint4_t*>(a.gamma + 8 * ch);
      uint4_t r = {0, 0, 0, 0};
      if (rot_row) r = *reinterpret_cast<const uint4_t*>(rot_row + (8 * ch) % a.D);
      *reinterpret_cast<uint4_t*>(dst + 8 * ch) = finish_chunk(x, inv, true, g, rot_row != nullptr, r, a.post_scale);
    }
  }
}

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// every row of both views, the table and the norm weight can be accessed in 16-byte chunks
static bool chunks_ok(const QkPrepArgs& a) {
  return a.D % 8 == 0 && aligned16(a.src) && aligned16(a.dst) && a.src_sb % 8 == 0 && a.src_ss % 8 == 0 &&
         a.src_sh % 8 == 0 && a.dst_sb % 8 == 0 && a.dst_ss % 8 == 0 && a.dst_sh % 8 == 0 &&
         (!a.rot || aligned16(a.rot)) && (!a.gamma || aligned16(a.gamma));
}

dt_status qk_prep_launch(hipStream_t s, const QkPrepArgs& a) {
  if (a.B <= 0 || a.S <= 0 || a.H <= 0) return DT_OK;
  if (a.norm_per_head || !a.gamma) {
    int64_t rows = (int64_t)a.B * a.S * a.H;
    const int lpr = a.D / 8;
    if (chunks_ok(a) && (lpr == 16 || lpr == 8 || lpr == 4)) {
      const int per_block = (256 / lpr) * kHeadPasses;
      int64_t blocks = (rows + per_block - 1) / per_block;
      if (blocks > 0x7fffffff) return DT_NO_KERNEL;
      if (lpr == 16) hipLaunchKernelGGL(qk_prep_head16_kernel<16>, dim3((unsigned)blocks), dim3(256), 0, s, a);
      else if (lpr == 8) hipLaunchKernelGGL(qk_prep_head16_kernel<8>, dim3((unsigned)blocks), dim3(256), 0, s, a);
      else hipLaunchKernelGGL(qk_prep_head16_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, s, a);
      return launch_status();
    }
    int64_t blocks = (rows + 3) / 4;
    if (blocks > 0x7fffffff) return DT_NO_KERNEL;
    hipLaunchKernelGGL(qk_prep_head_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
  } else {
    const int64_t rows = (int64_t)a.B * a.S;
    if (chunks_ok(a) && (int64_t)a.H * a.D <= 8 * 64 * kRowChunks) {
      int64_t blocks = (rows + 3) / 4;
      if (blocks > 0x7fffffff) return DT_NO_KERNEL;
      hipLaunchKernelGGL(qk_prep_row16_kernel, dim3((unsigned)blocks), dim3(256), 0, s, a);
      return launch_status();
    }
    if (rows > 0x7fffffff) return DT_NO_KERNEL;
    hipLaunchKernelGGL(qk_prep_row_kernel, dim3((unsigned)rows), dim3(256), 0, s, a);
  }
  return launch_status();
}

}  // namespace dt

DT_EXPORT dt_status dt_qk_norm_rope_f16(dt_stream stream, dt_view4 x, int32_t B, int64_t S, int32_t H, int32_t D,
                                        const uint16_t* gamma, float eps, int32_t norm_per_head, const uint16_t* rot,
                                        int64_t rot_pos0, float post_scale) {
  using namespace dt;
  if (B < 0 || S < 0 || H <= 0 || D <= 0) return DT_INVALID;
  if (B == 0 || S == 0) return DT_OK;
  if (!x.ptr) return DT_INVALID;
  if (D % 2 != 0 || D > 128) return DT_NO_KERNEL;
  if ((reinterpret_cast<uintptr_t>(x.ptr) & 3) || (x.stride_b & 1) || (x.stride_s & 1) || (x.stride_h & 1))
    return DT_INVALID;
  if (rot && ((reinterpret_cast<uintptr_t>(rot) & 3) || rot_pos0 < 0)) return DT_INVALID;
  if (gamma && !norm_per_head && x.stride_h != D) return DT_INVALID;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  QkPrepArgs a;
  a.src = static_cast<const uint16_t*>(x.ptr);
  a.dst = static_cast<uint16_t*>(x.ptr);
  a.src_sb = a.dst_sb = x.stride_b;
  a.src_ss = a.dst_ss = x.stride_s;
  a.src_sh = a.dst_sh = x.stride_h;
  a.B = B;
  a.S = S;
  a.H = H;
  a.D = D;
  a.gamma = gamma;
  a.eps = eps;
  a.norm_per_head = norm_per_head;
  a.rot = rot;
  a.rot_pos0 = rot_pos0;
  a.post_scale = post_scale;
  return qk_prep_launch(as_stream(stream), a);
}

// Internal: the norm + rotate + scale pass, out of place (used by the
// attention entry point to stage Q and K) or in place.
#pragma once
#include "dt_common.h"

namespace dt {

struct QkPrepArgs {
  const uint16_t* src;
  uint16_t* dst;
  int64_t src_sb, src_ss, src_sh;
  int64_t dst_sb, dst_ss, dst_sh;
  int32_t B;
  int64_t S;
  int32_t H, D;
  const uint16_t* gamma;
  float eps;
  int32_t norm_per_head;
  const uint16_t* rot;
  int64_t rot_pos0;
  float post_scale;
};

dt_status qk_prep_launch(hipStream_t s, const QkPrepArgs& a);

#if defined(__HIPCC__)
// The pass's arithmetic on one 16-byte chunk (8 elements = 4 complex pairs), shared with the attention kernel, which
// applies it to the query fragments it holds in registers.
__device__ __forceinline__ float round_h(float v) { return round_f16(v); }

// normalise-rotate-scale the 8 elements of one chunk; g and r are the chunk's norm weights and table entries
__device__ __forceinline__ uint4_t finish_chunk(const float (&x)[8], float inv, bool has_gamma, const uint4_t& g,
                                                bool has_rot, const uint4_t& r, float post_scale) {
  uint4_t out;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    float a = x[2 * q], b = x[2 * q + 1];
    if (has_gamma) {
      a = round_h(a * inv * (float)bits_to_half((uint16_t)g[q]));
      b = round_h(b * inv * (float)bits_to_half((uint16_t)(g[q] >> 16)));
    }
    if (has_rot) {
      const float c = (float)bits_to_half((uint16_t)r[q]), sn = (float)bits_to_half((uint16_t)(r[q] >> 16));
      const float na = round_h(a * c - b * sn);
      const float nb = round_h(a * sn + b * c);
      a = na;
      b = nb;
    }
    if (post_scale != 1.0f) {
      a = round_h(a * post_scale);
      b = round_h(b * post_scale);
    }
    out[q] = (uint32_t)half_to_bits((half_t)a) | ((uint32_t)half_to_bits((half_t)b) << 16);
  }
  return out;
}

__device__ __forceinline__ void unpack_chunk(const uint4_t& v, float (&x)[8]) {
#pragma unroll
  for (int q = 0; q < 4; q++) {
    x[2 * q] = (float)bits_to_half((uint16_t)v[q]);
    x[2 * q + 1] = (float)bits_to_half((uint16_t)(v[q] >> 16));
  }
}
#endif

}  // namespace dt

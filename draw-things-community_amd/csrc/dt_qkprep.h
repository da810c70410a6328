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

}  // namespace dt

// Internal argument block of the attention kernel.
#pragma once
#include "dt_common.h"

namespace dt {

constexpr int kMaxSeg = 4;

struct SdpaSeg {
  const uint16_t* ptr;
  int64_t sb, ss, sh;
  int64_t start;  // first joint position of this segment
};

struct SdpaArgs {
  int32_t B, Hq, Hk, group, D;
  int64_t Sq, Skv;
  int32_t n_qseg, n_kvseg;
  SdpaSeg q[kMaxSeg], k[kMaxSeg], v[kMaxSeg];
  uint16_t* o;
  int64_t o_sb, o_ss, o_sh;
  float scale_log2e;
  int32_t q_tiles, total_blocks;  // filled by the launcher
};

dt_status sdpa_launch(hipStream_t s, const SdpaArgs& a);

// Device address of the current device's static scratch array (the one dt_sdpa_f16_static uses); looked up once
// per device.  nullptr on failure.
void* sdpa_static_scratch();

}  // namespace dt

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
  // Optional per-head RMSNorm and RoPE rotation of the queries, applied to the query fragments on their way into
  // registers (same arithmetic and rounding as the norm / rotate pass): q_gamma[i] is segment i's norm weight [D]
  // or null, q_rot the table [joint query rows, D] or null.
  const uint16_t* q_gamma[kMaxSeg];
  const uint16_t* q_rot;
  float q_eps;
  int32_t q_prep;  // any of the above is set
  // Key-split launch (optional; partials == nullptr runs one workgroup per task): workspace for the pieces' partial
  // results and the per-task tile counters, sized and laid out by sdpa_split_plan().
  float* partials;
  int32_t* counters;
  int64_t units;               // tasks * key tiles
  int32_t split_workgroups;
  int32_t q_tiles, total_blocks;  // filled by the launcher
};

// Floats of one partial-result slot of the key-split kernel: 512 threads x (DP / 32 * 16 accumulators + reference
// maximum + row-sum share).
constexpr int sdpa_split_slot_floats(int dp) { return (dp / 32) * 16 * 512 + 2 * 512; }

// How a launch would be split along the keys, and the workspace that takes.
struct SdpaSplit {
  int32_t workgroups;     // one equal run of (task, key tile) units each
  int32_t tasks;          // B * Hq * ceil(Sq / 256)
  int64_t units;          // tasks * ceil(Skv / 64)
  size_t counter_bytes;   // per-task tile counters (256-byte aligned), followed by
  size_t partial_bytes;   // two slots per workgroup
  size_t bytes() const { return counter_bytes + partial_bytes; }
};
// True when splitting pays: the task count leaves a good part of the last round of workgroups idle (or does not fill
// one round) and there are enough key tiles to cut.  Uses the compute-unit count of the calling thread's current device.
bool sdpa_split_plan(int32_t B, int32_t Hq, int32_t D, int64_t Sq, int64_t Skv, SdpaSplit* plan);

dt_status sdpa_launch(hipStream_t s, const SdpaArgs& a);

// Device address of the current device's static scratch array (the one dt_sdpa_f16_static uses); looked up once
// per device.  nullptr on failure.
void* sdpa_static_scratch();

}  // namespace dt

// K1 kernel template and its per-bit-width launcher, shared by dt_dense.hip (host side) and the
// dt_dense_q*.hip translation units that instantiate it (one per index width, so they build in parallel).
#pragma once
#include <numeric>
#include <type_traits>

#include "dt_common.h"
#include "dt_layout.h"
#include "dt_qkprep.h"

namespace dt {

constexpr int kMaxWeights = 8;
constexpr int kMaxGroups = 4;
constexpr int BK = 32;
constexpr int kPalLdsBytes = 32768;
// LDS a tile shape can spare for palettes: the tiles of 128 features have a weight ring half the size of the
// 256-feature tiles' (and the 128 x 128 tile X slots half the size too), which leaves room for a per-row table of
// 256-entry palettes (128 rows x 512 B = 64 KB; with 256 tokens: 64 KB of X slots + 24 KB of ring + 64 KB = 152 KB).
constexpr int pal_lds_bytes(int BM, int BN) { return BN == 128 ? 65536 : kPalLdsBytes; }

enum PalMode : int {
  kPalShared = 0,  // palettes of every block the tile's rows touch, loaded once, slot = block - first block
  kPalRow = 1,     // one palette per row in a transposed table, a row's column rewritten where its block changes
  kPalGlobal = 2,  // lookups go to global memory (any layout)
  kPlainF16 = 3    // weight is plain fp16, no palette
};

struct DenseWeight {
  const uint8_t* data;
  const uint16_t* bias;
  uint16_t* y;
  int64_t ldy;
  int32_t n;           // rows of this weight
  int32_t tile_begin;  // first N-tile index of this weight
  // optional fused epilogue on 128-wide heads: RMSNorm weight, RoPE table, its first row, epsilon
  const uint16_t* gamma;
  const uint16_t* rot;
  int64_t rot_pos0;
  float eps;
  // optional elementwise tail: scalar scale, fp16 addend, activation, per-feature gate, accumulation into an
  // fp32 residual stream
  float scale;           // 1 = none
  const uint16_t* add;   // [m, n] fp16 with row stride ld_add; null = none
  int64_t ld_add;
  int32_t act;          // DT_ACT_*
  const uint16_t* gate;  // [n] or null
  float* res;            // [m, n] fp32 with row stride ld_res, updated in place; null = none
  int64_t ld_res;
  const float* gate32;   // [n] fp32 or null: the residual receives float(result) * gate32 (no fp16 product)
  const uint16_t* mul;   // [m, n] fp16 with row stride ld_mul, multiplies the result; null = none
  int64_t ld_mul;
};

// The elementwise tail on one value that has already been rounded to fp16, with
// the rounding the op-by-op graph applies: after the scale, after the addition,
// after the activation and after the gate.
__device__ __forceinline__ float act_gelu_tanh(float x) {
  // 0.5 x (1 + tanh(u)) = x sigmoid(2u) = x / (1 + exp(-2u)): no cancellation for large negative x
  const float u = 0.7978845608028654f * (x + 0.044715f * x * x * x);
  const float e = __builtin_amdgcn_exp2f(u * -2.885390081777927f);  // exp(-2u)
  return x * __builtin_amdgcn_rcpf(1.0f + e);
}
__device__ __forceinline__ float act_swish(float x) {
  return x * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
// 1 + erf(z) = erfc(-z): no cancellation for large negative x
__device__ __forceinline__ float act_gelu_erf(float x) { return 0.5f * x * erfcf(x * -0.7071067811865476f); }
__device__ __forceinline__ float post_value(float v, float scale, bool has_add, float add, bool has_mul, float mul, int act,
                                            bool has_gate, float gate) {
  if (scale != 1.0f) v = round_f16(v * scale);
  if (has_add) v = round_f16(v + add);
  if (has_mul) v = round_f16(v * mul);
  if (act == DT_ACT_GELU_TANH) v = (float)(half_t)act_gelu_tanh(v);
  else if (act == DT_ACT_SWISH) v = (float)(half_t)act_swish(v);
  else if (act == DT_ACT_GELU_ERF) v = (float)(half_t)act_gelu_erf(v);
  if (has_gate) v = round_f16(v * gate);
  return v;
}

// One X with the weights applied to it; a launch runs up to kMaxGroups of them
// (same K and weight format), their tiles numbered one group after the other.
struct DenseGroup {
  const uint16_t* x;
  int64_t ldx;
  int32_t m;
  int32_t tiles_m, tiles_n;
  int32_t tile_begin;    // first tile of this group in the launch
  int32_t w_begin, w_end;  // its weights in DenseArgs::w
};

struct DenseArgs {
  int32_t k;
  int32_t nib;
  int32_t pal_step;  // K-tiles between columns at which a row can enter a new palette block: gcd(K, nib) / 32
  int32_t n_groups;
  int32_t total_tiles;
  DenseGroup g[kMaxGroups];
  DenseWeight w[kMaxWeights];
};

__device__ __forceinline__ uint4_t ld_global_16(const void* p) {
  return *reinterpret_cast<const uint4_t*>(p);
}

// Per-thread cursor over one weight row's packed indices, advanced one K-tile
// (32 elements) at a time so the main loop needs no division.
struct RowCursor {
  uint32_t off;   // byte offset of the current granule's first index dword
  uint32_t poff;  // byte offset of the current block's palette
  int32_t r;      // element offset inside the current block (multiple of 32)
  int32_t slot;   // palette slot in LDS (shared mode: block - first block of the tile)
};

// LDS tiles are [rows][32 halfs] with 64-byte rows and no padding; the 16-byte
// chunk c of row r lives at chunk c ^ ((r >> 2) & 3).  The LDS of this part
// serves 16 lanes of a 16-byte access per clock over 64 banks, so 16
// consecutive rows of one chunk column (the MFMA operand reads and the
// unpackers' row-per-lane writes) must land on 16 distinct 16-byte bank
// groups: 4 * (r % 4) + (c ^ (r / 4 % 4)) does.  Measured conflict-free for
// the operand reads, the 4-lanes-per-row tile writes and the row-per-lane writes.
__device__ __forceinline__ int lds_chunk(int row, int c) { return row * BK + ((c ^ ((row >> 2) & 3)) << 3); }

// Pair slots are [rows][64 halfs] (two K-tiles side by side): logical chunk c
// (0..7) of row r sits at 16-byte slot c ^ (r / 2 % 8), which puts 16
// consecutive rows of one chunk column on 16 distinct 16-byte bank groups.
__device__ __forceinline__ int pair_chunk(int row, int slot) { return slot ^ ((row >> 1) & 7); }

constexpr int kWaitVm0Lgkm0 = 0x0070;  // s_waitcnt vmcnt(0) lgkmcnt(0)
constexpr int kWaitLgkm0 = 0xc07f;     // s_waitcnt lgkmcnt(0)


// Sum over the 16 lanes of a DPP row (lanes 16 k .. 16 k + 15), left in every lane of the row.
__device__ __forceinline__ float row16_sum(float v) {
  auto dpp = [](float x, auto ctrl) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), decltype(ctrl)::value, 0xf, 0xf, false));
  };
  v += dpp(v, std::integral_constant<int, 0xB1>{});   // quad_perm [1, 0, 3, 2]
  v += dpp(v, std::integral_constant<int, 0x4E>{});   // quad_perm [2, 3, 0, 1]
  v += dpp(v, std::integral_constant<int, 0x124>{});  // row_ror 4
  v += dpp(v, std::integral_constant<int, 0x128>{});  // row_ror 8
  return v;
}

// Two floats rounded to fp16 (round to nearest even) in one dword, as one packed conversion.
__device__ __forceinline__ uint32_t pack_h2(float a, float b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, f16x2));
}

// ---- epilogue, shared by the tiled kernels -------------------------------------------------------------------
// acc: the wave's WN x WM slice as TN x TM blocks of 32 x 32 (rows = features, columns = tokens).  nw / mw: first
// feature (inside weight w) and first token of the slice; m_total: rows of X.  smem: the workgroup's LDS, free
// for reuse (the caller's K loop ended with a barrier); the wave parks its slice at smem + wave * WM * WN halfs.
template <int WN, int WM, bool POST>
__device__ __forceinline__ void dense_epilogue(float16_t (&acc)[WN / 32][WM / 32], unsigned char* smem, int wave, int lane,
                                               int nw, int64_t mw, const DenseWeight& w, int m_total) {
  constexpr int TN = WN / 32, TM = WM / 32;
  const int l32 = lane & 31, hi = lane >> 5;
  const bool head = WN == 128 && !POST && (w.gamma || w.rot);
  // ---- epilogue --------------------------------------------------------------
  // The K loop ended with a barrier, so its LDS tiles are free.  Every wave parks
  // its WN x WM slice -- bias added, rounded to fp16: the Dense's own result -- in
  // its own part of LDS as [token][feature] rows and then walks it row by row in a
  // short loop: RPI token rows per trip, CH lanes of 8 consecutive features per
  // row, so that every access to memory is a whole 16-byte chunk of a row (32 bytes
  // for the fp32 stream) and the code stays small (a fully unrolled walk over the
  // accumulators spends most of its time fetching instructions: measured 47 us per
  // workgroup for the GELU tail, against 7 us for this form).  The tails -- per-head
  // RMSNorm + RoPE, or scale / addend / activation / gate / residual -- run in that
  // loop, rounding to fp16 wherever the separate ops would; a plain Dense just
  // stores the parked rows.
  constexpr int CH = WN / 8;    // 16-byte chunks per parked row
  constexpr int RPI = 64 / CH;  // token rows per trip
  half_t* const park = reinterpret_cast<half_t*>(smem) + wave * (WM * WN);
  {
    // Accumulator block (i, j): lane holds token (lane & 31) of the block and
    // features 8 g + 4 (lane / 32) + (0..3), g = 0..3.  Chunk c of token t is
    // parked at chunk c ^ (t % CH): the 8-byte writes of 32 tokens spread over the banks.
#pragma unroll
    for (int i = 0; i < TN; i++)
#pragma unroll
      for (int gq = 0; gq < 4; gq++) {
        const int nn = nw + i * 32 + 8 * gq + 4 * hi;
        float b4[4] = {0.f, 0.f, 0.f, 0.f};
        if (w.bias) {
          if (nn + 3 < w.n && (reinterpret_cast<uintptr_t>(w.bias) & 7) == 0) {
            const uint2_t bb = *reinterpret_cast<const uint2_t*>(w.bias + nn);
            b4[0] = (float)bits_to_half((uint16_t)bb[0]);
            b4[1] = (float)bits_to_half((uint16_t)(bb[0] >> 16));
            b4[2] = (float)bits_to_half((uint16_t)bb[1]);
            b4[3] = (float)bits_to_half((uint16_t)(bb[1] >> 16));
          } else {
#pragma unroll
            for (int e = 0; e < 4; e++)
              if (nn + e < w.n) b4[e] = (float)bits_to_half(w.bias[nn + e]);
          }
        }
#pragma unroll
        for (int j = 0; j < TM; j++) {
          const int t = j * 32 + l32;
          const uint2_t pk = {pack_h2(acc[i][j][4 * gq] + b4[0], acc[i][j][4 * gq + 1] + b4[1]),
                              pack_h2(acc[i][j][4 * gq + 2] + b4[2], acc[i][j][4 * gq + 3] + b4[3])};
          *reinterpret_cast<uint2_t*>(park + t * WN + (((i * 4 + gq) ^ (t & (CH - 1))) << 3) + 4 * hi) = pk;
        }
      }
  }
  // a wave's LDS operations execute in order: its reads below see the writes above
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

  const int c = lane & (CH - 1), rsub = lane / CH;
  const int nn = nw + 8 * c;    // first of this lane's 8 features
  if (nw >= w.n) return;
  // this lane's column data
  float gt[8];  // the gate, or the RMSNorm weight of a head tile
#pragma unroll
  for (int e = 0; e < 8; e++) gt[e] = 1.f;
  auto lo16 = [](uint32_t v) { return (float)bits_to_half((uint16_t)v); };
  auto hi16 = [](uint32_t v) { return (float)bits_to_half((uint16_t)(v >> 16)); };
  if (head && w.gamma) {
    if ((reinterpret_cast<uintptr_t>(w.gamma) & 15) == 0) {
      const uint4_t gg = *reinterpret_cast<const uint4_t*>(w.gamma + 8 * c);
#pragma unroll
      for (int q = 0; q < 4; q++) {
        gt[2 * q] = lo16(gg[q]);
        gt[2 * q + 1] = hi16(gg[q]);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; e++) gt[e] = (float)bits_to_half(w.gamma[8 * c + e]);
    }
  }
  if constexpr (POST) {
#pragma unroll
    for (int e = 0; e < 8; e++)
      if (nn + e < w.n) {
        if (w.gate) gt[e] = (float)bits_to_half(w.gate[nn + e]);
        if (w.gate32) gt[e] = w.gate32[nn + e];
      }
  }
  // what a row needs from memory before its arithmetic
  struct RowIn {
    uint4_t add;  // the addend, or the RoPE table row of a head tile
    uint4_t mul;
    float4_t r0, r1;
  };
  // FAST: the wave's slice lies inside the matrix and every row meets the vector alignment
  // ACT: the activation when it is known where the loop is instantiated (the fast form is instantiated once
  // per activation, so that its body holds one activation's code), or -1 = taken from the arguments at run time
  auto walk = [&](auto fast_tag, auto act_tag) {
    constexpr bool FAST = decltype(fast_tag)::value;
    constexpr int ACT = decltype(act_tag)::value;
    auto fetch = [&](int it, RowIn& in) {
      const int t = it * RPI + rsub;
      const int64_t gm = mw + t;
      if (head && w.rot) in.add = *reinterpret_cast<const uint4_t*>(w.rot + (w.rot_pos0 + gm) * WN + 8 * c);
      if constexpr (POST) {
        if (w.add) in.add = *reinterpret_cast<const uint4_t*>(w.add + gm * w.ld_add + nn);
        if (w.mul) in.mul = *reinterpret_cast<const uint4_t*>(w.mul + gm * w.ld_mul + nn);
        if (w.res) {
          in.r0 = *reinterpret_cast<const float4_t*>(w.res + gm * w.ld_res + nn);
          in.r1 = *reinterpret_cast<const float4_t*>(w.res + gm * w.ld_res + nn + 4);
        }
      }
    };
    // Trips go in groups of GRP: the rows a group needs from memory are requested one group ahead, before the
    // previous group's stores (a load behind a store waits for it), so a trip does not wait a memory round trip.
    constexpr int TRIPS = WM / RPI;
    constexpr int GRP = (FAST && !POST) ? 4 : 1;
    static_assert(TRIPS % GRP == 0, "trips per group");
    RowIn cur[GRP];
    if constexpr (FAST) {
#pragma unroll
      for (int j = 0; j < GRP; j++) fetch(j, cur[j]);
    }
    for (int it0 = 0; it0 < TRIPS; it0 += GRP) {
      RowIn nxt[GRP];
      if constexpr (FAST) {
        if (it0 + GRP < TRIPS) {
#pragma unroll
          for (int j = 0; j < GRP; j++) fetch(it0 + GRP + j, nxt[j]);
        }
      }
#pragma unroll
      for (int j = 0; j < GRP; j++) {
      const int it = it0 + j;
      const int t = it * RPI + rsub;
      const int64_t gm = mw + t;
      const bool row_ok = FAST || gm < m_total;
      const int64_t gmc = row_ok ? gm : 0;
      const uint4_t raw = *reinterpret_cast<const uint4_t*>(park + t * WN + ((c ^ (t & (CH - 1))) << 3));
      float v[8] = {lo16(raw[0]), hi16(raw[0]), lo16(raw[1]), hi16(raw[1]),
                    lo16(raw[2]), hi16(raw[2]), lo16(raw[3]), hi16(raw[3])};
      float res[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
      if (head) {
        // per-head RMSNorm and RoPE: a parked row is one head, spread over the CH = 16 lanes of a DPP row
        if (w.gamma) {
          float ss = 0.f;
#pragma unroll
          for (int e = 0; e < 8; e++) ss += v[e] * v[e];
          ss = row16_sum(ss);
          const float inv = 1.0f / sqrtf(ss / (float)WN + w.eps);
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = round_f16(v[e] * inv * gt[e]);
        }
        if (w.rot) {
          uint4_t rr;
          if constexpr (FAST) {
            rr = cur[j].add;
          } else {
            const uint16_t* rrow = w.rot + (w.rot_pos0 + gmc) * WN + 8 * c;
#pragma unroll
            for (int q = 0; q < 4; q++) rr[q] = (uint32_t)rrow[2 * q] | ((uint32_t)rrow[2 * q + 1] << 16);
          }
#pragma unroll
          for (int q = 0; q < 4; q++) {
            const float cs = lo16(rr[q]), sn = hi16(rr[q]);
            const float re = v[2 * q], im = v[2 * q + 1];
            v[2 * q] = round_f16(re * cs - im * sn);
            v[2 * q + 1] = round_f16(re * sn + im * cs);
          }
        }
      }
      if constexpr (POST) {
        float ad[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
        if (w.add) {
          if constexpr (FAST) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
              ad[2 * q] = lo16(cur[j].add[q]);
              ad[2 * q + 1] = hi16(cur[j].add[q]);
            }
          } else if (row_ok) {
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (nn + e < w.n) ad[e] = (float)bits_to_half(w.add[gmc * w.ld_add + nn + e]);
          }
        }
        float ml[8] = {1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f, 1.f};
        if (w.mul) {
          if constexpr (FAST) {
#pragma unroll
            for (int q = 0; q < 4; q++) {
              ml[2 * q] = lo16(cur[j].mul[q]);
              ml[2 * q + 1] = hi16(cur[j].mul[q]);
            }
          } else if (row_ok) {
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (nn + e < w.n) ml[e] = (float)bits_to_half(w.mul[gmc * w.ld_mul + nn + e]);
          }
        }
        if (w.res) {
          if constexpr (FAST) {
#pragma unroll
            for (int e = 0; e < 4; e++) {
              res[e] = cur[j].r0[e];
              res[4 + e] = cur[j].r1[e];
            }
          } else if (row_ok) {
#pragma unroll
            for (int e = 0; e < 8; e++)
              if (nn + e < w.n) res[e] = w.res[gmc * w.ld_res + nn + e];
          }
        }
        // post_value's steps, each over the row's 8 values under one uniform test (a step that is off costs a
        // branch, not eight selects)
        const auto rh = [](float x) { return round_f16(x); };
        if (w.scale != 1.0f) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(v[e] * w.scale);
        }
        if (w.add) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(v[e] + ad[e]);
        }
        if (w.mul) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(v[e] * ml[e]);
        }
        const int act = ACT >= 0 ? ACT : w.act;
        if (act == DT_ACT_GELU_TANH) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(act_gelu_tanh(v[e]));
        } else if (act == DT_ACT_SWISH) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(act_swish(v[e]));
        } else if (act == DT_ACT_GELU_ERF) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(act_gelu_erf(v[e]));
        }
        if (w.gate) {
#pragma unroll
          for (int e = 0; e < 8; e++) v[e] = rh(v[e] * gt[e]);
        }
        if (w.res) {
#pragma unroll
          for (int e = 0; e < 8; e++) {
            float pr = w.gate32 ? v[e] * gt[e] : v[e];  // the fp32 gate's product is its own op: rounded before the addition
            asm volatile("" : "+v"(pr));
            res[e] += pr;
          }
        }
      }
      const uint4_t out = {pack_h2(v[0], v[1]), pack_h2(v[2], v[3]), pack_h2(v[4], v[5]), pack_h2(v[6], v[7])};
      if constexpr (FAST) {
        if constexpr (POST) {
          if (w.res) {
            *reinterpret_cast<float4_t*>(w.res + gm * w.ld_res + nn) = float4_t{res[0], res[1], res[2], res[3]};
            *reinterpret_cast<float4_t*>(w.res + gm * w.ld_res + nn + 4) = float4_t{res[4], res[5], res[6], res[7]};
          }
        }
        if (w.y) *reinterpret_cast<uint4_t*>(w.y + gm * w.ldy + nn) = out;
      } else if (row_ok) {
#pragma unroll
        for (int e = 0; e < 8; e++)
          if (nn + e < w.n) {
            if constexpr (POST) {
              if (w.res) w.res[gmc * w.ld_res + nn + e] = res[e];
            }
            if (w.y) w.y[gmc * w.ldy + nn + e] = (uint16_t)(out[e >> 1] >> (16 * (e & 1)));
          }
      }
      }
      if constexpr (FAST) {
#pragma unroll
        for (int j = 0; j < GRP; j++) cur[j] = nxt[j];
      }
    }
  };
  const bool aligned16 = (!w.y || (((w.ldy & 7) == 0) && (reinterpret_cast<uintptr_t>(w.y) & 15) == 0)) &&
                         (!(head && w.rot) || (reinterpret_cast<uintptr_t>(w.rot) & 15) == 0) &&
                         (!POST || ((!w.add || (((w.ld_add & 7) == 0) && (reinterpret_cast<uintptr_t>(w.add) & 15) == 0)) &&
                                    (!w.mul || (((w.ld_mul & 7) == 0) && (reinterpret_cast<uintptr_t>(w.mul) & 15) == 0)) &&
                                    (!w.res || (((w.ld_res & 3) == 0) && (reinterpret_cast<uintptr_t>(w.res) & 15) == 0))));
  if (aligned16 && nw + WN <= w.n && mw + WM <= m_total) {
    if constexpr (POST) {
      switch (w.act) {
        case DT_ACT_GELU_TANH: walk(std::true_type{}, std::integral_constant<int, DT_ACT_GELU_TANH>{}); break;
        case DT_ACT_SWISH: walk(std::true_type{}, std::integral_constant<int, DT_ACT_SWISH>{}); break;
        case DT_ACT_GELU_ERF: walk(std::true_type{}, std::integral_constant<int, DT_ACT_GELU_ERF>{}); break;
        default: walk(std::true_type{}, std::integral_constant<int, DT_ACT_NONE>{}); break;
      }
    } else {
      walk(std::true_type{}, std::integral_constant<int, DT_ACT_NONE>{});
    }
  } else {
    walk(std::false_type{}, std::integral_constant<int, -1>{});
  }
}

// 512 threads = 8 waves, two per SIMD, all eight running MFMAs on a (BN/2) x
// (BM/4) slice.  Every thread issues its share of the memory -> LDS transfer of
// X and unpacks / looks up half a granule (16 weights) of one W row per
// K-tile, so the LDS instructions -- the scarce resource: a wave can issue one
// only every few tens of clocks and the CU's LDS pipe handles one every 2-4 --
// are spread evenly over all waves and between their MFMAs.  The accumulators
// are held transposed (rows = output features n, columns = tokens m) so that
// each lane ends up with runs of consecutive n for one token: 16-byte stores.
// POST selects the epilogue with the elementwise tail.
template <int Q, int BM, int BN, int MODE, bool POST>
__global__ void __launch_bounds__(512) dense_qx_kernel(const DenseArgs a) {
  constexpr int WN = BN / 2, WM = BM / 4;   // per-wave slice: WN features x WM tokens
  constexpr int TN = WN / 32, TM = WM / 32;
  constexpr int AP = BM * (BK / 4) / 512;  // 16-byte chunks of X per thread per pair of K-tiles
  constexpr int BP = MODE == kPlainF16 ? BN * (BK / 4) / 512 : 0;  // plain fp16 weight: the same
  constexpr int QW = MODE == kPlainF16 ? 1 : Q;  // dwords per granule
  constexpr int HW = (QW + 1) / 2;               // dwords that hold either half of a granule
  constexpr int NST = 3;                         // ring depth of the unpacked weight tiles
  constexpr int B_STAGE = BN * BK;
  constexpr int PROW = 2 * BK;                   // halfs per row of a pair slot
  static_assert(BM % 128 == 0 && BN % 128 == 0 && BN <= 256, "tile");

  // One LDS array, carved up by hand so that the epilogue can reuse all of it.  The palettes come first:
  // their addresses then fit an instruction offset.  X (and a plain fp16 W) lives in two pair slots, each
  // holding two K-tiles as [rows][64 halfs]: one is read while the next pair is in flight into the other.
  constexpr bool HAS_PAL = MODE == kPalShared || MODE == kPalRow;
  constexpr int PAL_BYTES = HAS_PAL ? pal_lds_bytes(BM, BN) : 0;
  constexpr int XS_BYTES = BM * PROW * 2;
  constexpr int WP_BYTES = MODE == kPlainF16 ? BN * PROW * 2 : 0;
  constexpr int BS_BYTES = MODE == kPlainF16 ? 0 : NST * B_STAGE * 2;
  constexpr int OFF_XA = PAL_BYTES, OFF_XB = OFF_XA + XS_BYTES, OFF_WA = OFF_XB + XS_BYTES, OFF_WB = OFF_WA + WP_BYTES;
  constexpr int OFF_BS = OFF_WB + WP_BYTES, LOOP_BYTES = OFF_BS + BS_BYTES;
  constexpr int OUT_BYTES = BM * BN * 2;  // the fp16 output tile, parked here by the epilogue
  constexpr int LDS_BYTES = LOOP_BYTES > OUT_BYTES ? LOOP_BYTES : OUT_BYTES;
  __shared__ __attribute__((aligned(4096))) unsigned char smem[LDS_BYTES];
  half_t* const XsA = reinterpret_cast<half_t*>(smem + OFF_XA);
  half_t* const XsB = reinterpret_cast<half_t*>(smem + OFF_XB);
  half_t* const WpA = reinterpret_cast<half_t*>(smem + OFF_WA);
  half_t* const WpB = reinterpret_cast<half_t*>(smem + OFF_WB);
  half_t* const Bs = reinterpret_cast<half_t*>(smem + OFF_BS);
  uint16_t* const Pal = reinterpret_cast<uint16_t*>(smem);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  // Weight staging: two threads per weight row, each unpacking half of the row's 32-index granule.  With 256 rows
  // that is every thread: waves 0-3 take weights 0..15 of rows 0..255, waves 4-7 weights 16..31.  With 128 rows it
  // is half of them, and the four waves that stage are one per SIMD (waves 0-3: rows 64 * (wave % 2) + lane, half
  // wave / 2); waves 4-7 only run MFMAs and the X transfers.
  const bool second = BN == 256 ? wave >= 4 : ((wave >> 1) & 1) != 0;
  const bool stager = BN == 256 || __builtin_amdgcn_readfirstlane(wave) < 4;  // wave-uniform
  const int lt = BN == 256 ? (tid & 255) : (lane + 64 * (wave & 1));
  const int wn = wave & 1, wm = ((wave >> 1) & 1) | ((wave >> 2) << 1);  // waves w and w+4 share a SIMD and take different m slices

  // Tile order: bands of 4 token tiles; inside a band feature tiles outermost,
  // token tiles innermost.  Workgroups are dealt round-robin to the 8 XCDs;
  // giving each XCD a contiguous run of that order makes the workgroups that
  // run together on an XCD cover a compact 2-D block of tiles (4 token tiles x 8
  // feature tiles at 32 CUs: an X slice is 16 KB per K-tile, a packed W slice 4-8 KB),
  // so every X and W panel slice is fetched into that XCD's L2 once per block
  // instead of once per tile column.
  const int total = a.total_tiles;
  int bid = blockIdx.x;
  {
    const int per = total / 8;
    if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  }
  int gi = 0;
#pragma unroll
  for (int i = 1; i < kMaxGroups; i++)
    if (i < a.n_groups && bid >= a.g[i].tile_begin) gi = i;
  const DenseGroup g = a.g[gi];
  bid -= g.tile_begin;
  int tm, tn;
  {
    constexpr int GM = 4;
    const int band_tiles = GM * g.tiles_n;
    const int band = bid / band_tiles;
    const int in_band = bid - band * band_tiles;
    const int rows_in_band = (g.tiles_m - band * GM) < GM ? (g.tiles_m - band * GM) : GM;
    tn = in_band / rows_in_band;
    tm = band * GM + (in_band - tn * rows_in_band);
  }

  int wi = g.w_begin;
#pragma unroll
  for (int i = 1; i < kMaxWeights; i++)
    if (i > g.w_begin && i < g.w_end && tn >= a.w[i].tile_begin) wi = i;
  const DenseWeight w = a.w[wi];
  const int n0 = (tn - w.tile_begin) * BN;
  const int m0 = tm * BM;
  const int K = a.k;
  const int nk = K / BK;
  const QxLayout lay = make_layout(Q, a.nib);
  const uint32_t pal_bytes = (uint32_t)lay.pal_bytes;
  // ---- per-thread load coordinates (32-bit byte offsets from uniform bases) ----
  // X (and a plain fp16 W) goes from memory straight into LDS, two K-tiles at
  // a time: eight lanes cover one row's 128 contiguous bytes, so every cache
  // line is requested once, whole.  A wave's load instruction fills 1 KB of
  // LDS = 8 rows of a pair slot, lane l landing on 16-byte slot l % 8 of row
  // l / 8; the lane fetches the chunk that the swizzle assigns to that slot.
  uint32_t a_off[AP];
#pragma unroll
  for (int i = 0; i < AP; i++) {
    const int row = 8 * (wave * AP + i) + (lane >> 3);
    const int c8 = pair_chunk(row, lane & 7);
    int gm = m0 + row;
    if (gm >= g.m) gm = g.m - 1;
    a_off[i] = (uint32_t)(((int64_t)gm * g.ldx + c8 * 8) * 2);
  }
  const char* xbase = reinterpret_cast<const char*>(g.x);
  const char* wbase = reinterpret_cast<const char*>(w.data);

  // weight row of this thread (two threads per row; each loads and unpacks one half of the row's granule)
  const int b_row = lt < BN ? lt : BN - 1;
  RowCursor cur;
  int64_t pal_first_block = 0;
  if constexpr (MODE == kPalShared) pal_first_block = ((int64_t)n0 * K) / a.nib;
  if constexpr (MODE != kPlainF16) {
    int gn = n0 + b_row;
    if (gn >= w.n) gn = w.n - 1;
    const int64_t e = (int64_t)gn * K;
    const int64_t blk = e / a.nib;
    const int64_t r = e - blk * a.nib;
    cur.off = (uint32_t)index_byte_offset(lay, blk, r);
    cur.poff = (uint32_t)palette_offset(lay, blk);
    cur.r = (int32_t)r;
    cur.slot = MODE == kPalShared ? (int32_t)(blk - pal_first_block) : b_row;
    if (second) cur.off += 4 * (Q / 2);  // first dword that holds an index of the granule's second half
  }
  uint32_t bf_off[BP > 0 ? BP : 1];
  if constexpr (MODE == kPlainF16) {
#pragma unroll
    for (int i = 0; i < BP; i++) {
      const int row = 8 * (wave * BP + i) + (lane >> 3);
      const int c8 = pair_chunk(row, lane & 7);
      int gn = n0 + row;
      if (gn >= w.n) gn = w.n - 1;
      bf_off[i] = (uint32_t)(((int64_t)gn * K + c8 * 8) * 2);
    }
  }

  // ---- palettes -> LDS --------------------------------------------------
  if constexpr (MODE == kPalShared) {
    int last_row = n0 + BN - 1;
    if (last_row >= w.n) last_row = w.n - 1;
    int64_t last_block = ((int64_t)last_row * K + (K - 1)) / a.nib;
    int n_pal = (int)(last_block - pal_first_block + 1);
    const int per_pal = 1 << (Q - 1);  // dwords per palette
    for (int i = tid; i < n_pal * per_pal; i += 512) {
      int p = i / per_pal, e = i - p * per_pal;
      const uint32_t* src =
          reinterpret_cast<const uint32_t*>(w.data + palette_offset(lay, pal_first_block + p));
      reinterpret_cast<uint32_t*>(Pal)[i] = src[e];
    }
  }
  // kPalRow: Pal is a table [128-row group][entry][row % 64][row / 64 % 2] of
  // fp16: rows r and r + 64 share a dword, so the 64 lanes of a wave (64
  // consecutive rows, one entry each) hit 64 different banks whatever entries
  // they ask for.  Each of a row's two threads keeps half of the row's column current.
  const int pal_col = (b_row >> 7) * (256 << Q) + (b_row & 63) * 4 + ((b_row >> 6) & 1) * 2;  // byte offset of this row's column
  auto fill_pal_column = [&](int64_t blk) {
    if (!stager) return;
    constexpr int ND = (1 << Q) / 4;  // dwords of palette per thread
    const uint32_t* src =
        reinterpret_cast<const uint32_t*>(w.data + palette_offset(lay, blk)) + (second ? ND : 0);
    char* dst = reinterpret_cast<char*>(Pal) + pal_col + (second ? (128 << Q) : 0);
#pragma unroll
    for (int d = 0; d < ND; d++) {
      const uint32_t v = src[d];
      *reinterpret_cast<uint16_t*>(dst + (2 * d) * 256) = (uint16_t)v;
      *reinterpret_cast<uint16_t*>(dst + (2 * d + 1) * 256) = (uint16_t)(v >> 16);
    }
  };
  int gn_row = n0 + b_row;  // this thread's weight row
  if (gn_row >= w.n) gn_row = w.n - 1;
  // rewrites the column if the row enters a new block at K-tile `tile`
  auto refresh_pal_column = [&](int tile) {
    const int64_t e = (int64_t)gn_row * K + (int64_t)tile * BK;
    const int64_t blk = e / a.nib;
    if (e == blk * a.nib) fill_pal_column(blk);
  };
  int next_pal_tile = a.pal_step;  // next K-tile at which some row may change block
  if constexpr (MODE == kPalRow) fill_pal_column(((int64_t)gn_row * K) / a.nib);

  // ---- staging --------------------------------------------------------------
  struct IdxSet {
    uint32_t b[HW];  // the dwords that hold this thread's half of the row's granule
    uint32_t poff;
    int32_t slot;
  };
  IdxSet WS[2];  // tile T travels in WS[T % 2]
  const int last_pair = nk / 2 - 1;
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);

  // Part i (of AP + BP) of the memory -> LDS transfer of K-tile pair q into a
  // pair slot (pairs past the end re-read the last one, harmlessly).
  auto issue_pair_part = [&](half_t* xs, half_t* wp, int q, int i) {
    if (q > last_pair) q = last_pair;
    const int64_t kb = (int64_t)q * (4 * BK);  // byte offset of the pair inside a row
    if (i < AP) {
      load_to_lds_16(xbase + kb, a_off[i], lds_address(xs) + (uint32_t)((wave_u * AP + i) * 1024));
    } else if constexpr (MODE == kPlainF16) {
      load_to_lds_16(wbase + kb, bf_off[i - AP], lds_address(wp) + (uint32_t)((wave_u * BP + i - AP) * 1024));
    }
  };
  auto issue_pair = [&](half_t* xs, half_t* wp, int q) {
#pragma unroll
    for (int i = 0; i < AP + BP; i++) issue_pair_part(xs, wp, q, i);
  };

  // Loads the indices of the tile the cursor points at (the last tile is re-read
  // harmlessly by the final iterations) and moves the cursor on by one tile.
  int issued = 0;  // tiles loaded so far
  auto issue_idx = [&](IdxSet& R) {
    if constexpr (MODE != kPlainF16) {
      if (!stager) return;
      const uint32_t* src = reinterpret_cast<const uint32_t*>(wbase + cur.off);
#pragma unroll
      for (int i = 0; i < HW; i++) R.b[i] = src[i];
      R.poff = cur.poff;
      R.slot = cur.slot;
      if (issued + 1 < nk) {
        issued++;
        cur.r += BK;
        cur.off += 4 * Q;
        if (cur.r >= a.nib) {
          cur.r = 0;
          cur.off += pal_bytes;
          cur.poff += (uint32_t)lay.block_stride;
          if constexpr (MODE == kPalShared) cur.slot++;
        }
      }
    }
  };

  // Staging of a weight tile, in pieces that the main loop spreads between its
  // MFMAs: unpack the 16 indices into palette byte offsets, look them up one
  // by one, write the 16 weights as two 16-byte chunks.  Threads past the tile's
  // last row repeat that row's work and write the same bytes again.
  uint32_t la[16];  // palette byte offsets, then the looked-up weights
  uint32_t be[HW + 1];
  const char* gpal = nullptr;
  uint32_t pal_base = 0;
  // piece 0 also turns the index dwords into a bit string; piece p yields offsets 4p .. 4p+3
  auto unpack_piece = [&](IdxSet& R, int p) {
    if constexpr (MODE != kPlainF16) {
      if (!stager) return;
      if (p == 0) {
        own_bits<Q, HW>(R.b, second, be);
        if constexpr (MODE == kPalRow) pal_base = (uint32_t)pal_col;
        else if constexpr (MODE == kPalGlobal) gpal = wbase + R.poff;
        else pal_base = (uint32_t)R.slot << (Q + 1);
      }
#pragma unroll
      for (int j = 4 * p; j < 4 * p + 4; j++)
        la[j] = own_index_at<Q, HW, (MODE == kPalRow ? 8 : 1)>(be, j, pal_base);
    }
  };
  auto lookup = [&](int j) {
    if (!stager) return;
    if constexpr (MODE == kPalGlobal)
      la[j] = *reinterpret_cast<const uint16_t*>(gpal + la[j]);
    else if constexpr (MODE != kPlainF16)
      la[j] = *reinterpret_cast<const uint16_t*>(reinterpret_cast<const char*>(Pal) + la[j]);
  };
  // Written as assembly, like the transfers: the closing s_waitcnt of an
  // iteration covers these stores, and the compiler has no reason to order
  // them against anything else.
  // unpacked weight tiles are chunk-major, [4 chunks of 8 k][BN rows][8 halfs]: a wave's 64 rows of one chunk are
  // 1 KB of consecutive addresses, for the row-per-lane writes here and for the row-per-lane operand reads alike
  auto w_chunk = [](int row, int c) { return (c * BN + row) * 8; };
  const uint32_t w_dst = lds_address(Bs) + 2u * (uint32_t)w_chunk(b_row, second ? 2 : 0);
  auto write_weights = [&](int stage, int h) {
    if constexpr (MODE != kPlainF16) {
      if (!stager) return;
      const uint4_t v = {la[8 * h] | (la[8 * h + 1] << 16), la[8 * h + 2] | (la[8 * h + 3] << 16),
                         la[8 * h + 4] | (la[8 * h + 5] << 16), la[8 * h + 6] | (la[8 * h + 7] << 16)};
      const uint32_t addr = w_dst + (uint32_t)(stage * B_STAGE * 2) + (uint32_t)(h * BN * 16);
      asm volatile("ds_write_b128 %0, %1" : : "v"(addr), "v"(v) : "memory");
    }
  };
  auto stage_to_lds = [&](IdxSet& R, int stage) {  // all at once (prologue)
#pragma unroll
    for (int p = 0; p < 4; p++) unpack_piece(R, p);
#pragma unroll
    for (int j = 0; j < 16; j++) lookup(j);
    write_weights(stage, 0);
    write_weights(stage, 1);
  };
  // Makes the wait for an index load happen here rather than at its first use.
  auto touch = [&](IdxSet& R) {
    if constexpr (MODE != kPlainF16) {
      if (!stager) return;
#pragma unroll
      for (int j = 0; j < HW; j++) asm volatile("" : "+v"(R.b[j]));
    }
  };

  float16_t acc[TN][TM];
#pragma unroll
  for (int i = 0; i < TN; i++)
#pragma unroll
    for (int j = 0; j < TM; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  // ---- fragment double buffer --------------------------------------------
  // MFMA A operand = W rows (features), B operand = X rows (tokens); lane holds
  // row (lane & 31), k-slots 8 * (lane / 32) .. + 7 of the 16-wide k-step.
  // In a pair slot the 16-byte chunk c (0..7: tile parity * 4 + k-step * 2 +
  // half) of row r sits at slot c ^ (r / 2 % 8); rows 32 apart share a swizzle.
  const int l32 = lane & 31, hi = lane >> 5;
  const int xrow = wm * WM + l32, wrow = wn * WN + l32;
  const int x_lane = xrow * PROW + ((hi ^ ((xrow >> 1) & 7)) << 3);  // halfs; chunk bits xor'ed per read
  const int w_lane = wrow * PROW + ((hi ^ ((wrow >> 1) & 7)) << 3);
  half8_t fw[2][TN], fx[2][TM];
  // par: tile of the pair (0/1), ks: k-step of the tile, stage: ring stage of the unpacked weights
  auto read_w = [&](int buf, int i, const half_t* wp, int par, int stage, int ks) {
    if constexpr (MODE == kPlainF16)
      fw[buf][i] = *reinterpret_cast<const half8_t*>(wp + (w_lane ^ ((4 * par + 2 * ks) << 3)) + i * 32 * PROW);
    else
      fw[buf][i] = *reinterpret_cast<const half8_t*>(Bs + stage * B_STAGE + ((2 * ks + hi) * BN + wrow + i * 32) * 8);
  };
  auto read_x = [&](int buf, int j, const half_t* xs, int par, int ks) {
    fx[buf][j] = *reinterpret_cast<const half8_t*>(xs + (x_lane ^ ((4 * par + 2 * ks) << 3)) + j * 32 * PROW);
  };
  auto mfma = [&](int buf, int i, int j) {
    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw[buf][i], fx[buf][j], acc[i][j], 0, 0, 0);
  };

  // ---- prologue: pair 0 in slot A, weights of tiles 0 and 1 in the ring --------
  issue_pair(XsA, WpA, 0);
  issue_idx(WS[0]);  // tile 0
  issue_idx(WS[1]);  // tile 1
  __syncthreads();   // palettes visible
  stage_to_lds(WS[0], 0);
  issue_idx(WS[0]);  // tile 2
  if constexpr (MODE == kPalRow) {
    if (next_pal_tile == 1) {  // tile 1 may already start a new palette block
      __syncthreads();
      refresh_pal_column(1);
      next_pal_tile += a.pal_step;
      __syncthreads();
    }
  }
  stage_to_lds(WS[1], 1);
  issue_idx(WS[1]);  // tile 3
  __builtin_amdgcn_s_waitcnt(kWaitVm0Lgkm0);
  __syncthreads();
  if constexpr (MODE == kPlainF16) issue_pair(XsB, WpB, 1);  // (the loop issues pair q + 2 from the middle of pair q)
#pragma unroll
  for (int i = 0; i < TN; i++) read_w(0, i, WpA, 0, 0, 0);
#pragma unroll
  for (int j = 0; j < TM; j++) read_x(0, j, XsA, 0, 0);

  // Iteration t: MFMAs of tile t (pair t / 2) while the weights of tile t+2
  // are unpacked into ring stage (t+2) % 3.  An even iteration starts the
  // transfer of the next pair into the other slot (free since the barrier
  // that ended tile t-1) and waits for it before its closing barrier, because
  // the odd iteration reads one k-step ahead into that pair.  Index registers
  // are refilled in odd iterations only, so the even iteration's wait covers
  // nothing that was issued just before it.
  //
  // A wave issues in order, and an LDS instruction occupies it for tens of
  // clocks, so the iteration is written as 16 slots of one MFMA followed by
  // a share of the LDS and VALU work: the fragment reads of the next k-step,
  // the palette lookups and the weight writes all issue while an MFMA of the
  // same wave (or of the wave it shares the SIMD with) is executing.
  int s_cur = 0, s_nxt = 1, s_fill = 2;
  auto iteration = [&](int t, int par, half_t* xs, half_t* wp, half_t* xs_other, half_t* wp_other) {
    if constexpr (MODE == kPalRow) {
      if (t + 2 == next_pal_tile) {
        // lookups of tile t+1 finished before the last barrier
        if (t + 2 < nk) refresh_pal_column(t + 2);
        next_pal_tile += a.pal_step;
        __syncthreads();
      }
    }
    IdxSet& R = WS[par];
    // the wait for the indices comes here, before the transfer goes out: vector
    // memory loads return in order, so a wait with the transfer outstanding
    // would last until it lands
    touch(R);
    if (par) issue_idx(WS[0]);  // tile t+3
    const half_t* xs_n = par == 0 ? xs : xs_other;  // fragments of tile t+1, k-step 0
    const half_t* wp_n = par == 0 ? wp : wp_other;
    constexpr int NM = TN * TM;  // MFMAs per k-step = slots per phase
    constexpr int NF = TN + TM;  // fragment reads per phase
    constexpr bool packed = MODE != kPlainF16;
    // Phase 0 (k-step 0): the fragments of k-step 1, one every third place;
    // between them the parts of the transfer (even iterations), the unpacking,
    // the refill of the index registers (odd iterations), the first 8 lookups.
    const int nd = par == 0 ? AP + BP : 0;
    const int ns0 = nd + (packed ? 4 + par + 8 : 0);
    auto stage0 = [&](int s) {
      if (s < nd) { issue_pair_part(xs_other, wp_other, (t >> 1) + 1, s); return; }
      s -= nd;
      if (!packed) return;
      if (s < 4) { unpack_piece(R, s); return; }
      s -= 4;
      if (par) {
        if (s == 0) { issue_idx(WS[1]); return; }  // tile t+4
        s -= 1;
      }
      if (s < 8) lookup(s);
    };
    // Phase 1 (k-step 1): the next tile's first fragments (every k-step 0
    // MFMA has been issued, so their registers are free), the other lookups,
    // the two weight writes.
    const int ns1 = packed ? 10 : 0;
    auto stage1 = [&](int s) {
      if (!packed) return;
      if (s < 8) lookup(8 + s);
      else if (s < 10) write_weights(s_fill, s - 8);
    };
    auto read0 = [&](int r) {
      if (r < TN) read_w(1, r, wp, par, s_cur, 1);
      else read_x(1, r - TN, xs, par, 1);
    };
    auto read1 = [&](int r) {
      if (r < TN) read_w(0, r, wp_n, par ^ 1, s_nxt, 0);
      else read_x(0, r - TN, xs_n, par ^ 1, 0);
    };
    // place k of a phase: a read at every third place while reads last, stage parts elsewhere
    auto place = [&](int k, int ns, auto&& rd, auto&& st) {
      if (k < 3 * NF) {
        if (k % 3 == 0) rd(k / 3);
        else if ((k / 3) * 2 + k % 3 - 1 < ns) st((k / 3) * 2 + k % 3 - 1);
      } else if (k - NF < ns) {
        st(k - NF);
      }
    };
    if constexpr (!packed) {
      // Plain fp16 weights: both operands arrive by transfer and nothing is written to LDS by the waves, so one
      // barrier per pair of K-tiles is enough, and it sits in the middle of the odd iteration: by then the pair in
      // flight has had two iterations to land, the reads of this pair's last k-step were issued half an
      // iteration ago, and what follows the barrier is exactly what needs it -- the first reads from the other
      // slot and the transfer of the pair after next into this one.
      constexpr int RPS = (NF + NM - 1) / NM;            // fragment reads per MFMA, front-loaded
      constexpr int PPS = (AP + BP + NM - 1) / NM;       // transfer parts per MFMA
#pragma unroll
      for (int m = 0; m < NM; m++) {
        __builtin_amdgcn_sched_barrier(0);
        mfma(0, m / TM, m % TM);
#pragma unroll
        for (int r = m * RPS; r < (m + 1) * RPS; r++)
          if (r < NF) read0(r);
      }
      if (par) {
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(kWaitVm0Lgkm0);
        __syncthreads();
      }
#pragma unroll
      for (int m = 0; m < NM; m++) {
        __builtin_amdgcn_sched_barrier(0);
        mfma(1, m / TM, m % TM);
#pragma unroll
        for (int r = m * RPS; r < (m + 1) * RPS; r++)
          if (r < NF) read1(r);
        if (par) {
          // this iteration's slot is free from the barrier on: the pair after next goes into it
#pragma unroll
          for (int q = m * PPS; q < (m + 1) * PPS; q++)
            if (q < AP + BP) issue_pair_part(xs, wp, (t >> 1) + 2, q);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      return;
    }
    const int n0 = NF + (ns0 > 2 * NF ? ns0 : 2 * NF);
    const int n1 = NF + (ns1 > 2 * NF ? ns1 : 2 * NF);
#pragma unroll
    for (int m = 0; m < NM; m++) {
      __builtin_amdgcn_sched_barrier(0);
      mfma(0, m / TM, m % TM);
#pragma unroll
      for (int k = m * n0 / NM; k < (m + 1) * n0 / NM; k++) place(k, ns0, read0, stage0);
    }
#pragma unroll
    for (int m = 0; m < NM; m++) {
      __builtin_amdgcn_sched_barrier(0);
      mfma(1, m / TM, m % TM);
#pragma unroll
      for (int k = m * n1 / NM; k < (m + 1) * n1 / NM; k++) place(k, ns1, read1, stage1);
    }
    __builtin_amdgcn_sched_barrier(0);
    if (par == 0)
      __builtin_amdgcn_s_waitcnt(kWaitVm0Lgkm0);
    else
      __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __syncthreads();
    const int s = s_cur;
    s_cur = s_nxt;
    s_nxt = s_fill;
    s_fill = s;
  };

  int t = 0;
  for (; t + 3 < nk; t += 4) {
    iteration(t, 0, XsA, WpA, XsB, WpB);
    iteration(t + 1, 1, XsA, WpA, XsB, WpB);
    iteration(t + 2, 0, XsB, WpB, XsA, WpA);
    iteration(t + 3, 1, XsB, WpB, XsA, WpA);
  }
  if (t < nk) {  // nk is even: two iterations left
    iteration(t, 0, XsA, WpA, XsB, WpB);
    iteration(t + 1, 1, XsA, WpA, XsB, WpB);
  }

  if constexpr (MODE == kPlainF16) {
    // the loop's last barrier lies before the last reads (and every transfer was waited for ahead of it)
    __builtin_amdgcn_s_waitcnt(kWaitVm0Lgkm0);
    __syncthreads();
  }
  dense_epilogue<WN, WM, POST>(acc, smem, wave, lane, n0 + wn * WN, (int64_t)m0 + wm * WM, w, g.m);
}

}  // namespace dt

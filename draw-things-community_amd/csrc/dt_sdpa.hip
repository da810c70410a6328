// K3: ScaledDotProductAttention, flash-style, fp16 in / fp32 statistics, gfx950.
//
// One 256-thread workgroup owns 4 * QB * 32 query rows of one (batch, head);
// each wave owns QB blocks of 32 rows.  K/V arrive in tiles of 64 keys that
// are staged through LDS (double-buffered, one barrier per tile).
//
// Everything is computed transposed so that the query index is the MFMA
// column (lane & 31) in every stage:
//   S^T = K Q^T          A = K tile rows from LDS, B = Q^T held in registers
//   O^T = V^T P^T        A = V^T from LDS,         B = P^T = the S^T accumulator
// The accumulator of a 32x32 MFMA holds, for column q = lane & 31, rows
// 8*(v/4) + 4*(lane/32) + (v%4), v = 0..15.  Feeding it back as the B operand
// only permutes the summation index, so the V^T operand is read from LDS with
// the same permutation and P never leaves registers.  The softmax row
// reductions are therefore in-lane plus one exchange with lane ^ 32.
#include "dt_common.h"
#include "dt_sdpa.h"

namespace dt {

constexpr int BKV = 64;  // keys per tile

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ float xor32(float v) { return __shfl_xor(v, 32, 64); }

// V^T tile in LDS: row d holds 64 keys as 16 units of 4 keys (8 bytes); unit u
// of row d is stored at unit u ^ f(d).  Writers (fixed key group, d = 8*g + j
// over 16 lanes) and readers (fixed unit, 16 consecutive d) both hit 16
// distinct units, i.e. all 32 banks once.
__device__ __forceinline__ int vt_swz(int d) { return (d & 15) ^ ((d >> 4) & 7); }

template <int DP>
struct SdpaSmem {
  static constexpr int KROW = DP + 8;  // halfs; 16 extra bytes per row spread 16-byte reads of 8 consecutive keys over all banks
  half_t k[2][BKV * KROW];
  half_t vt[2][DP * BKV];
};

template <int DP, int QB>
__global__ void __launch_bounds__(256) sdpa_kernel(const SdpaArgs a) {
  constexpr int KROW = SdpaSmem<DP>::KROW;
  constexpr int DCH = DP / 8;                 // 16-byte chunks per row
  constexpr int K_LOADS = BKV * DCH / 256;    // per thread per tile (4 at DP = 128)
  constexpr int V_TASKS = (BKV / 4) * DCH;    // 4-key x 8-d transposes per tile
  constexpr int DB = DP / 32;                 // 32-wide blocks of the head dimension
  constexpr int KS = DP / 16;                 // MFMA k-steps over the head dimension
  constexpr int QROWS = 4 * QB * 32;

  __shared__ __attribute__((aligned(16))) SdpaSmem<DP> sm;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int l32 = lane & 31;
  const int hi = lane >> 5;

  // XCD-aware order: tiles of one (batch, head) are consecutive, and each XCD
  // gets a contiguous run, so a head's K/V stay in one XCD's L2.
  int bid = blockIdx.x;
  {
    const int per = a.total_blocks / 8;
    if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  }
  const int qt = bid % a.q_tiles;
  const int bh = bid / a.q_tiles;
  const int h = bh % a.Hq;
  const int b = bh / a.Hq;
  const int hk = h / a.group;
  const int64_t Sq = a.Sq, Skv = a.Skv;
  const int D = a.D;

  // ---- Q^T fragments straight from global memory -----------------------
  // B operand of K Q^T: lane holds query column l32, head-dim slots 16*ks + 8*hi + 0..7.
  half8_t qf[QB][KS];
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    int64_t qi = (int64_t)qt * QROWS + (wave * QB + qb) * 32 + l32;
    if (qi >= Sq) qi = Sq - 1;
    int sg = 0;
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++)
      if (i < a.n_qseg && qi >= a.q[i].start) sg = i;
    const uint16_t* qp = a.q[sg].ptr + b * a.q[sg].sb + (qi - a.q[sg].start) * a.q[sg].ss + h * a.q[sg].sh;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const int d0 = ks * 16 + hi * 8;
      uint4_t v = uint4_t{0, 0, 0, 0};
      if (d0 < D) v = *reinterpret_cast<const uint4_t*>(qp + d0);
      qf[qb][ks] = __builtin_bit_cast(half8_t, v);
    }
  }

  // ---- K / V tile loaders ------------------------------------------------
  uint4_t k_reg[K_LOADS];
  uint4_t v_reg[4];
  const bool v_on = tid < V_TASKS;
  const int v_kg = tid / DCH, v_dg = tid % DCH;

  auto kv_row_ptr = [&](const SdpaSeg* segs, int64_t kj) -> const uint16_t* {
    int sg = 0;
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++)
      if (i < a.n_kvseg && kj >= segs[i].start) sg = i;
    return segs[sg].ptr + b * segs[sg].sb + (kj - segs[sg].start) * segs[sg].ss + hk * segs[sg].sh;
  };

  auto issue_kv = [&](int64_t j0) {
#pragma unroll
    for (int i = 0; i < K_LOADS; i++) {
      const int c = tid + i * 256;
      const int row = c / DCH, dc = c % DCH;
      const int64_t kj = j0 + row;
      uint4_t v = uint4_t{0, 0, 0, 0};
      if (kj < Skv && dc * 8 < D) v = *reinterpret_cast<const uint4_t*>(kv_row_ptr(a.k, kj) + dc * 8);
      k_reg[i] = v;
    }
    if (v_on) {
#pragma unroll
      for (int i = 0; i < 4; i++) {
        const int64_t kj = j0 + v_kg * 4 + i;
        uint4_t v = uint4_t{0, 0, 0, 0};  // rows past the end must be zero: 0 * garbage could be NaN
        if (kj < Skv && v_dg * 8 < D) v = *reinterpret_cast<const uint4_t*>(kv_row_ptr(a.v, kj) + v_dg * 8);
        v_reg[i] = v;
      }
    }
  };

  auto stage_kv = [&](int st) {
#pragma unroll
    for (int i = 0; i < K_LOADS; i++) {
      const int c = tid + i * 256;
      const int row = c / DCH, dc = c % DCH;
      *reinterpret_cast<uint4_t*>(&sm.k[st][row * KROW + dc * 8]) = k_reg[i];
    }
    if (v_on) {
      // 4 keys x 8 d in registers -> 8 rows of V^T, 4 keys (8 bytes) each
#pragma unroll
      for (int jj = 0; jj < 4; jj++) {
        // dword jj of each key row holds d = 2*jj, 2*jj + 1
        const uint32_t r0 = v_reg[0][jj], r1 = v_reg[1][jj], r2 = v_reg[2][jj], r3 = v_reg[3][jj];
        const uint32_t lo01 = __builtin_amdgcn_perm(r1, r0, 0x05040100);  // (k0.lo, k1.lo)
        const uint32_t lo23 = __builtin_amdgcn_perm(r3, r2, 0x05040100);
        const uint32_t hi01 = __builtin_amdgcn_perm(r1, r0, 0x07060302);  // (k0.hi, k1.hi)
        const uint32_t hi23 = __builtin_amdgcn_perm(r3, r2, 0x07060302);
        const int d_even = v_dg * 8 + 2 * jj;
        const int d_odd = d_even + 1;
        *reinterpret_cast<uint2_t*>(&sm.vt[st][d_even * BKV + ((v_kg ^ vt_swz(d_even)) << 2)]) = uint2_t{lo01, lo23};
        *reinterpret_cast<uint2_t*>(&sm.vt[st][d_odd * BKV + ((v_kg ^ vt_swz(d_odd)) << 2)]) = uint2_t{hi01, hi23};
      }
    }
  };

  // ---- running state -----------------------------------------------------
  float16_t oacc[QB][DB];
  float m_run[QB], l_run[QB];
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    m_run[qb] = -INFINITY;
    l_run[qb] = 0.f;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int v = 0; v < 16; v++) oacc[qb][db][v] = 0.f;
  }

  const float c = a.scale_log2e;
  const int n_tiles = (int)((Skv + BKV - 1) / BKV);

  issue_kv(0);
  stage_kv(0);
  __syncthreads();

  for (int t = 0; t < n_tiles; t++) {
    const int cur = t & 1;
    const bool more = t + 1 < n_tiles;
    if (more) issue_kv((int64_t)(t + 1) * BKV);

    // ---- S^T = K Q^T ------------------------------------------------------
    float16_t sacc[QB][2];
#pragma unroll
    for (int qb = 0; qb < QB; qb++)
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = 0; v < 16; v++) sacc[qb][kb][v] = 0.f;
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
#pragma unroll
      for (int kb = 0; kb < 2; kb++) {
        const half8_t kf =
            *reinterpret_cast<const half8_t*>(&sm.k[cur][(kb * 32 + l32) * KROW + ks * 16 + hi * 8]);
#pragma unroll
        for (int qb = 0; qb < QB; qb++)
          sacc[qb][kb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf, qf[qb][ks], sacc[qb][kb], 0, 0, 0);
      }
    }

    // ---- online softmax (per query column, statistics in fp32) -----------
    const bool ragged = (int64_t)(t + 1) * BKV > Skv;
    half8_t pf[QB][2][2];
#pragma unroll
    for (int qb = 0; qb < QB; qb++) {
      float mx = -INFINITY;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          float s = sacc[qb][kb][v] * c;
          if (ragged) {
            const int64_t kj = (int64_t)t * BKV + kb * 32 + 8 * (v >> 2) + 4 * hi + (v & 3);
            if (kj >= Skv) s = -INFINITY;
          }
          sacc[qb][kb][v] = s;
          mx = fmaxf(mx, s);
        }
      mx = fmaxf(mx, xor32(mx));
      const float m_new = fmaxf(m_run[qb], mx);
      const float alpha = fast_exp2(m_run[qb] - m_new);  // first tile: exp2(-inf) = 0
      m_run[qb] = m_new;
      float psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          const float p = fast_exp2(sacc[qb][kb][v] - m_new);
          sacc[qb][kb][v] = p;
          psum += p;
        }
      l_run[qb] = l_run[qb] * alpha + psum;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[qb][db][v] *= alpha;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
          for (int e = 0; e < 8; e++) pf[qb][kb][tt][e] = (half_t)sacc[qb][kb][8 * tt + e];
    }

    // ---- O^T += V^T P^T ----------------------------------------------------
    // k-slot e of lane half `hi` in step (kb, tt) is key kb*32 + 16*tt + 8*(e/4) + 4*hi + (e%4)
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int tt = 0; tt < 2; tt++) {
        const int u0 = (kb * 32 + 16 * tt) / 4 + hi;  // unit of keys base + 4*hi .. +3
#pragma unroll
        for (int db = 0; db < DB; db++) {
          const int d = db * 32 + l32;
          const int sw = vt_swz(d);
          const half4_t lo = *reinterpret_cast<const half4_t*>(&sm.vt[cur][d * BKV + ((u0 ^ sw) << 2)]);
          const half4_t hi4 = *reinterpret_cast<const half4_t*>(&sm.vt[cur][d * BKV + (((u0 + 2) ^ sw) << 2)]);
          const half8_t vf = half8_t{lo[0], lo[1], lo[2], lo[3], hi4[0], hi4[1], hi4[2], hi4[3]};
#pragma unroll
          for (int qb = 0; qb < QB; qb++)
            oacc[qb][db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf, pf[qb][kb][tt], oacc[qb][db], 0, 0, 0);
        }
      }

    if (more) stage_kv(cur ^ 1);
    __syncthreads();
  }

  // ---- normalise and store O ----------------------------------------------
#pragma unroll
  for (int qb = 0; qb < QB; qb++) {
    const int64_t qi = (int64_t)qt * QROWS + (wave * QB + qb) * 32 + l32;
    const float l_tot = l_run[qb] + xor32(l_run[qb]);
    const float inv = 1.0f / l_tot;
    if (qi >= Sq) continue;
    uint16_t* op = a.o + b * a.o_sb + qi * a.o_ss + h * a.o_sh;
#pragma unroll
    for (int db = 0; db < DB; db++)
#pragma unroll
      for (int g = 0; g < 4; g++) {
        const int d0 = db * 32 + 8 * g + 4 * hi;
        if (d0 < D) {
          half4_t o4;
#pragma unroll
          for (int e = 0; e < 4; e++) o4[e] = (half_t)(oacc[qb][db][4 * g + e] * inv);
          *reinterpret_cast<half4_t*>(op + d0) = o4;
        }
      }
  }
}

template <int DP, int QB>
static dt_status launch(hipStream_t s, SdpaArgs a) {
  const int qrows = 4 * QB * 32;
  a.q_tiles = (int)((a.Sq + qrows - 1) / qrows);
  int64_t total = (int64_t)a.q_tiles * a.Hq * a.B;
  if (total > 0x7fffffff) return DT_NO_KERNEL;
  a.total_blocks = (int)total;
  hipLaunchKernelGGL((sdpa_kernel<DP, QB>), dim3((unsigned)total), dim3(256), 0, s, a);
  return launch_status();
}

dt_status sdpa_launch(hipStream_t s, const SdpaArgs& a) {
  if (a.B <= 0 || a.Sq <= 0) return DT_OK;
  const bool big = a.Sq >= 2048;
  if (a.D <= 64) return big ? launch<64, 2>(s, a) : launch<64, 1>(s, a);
  return big ? launch<128, 2>(s, a) : launch<128, 1>(s, a);
}

}  // namespace dt

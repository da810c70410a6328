// K3: ScaledDotProductAttention, flash-style, fp16 in / fp32 statistics, gfx950.
//
// One 512-thread workgroup (8 waves, two per SIMD) owns 256 query rows of one
// (batch, head); each wave owns 32 of them.  K/V arrive in tiles of 64 keys,
// transferred from memory straight into LDS, row-major (double-buffered, one
// barrier per tile).
//
// Everything is computed transposed so that the query index is the MFMA
// column (lane & 31) in every stage:
//   S^T = K Q^T          A = K tile rows from LDS, B = Q^T held in registers
//   O^T = V^T P^T        A = V^T, B = P^T = the S^T accumulator itself
// The accumulator of a 32x32 MFMA holds, for column q = lane & 31, rows
// 8*(v/4) + 4*(lane/32) + (v%4), v = 0..15.  Feeding it back as the B operand
// only permutes the summation index, so the V^T operand is fetched with the
// same permutation and P never leaves registers; the softmax row reductions
// are in-lane plus one exchange with lane ^ 32.  V stays row-major in LDS:
// the V^T operand (head dimension along lanes, keys along registers) comes
// from ds_read_b64_tr_b16, which hands lane j of a 16-lane group the element
// column (j % 4) of the rows addressed by lanes (j / 4) + {0, 4, 8, 12}.
#include <atomic>
#include <cstdlib>

#include "dt_common.h"
#include "dt_qkprep.h"
#include "dt_sdpa.h"

namespace dt {

constexpr int BKV = 64;     // keys per tile
constexpr int QWAVES = 8;   // waves per workgroup, 32 query rows each
constexpr int QROWS = QWAVES * 32;

typedef short short4_t __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// LDS layouts (measured bank-conflict free on this part: 64 banks, 16 lanes of
// a 16-byte access or 32 lanes of an 8-byte access per clock).
// K tile: [64 keys][DP] halfs; 16-byte chunk c of key row r is stored at a
// swizzled chunk so that 16 consecutive rows of one chunk column spread over
// all banks.
template <int DP>
__device__ __forceinline__ int k_chunk_swz(int row, int c) {
  if constexpr (DP == 128) return c ^ (row & 15);
  return c ^ ((row >> 1) & 7);
}
// V tile: [64 keys][DP] halfs; the transposing read touches 4 consecutive key
// rows x 64 contiguous bytes per 32 lanes, so 64-byte units are swizzled over
// the row index.
template <int DP>
__device__ __forceinline__ int v_unit_swz(int row, int u) {
  if constexpr (DP == 128) return u ^ (row & 3);
  return u ^ ((row >> 1) & 1);
}

// SPLIT: the (task, key tile) pairs of the whole launch -- a task being the 256 query rows of one (batch, head) --
// are laid end to end and cut into one equal run per workgroup, so that a launch whose task count is no multiple
// of the compute units still keeps all of them busy to the end.  A workgroup walks its run task by task.  A piece
// that covers a whole task is finished as usual.  Any other piece leaves its unnormalised fp32 output, reference
// maximum and row sums in a workspace slot and adds its tile count to the task's counter; the piece that brings the
// counter to the task's tile count -- the last to arrive, whichever that is -- folds all the task's pieces together,
// in the fixed order of their workgroups, and writes the output.  Nobody waits for anybody: there is no spinning
// anywhere, and the result does not depend on which piece arrives last.
template <int DP, bool PREMUL, bool ONESEG, bool SPLIT>
__global__ void __launch_bounds__(512) sdpa_kernel(const SdpaArgs a) {
  constexpr int ROWB = DP * 2;                 // bytes per tile row
  constexpr int DCH = DP / 8;                  // 16-byte chunks per row
  constexpr int TILE_B = BKV * ROWB;           // bytes of one K (or V) tile
  constexpr int LOADS = BKV * DCH / 512;       // 16-byte chunks per thread per tile (2 at DP = 128)
  constexpr int DB = DP / 32;                  // 32-wide blocks of the head dimension
  constexpr int KS = DP / 16;                  // MFMA k-steps over the head dimension
  static_assert(LOADS >= 1, "tile");

  // Two stages each for K and V: a tile is read from one while the next is in
  // flight into the other.
  __shared__ __attribute__((aligned(1024))) unsigned char Ks0[TILE_B];
  __shared__ __attribute__((aligned(1024))) unsigned char Ks1[TILE_B];
  __shared__ __attribute__((aligned(1024))) unsigned char Vs0[TILE_B];
  __shared__ __attribute__((aligned(1024))) unsigned char Vs1[TILE_B];

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
  const int64_t Sq = a.Sq, Skv = a.Skv;
  const int D = a.D;
  const int n_tiles = (int)((Skv + BKV - 1) / BKV);

  // ---- per-thread constants of the K / V tile loaders ---------------------
  // Tiles go from memory straight into LDS.  A wave's transfer instruction
  // fills 1 KB of a tile, lane l landing on its 16-byte slot l; each thread
  // issues LOADS of them per K tile and per V tile and fetches the chunk that
  // the swizzle assigns to its slot.  Lanes whose chunk lies past D stay idle
  // (those slots keep the zeros they were given at the start), and so do, for
  // K, lanes whose row lies past the last key (their scores are masked whatever
  // the slot holds); V rows past the last key are zeroed (see zero_slot).
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  int ld_row[LOADS], k_ch[LOADS], v_ch[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; i++) {
    const int off = (wave * LOADS + i) * 1024 + lane * 16;
    const int row = off / ROWB, pc = (off % ROWB) / 16;
    ld_row[i] = row;
    k_ch[i] = k_chunk_swz<DP>(row, pc);  // the swizzles are involutions
    v_ch[i] = v_unit_swz<DP>(row, pc >> 2) * 4 + (pc & 3);
  }
  // slots that no transfer will ever write must not hold NaN patterns
  if (D < DP || Skv % BKV != 0) {
    for (int i = tid * 16; i < TILE_B; i += 512 * 16) {
      *reinterpret_cast<uint4_t*>(Ks0 + i) = uint4_t{0, 0, 0, 0};
      *reinterpret_cast<uint4_t*>(Ks1 + i) = uint4_t{0, 0, 0, 0};
      *reinterpret_cast<uint4_t*>(Vs0 + i) = uint4_t{0, 0, 0, 0};
      *reinterpret_cast<uint4_t*>(Vs1 + i) = uint4_t{0, 0, 0, 0};
    }
    __syncthreads();
  }

  // ---- per-lane LDS read offsets --------------------------------------------
  // K operand: key row kb*32 + l32, chunk 2*ks + hi
  int k_rd[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ks++) k_rd[ks] = l32 * ROWB + k_chunk_swz<DP>(l32, 2 * ks + hi) * 16;
  // V^T operand through the transposing read: lane i of a 16-lane group addresses
  // key row (i / 4) of a 4-key run and 4 head-dim elements at 4 * (i % 4); the
  // two groups of a half-wave cover head-dim 0..15 and 16..31 of block db.
  const int li = lane & 15, dg = (lane >> 4) & 1;
  int v_rd[DB];
#pragma unroll
  for (int db = 0; db < DB; db++) {
    const int row = 4 * hi + (li >> 2);  // + multiples of 4 per k-step: the swizzle depends on row & 3 (or (row >> 1) & 1) only
    v_rd[db] = row * ROWB + v_unit_swz<DP>(row, db) * 64 + dg * 32 + (li & 3) * 8;
  }
  const float c = PREMUL ? 1.0f : a.scale_log2e;

  // ---- the run of work of this workgroup ----------------------------------
  // Not SPLIT: one task, all of its key tiles.  SPLIT: units [u, u_end) of the launch's (task, key tile) pairs.
  int u = 0, u_end = 0;  // (a split launch holds fewer than 2^31 units)
  if constexpr (SPLIT) {
    u = (int)((int64_t)bid * a.units / a.total_blocks);
    u_end = (int)((int64_t)(bid + 1) * a.units / a.total_blocks);
  }
  [[maybe_unused]] int piece_no = 0;
  [[maybe_unused]] __shared__ int s_last;
  for (;;) {
  int task = bid, t_lo = 0, t_hi = n_tiles;
  if constexpr (SPLIT) {
    if (u >= u_end) break;
    task = u / n_tiles;
    t_lo = u - task * n_tiles;
    t_hi = (u_end - u) < (n_tiles - t_lo) ? t_lo + (u_end - u) : n_tiles;
  }
  const int qt = task % a.q_tiles;
  const int bh = task / a.q_tiles;
  const int h = bh % a.Hq;
  const int b = bh / a.Hq;
  const int hk = h / a.group;

  // ---- Q^T fragments straight from global memory -----------------------
  // B operand of K Q^T: lane holds query column l32, head-dim slots 16*ks + 8*hi + 0..7.
  half8_t qf[KS];
  {
    int64_t qi = (int64_t)qt * QROWS + wave * 32 + l32;
    if (qi >= Sq) qi = Sq - 1;
    int sg = 0;
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++)
      if (i < a.n_qseg && qi >= a.q[i].start) sg = i;
    const uint16_t* qp = a.q[sg].ptr + b * a.q[sg].sb + (qi - a.q[sg].start) * a.q[sg].ss + h * a.q[sg].sh;
    uint4_t qraw[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ks++) {
      const int d0 = ks * 16 + hi * 8;
      qraw[ks] = uint4_t{0, 0, 0, 0};
      if (d0 < D) qraw[ks] = *reinterpret_cast<const uint4_t*>(qp + d0);
    }
    if (a.q_prep) {  // uniform
      // RMSNorm over the head, then the rotation: the row's D elements sit in this lane and in lane ^ 32
      const uint16_t* gam = a.q_gamma[sg];
      const uint16_t* rrow = a.q_rot ? a.q_rot + qi * D : nullptr;
      float inv = 1.f;
      if (gam) {
        float ss = 0.f;
#pragma unroll
        for (int ks = 0; ks < KS; ks++) {
          float x[8];
          unpack_chunk(qraw[ks], x);
#pragma unroll
          for (int e = 0; e < 8; e++) ss += x[e] * x[e];
        }
        ss = sum32(ss);
        inv = 1.0f / sqrtf(ss / (float)D + a.q_eps);
      }
      auto chunk16 = [](const uint16_t* p) __attribute__((always_inline)) {
        if ((reinterpret_cast<uintptr_t>(p) & 15) == 0) return *reinterpret_cast<const uint4_t*>(p);
        uint4_t v;
#pragma unroll
        for (int q = 0; q < 4; q++) v[q] = (uint32_t)p[2 * q] | ((uint32_t)p[2 * q + 1] << 16);
        return v;
      };
#pragma unroll
      for (int ks = 0; ks < KS; ks++) {
        const int d0 = ks * 16 + hi * 8;
        if (d0 < D) {
          float x[8];
          unpack_chunk(qraw[ks], x);
          const uint4_t g = gam ? chunk16(gam + d0) : uint4_t{0, 0, 0, 0};
          const uint4_t r = rrow ? chunk16(rrow + d0) : uint4_t{0, 0, 0, 0};
          qraw[ks] = finish_chunk(x, inv, gam != nullptr, g, rrow != nullptr, r, 1.0f);
        }
      }
    }
#pragma unroll
    for (int ks = 0; ks < KS; ks++) qf[ks] = __builtin_bit_cast(half8_t, qraw[ks]);
  }

  // ---- K / V tile loaders ------------------------------------------------
  // ONESEG: K and V are one run of rows each and small enough for 32-bit byte
  // offsets from a uniform base; a tile step adds a uniform stride.
  // Otherwise the segment of a tile is looked up once per tile (uniformly): a
  // tile that lies inside one segment is fetched from that segment's base with
  // per-lane 32-bit offsets, a tile that straddles segments row by row.
  uint32_t k_off[LOADS], v_off[LOADS];
  const char* k_base = nullptr;
  const char* v_base = nullptr;
  uint32_t k_step = 0, v_step = 0;
  const int64_t keys_ahead = Skv - (int64_t)t_lo * BKV;                     // keys from this piece's first tile on
  int rows_left = (int)(keys_ahead < 0x7fffffff ? keys_ahead : 0x7fffffff);  // ONESEG: keys from the next K tile on
  int rows_left_v = rows_left;
  if constexpr (ONESEG) {
    k_base = reinterpret_cast<const char*>(a.k[0].ptr + b * a.k[0].sb + hk * a.k[0].sh);
    v_base = reinterpret_cast<const char*>(a.v[0].ptr + b * a.v[0].sb + hk * a.v[0].sh);
    k_step = (uint32_t)(a.k[0].ss * BKV * 2);
    v_step = (uint32_t)(a.v[0].ss * BKV * 2);
#pragma unroll
    for (int i = 0; i < LOADS; i++) {
      k_off[i] = (uint32_t)((ld_row[i] * a.k[0].ss + k_ch[i] * 8) * 2) + (uint32_t)t_lo * k_step;
      v_off[i] = (uint32_t)((ld_row[i] * a.v[0].ss + v_ch[i] * 8) * 2) + (uint32_t)t_lo * v_step;
    }
  }
  // General case: a uniform cursor holds the segment the next tile starts in --
  // address of the tile's first row, row stride, last row of the segment --
  // and is re-read from the argument block only when a tile starts past that
  // segment's end.  Tiles inside the segment are fetched with per-lane 32-bit
  // offsets from the cursor; a tile that straddles segments goes row by row.
  struct SegCursor {
    const char* base;  // first row of the next tile (this batch and head)
    int64_t ss;        // row stride, elements
    int64_t end;       // first joint row past the segment
    int64_t row0;      // first joint row of the next tile
  };
  // (an end of 0 makes the first tile look its segment up)
  SegCursor kcur{nullptr, 0, 0, (int64_t)t_lo * BKV}, vcur{nullptr, 0, 0, (int64_t)t_lo * BKV};
  auto seek = [&](const SdpaSeg* segs, SegCursor& c, uint32_t (&off)[LOADS], const int (&chs)[LOADS])
                  __attribute__((always_inline)) {
    int sg = 0;
#pragma unroll
    for (int i = 1; i < kMaxSeg; i++)
      if (i < a.n_kvseg && c.row0 >= segs[i].start) sg = i;
    c.ss = segs[sg].ss;
    c.end = (sg + 1 < a.n_kvseg) ? segs[sg + 1].start : Skv;
    c.base = reinterpret_cast<const char*>(segs[sg].ptr + b * segs[sg].sb + hk * segs[sg].sh +
                                           (c.row0 - segs[sg].start) * c.ss);
#pragma unroll
    for (int i = 0; i < LOADS; i++) off[i] = (uint32_t)((ld_row[i] * c.ss + chs[i] * 8) * 2);
  };
  // (zero_tail: rows of the tile past the last key get zeros instead of keeping an earlier tile's bytes -- for V,
  // whose stale rows would otherwise meet a probability of exactly zero in the second MFMA: 0 x Inf = NaN)
  auto zero_slot = [&](unsigned char* dst, int i) __attribute__((always_inline)) {
    *reinterpret_cast<uint4_t*>(dst + (wave * LOADS + i) * 1024 + lane * 16) = uint4_t{0, 0, 0, 0};
  };
  auto issue_general = [&](const SdpaSeg* segs, SegCursor& c, uint32_t (&off)[LOADS], const int (&chs)[LOADS],
                           unsigned char* dst, bool zero_tail) __attribute__((always_inline)) {
    if (c.row0 < Skv) {
      if (c.row0 >= c.end) seek(segs, c, off, chs);  // uniform
      const int64_t last = c.row0 + BKV < Skv ? c.row0 + BKV : Skv;
      if (zero_tail && last - c.row0 < BKV) {  // uniform: the ragged last tile
#pragma unroll
        for (int i = 0; i < LOADS; i++)
          if (c.row0 + ld_row[i] >= Skv) zero_slot(dst, i);
      }
      if (last <= c.end && c.ss > 0 && c.ss < (1 << 24)) {
        const int n_rows = (int)(last - c.row0);
        const void* base = c.base;
#pragma unroll
        for (int i = 0; i < LOADS; i++)
          if (ld_row[i] < n_rows && chs[i] * 8 < D)
            load_to_lds_16(base, off[i], lds_address(dst) + (uint32_t)((wave_u * LOADS + i) * 1024));
      } else {
#pragma unroll
        for (int i = 0; i < LOADS; i++) {
          const int64_t kj = c.row0 + ld_row[i];
          if (kj < Skv && chs[i] * 8 < D) {
            int sl = 0;
#pragma unroll
            for (int u = 1; u < kMaxSeg; u++)
              if (u < a.n_kvseg && kj >= segs[u].start) sl = u;
            const uint16_t* src =
                segs[sl].ptr + b * segs[sl].sb + (kj - segs[sl].start) * segs[sl].ss + hk * segs[sl].sh + chs[i] * 8;
            load_to_lds_16(src, lds_address(dst) + (uint32_t)((wave_u * LOADS + i) * 1024));
          }
        }
      }
    }
    c.base += c.ss * (BKV * 2);
    c.row0 += BKV;
  };
  // starts the transfer of the next K (or V) tile and moves on by one tile
  auto issue_k = [&](unsigned char* dst) __attribute__((always_inline)) {
    if constexpr (ONESEG) {
#pragma unroll
      for (int i = 0; i < LOADS; i++) {
        if (ld_row[i] < rows_left && k_ch[i] * 8 < D)
          load_to_lds_16(k_base, k_off[i], lds_address(dst) + (uint32_t)((wave_u * LOADS + i) * 1024));
        k_off[i] += k_step;
      }
      rows_left -= BKV;
    } else {
      issue_general(a.k, kcur, k_off, k_ch, dst, false);
    }
  };
  auto issue_v = [&](unsigned char* dst) __attribute__((always_inline)) {
    if constexpr (ONESEG) {
      if (rows_left_v < BKV) {  // uniform: the ragged last tile
#pragma unroll
        for (int i = 0; i < LOADS; i++)
          if (ld_row[i] >= rows_left_v) zero_slot(dst, i);
      }
#pragma unroll
      for (int i = 0; i < LOADS; i++) {
        if (ld_row[i] < rows_left_v && v_ch[i] * 8 < D)
          load_to_lds_16(v_base, v_off[i], lds_address(dst) + (uint32_t)((wave_u * LOADS + i) * 1024));
        v_off[i] += v_step;
      }
      rows_left_v -= BKV;
    } else {
      issue_general(a.v, vcur, v_off, v_ch, dst, true);
    }
  };
  // ---- running state -----------------------------------------------------
  float16_t oacc[DB];
#pragma unroll
  for (int db = 0; db < DB; db++)
#pragma unroll
    for (int v = 0; v < 16; v++) oacc[db][v] = 0.f;
  float m_ref = -INFINITY;  // reference for the exponentials (raw score units); trails the true running maximum
  float l_run = 0.f;        // this lane's share of the row sum

  float16_t sacc[2];   // S^T of the tile in flight (keys x queries)
  half8_t pf[2][2];    // its probabilities, as the B operand of the second MFMA

  // S^T = K Q^T for the K tile in stage st
  auto s_phase = [&](const unsigned char* kt) __attribute__((always_inline)) {
#pragma unroll
    for (int kb = 0; kb < 2; kb++)
#pragma unroll
      for (int v = 0; v < 16; v++) sacc[kb][v] = 0.f;
    // K fragments are read two k-steps (4 reads) ahead of the MFMAs that use them
    half8_t kf[2][4];
    // (a k-step that lies wholly in the zero padding of a short head -- the fourth at D = 40 -- is left out)
    auto live = [&](int ks) __attribute__((always_inline)) { return DP != 64 || ks * 16 < D; };
    auto read_k = [&](int buf, int g) __attribute__((always_inline)) {
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (live(2 * g + (u >> 1)))
          kf[buf][u] = *reinterpret_cast<const half8_t*>(kt + (u & 1) * 32 * ROWB + k_rd[2 * g + (u >> 1)]);
    };
    read_k(0, 0);
#pragma unroll
    for (int g = 0; g < KS / 2; g++) {
      __builtin_amdgcn_sched_barrier(0);
      if (g + 1 < KS / 2) read_k((g + 1) & 1, g + 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int u = 0; u < 4; u++)
        if (live(2 * g + (u >> 1)))
          sacc[u & 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[g & 1][u], qf[2 * g + (u >> 1)], sacc[u & 1], 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // online softmax of tile t (per query column, statistics in fp32): sacc -> pf
  auto softmax_phase = [&](int t) __attribute__((always_inline)) {
    const int rem = (int)(Skv - (int64_t)t * BKV);  // keys left, this tile included
    const bool ragged = rem < BKV;
    if (PREMUL || ragged) {
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = 0; v < 16; v++) {
          float s = sacc[kb][v];
          if (PREMUL) s *= a.scale_log2e;
          if (ragged) {
            const int kj = kb * 32 + 8 * (v >> 2) + 4 * hi + (v & 3);
            if (kj >= rem) s = -INFINITY;
          }
          sacc[kb][v] = s;
        }
    }
    // Probabilities against the current reference, and this lane's share of their row sum.  The tile's maximum is
    // not looked for: as long as every lane's sum stays below 2^10 no probability exceeds that (fp16 holds 2^16),
    // which is all that the reference is there to ensure.
    float psum;
    auto probabilities = [&]() __attribute__((always_inline)) {
      const float mc = m_ref * c;
      psum = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int tt = 0; tt < 2; tt++)
#pragma unroll
          for (int e = 0; e < 8; e++) {
            const float p = fast_exp2(__builtin_fmaf(sacc[kb][8 * tt + e], c, -mc));
            psum += p;
            pf[kb][tt][e] = (half_t)p;
          }
    };
    probabilities();
    // (the first tile arrives here with the reference at -inf: its sums are inf; a NaN fails the test too)
    if (__builtin_amdgcn_ballot_w64(!(psum <= 1024.0f)) != 0) {
      // some row's scores have outgrown the reference: move every row's reference up to its running maximum,
      // rescale what has been accumulated, and redo this tile's probabilities
      float mx = sacc[0][0];
#pragma unroll
      for (int kb = 0; kb < 2; kb++)
#pragma unroll
        for (int v = (kb == 0 ? 1 : 0); v < 16; v++) mx = fmaxf(mx, sacc[kb][v]);
      mx = max32(mx);
      const float m_new = fmaxf(m_ref, mx);
      const float alpha = fast_exp2((m_ref - m_new) * c);  // first tile: exp2(-inf) = 0
      m_ref = m_new;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++) oacc[db][v] *= alpha;
      probabilities();
    }
    l_run += psum;
  };

  // O^T += V^T P^T for the V tile in stage st.
  // k-slot e of lane half `hi` in 16-key step s is key 16*s + 8*(e/4) + 4*hi + (e%4).
  auto pv_phase = [&](const unsigned char* vt) __attribute__((always_inline)) {
    typedef __attribute__((address_space(3))) short4_t lds_s4;
    typedef short short8_t __attribute__((ext_vector_type(8)));
    // V^T fragments of the next 16-key step are read while the current step's MFMAs run
    short4_t vlo[2][DB], vhi[2][DB];
    auto read_v = [&](int buf, int step) __attribute__((always_inline)) {
      const int koff = 16 * step * ROWB;
#pragma unroll
      for (int db = 0; db < DB; db++) {
        vlo[buf][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(vt + koff + v_rd[db]));
        vhi[buf][db] = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(vt + koff + 8 * ROWB + v_rd[db]));
      }
    };
    read_v(0, 0);
#pragma unroll
    for (int step = 0; step < 4; step++) {
      __builtin_amdgcn_sched_barrier(0);
      if (step + 1 < 4) read_v((step + 1) & 1, step + 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int db = 0; db < DB; db++) {
        const short4_t lo = vlo[step & 1][db], h4 = vhi[step & 1][db];
        const short8_t v8 = short8_t{lo[0], lo[1], lo[2], lo[3], h4[0], h4[1], h4[2], h4[3]};
        oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, v8), pf[step >> 1][step & 1], oacc[db], 0, 0, 0);
      }
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- pipeline ---------------------------------------------------------------
  // Interval t (between two barriers) has K tile t and V tile t-1 readable in
  // LDS while K tile t+1 and V tile t are written.  Every wave runs
  //   O += V(t-1) P(t-1) ;  S(t) = K(t) Q ;  P(t) = softmax(S(t))
  // per interval -- two MFMA phases back to back, then one VALU phase.  The two
  // waves of a SIMD (w and w+4) run that cycle half a period apart: the second
  // one starts each interval with the softmax of the scores it produced in the
  // previous interval, so one wave's exponentials overlap the other's MFMAs.
  const bool second = wave >= 4;
  issue_k(Ks0);  // K(0)
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the tile has landed
  __syncthreads();

  // interval t (key tiles t_lo .. t_hi - 1 of the task): K(t) is in k_cur, V(t-1) in v_prev; K(t+1) goes to
  // k_next, V(t) to v_cur
  auto interval = [&](int t, const unsigned char* k_cur, unsigned char* k_next, const unsigned char* v_prev,
                      unsigned char* v_cur) __attribute__((always_inline)) {
    if (t + 1 < t_hi) issue_k(k_next);
    if (t < t_hi) issue_v(v_cur);
    // the wave doing softmax arithmetic gets issue priority: its exponentials only make progress in
    // the gaps the other wave's MFMA stream leaves (measured: +1 %; the opposite assignment -2 %)
    if (!second) {
      __builtin_amdgcn_s_setprio(0);
      if (t > t_lo) pv_phase(v_prev);
      if (t < t_hi) {
        s_phase(k_cur);
        __builtin_amdgcn_s_setprio(2);
        softmax_phase(t);
      }
    } else {
      if (t > t_lo) {
        __builtin_amdgcn_s_setprio(2);
        softmax_phase(t - 1);
        __builtin_amdgcn_s_setprio(0);
        pv_phase(v_prev);
      }
      if (t < t_hi) s_phase(k_cur);
    }
    __builtin_amdgcn_s_waitcnt(0x0f70);
    __syncthreads();
  };
  for (int t = t_lo; t <= t_hi; t += 2) {
    interval(t, Ks0, Ks1, Vs1, Vs0);
    if (t + 1 <= t_hi) interval(t + 1, Ks1, Ks0, Vs0, Vs1);
  }
  __builtin_amdgcn_s_setprio(0);

  // ---- normalise and store O ----------------------------------------------
  // O^T block db: lane holds query column l32 and head-dim 8*g + 4*hi + (0..3);
  // swapping the odd groups of the low half-wave with the even groups of the
  // high half-wave leaves every lane with runs of 8 consecutive head-dim
  // elements (16-byte stores).
  auto store_output = [&]() __attribute__((always_inline)) {
    const int64_t qi = (int64_t)qt * QROWS + wave * 32 + l32;
    const float l_tot = sum32(l_run);
    const float inv = 1.0f / l_tot;
    uint16_t* op = a.o + b * a.o_sb + (qi < Sq ? qi : 0) * a.o_ss + h * a.o_sh;
    const bool vec_ok = ((a.o_sb | a.o_ss | a.o_sh) & 7) == 0 && (reinterpret_cast<uintptr_t>(a.o) & 15) == 0;
#pragma unroll
    for (int db = 0; db < DB; db++) {
      uint32_t pk[4][2];
#pragma unroll
      for (int g = 0; g < 4; g++) {
        pk[g][0] = (uint32_t)half_to_bits((half_t)(oacc[db][4 * g] * inv)) |
                   ((uint32_t)half_to_bits((half_t)(oacc[db][4 * g + 1] * inv)) << 16);
        pk[g][1] = (uint32_t)half_to_bits((half_t)(oacc[db][4 * g + 2] * inv)) |
                   ((uint32_t)half_to_bits((half_t)(oacc[db][4 * g + 3] * inv)) << 16);
      }
#pragma unroll
      for (int gp = 0; gp < 2; gp++) {
        uint32_t run[4];
#pragma unroll
        for (int e = 0; e < 2; e++) {
          auto r = __builtin_amdgcn_permlane32_swap(pk[2 * gp][e], pk[2 * gp + 1][e], false, false);
          run[e] = r[0];
          run[2 + e] = r[1];
        }
        const int d0 = db * 32 + 16 * gp + 8 * hi;
        if (qi < Sq && d0 < D) {
          if (vec_ok) {
            *reinterpret_cast<uint4_t*>(op + d0) = uint4_t{run[0], run[1], run[2], run[3]};
          } else {
            *reinterpret_cast<uint2_t*>(op + d0) = uint2_t{run[0], run[1]};
            *reinterpret_cast<uint2_t*>(op + d0 + 4) = uint2_t{run[2], run[3]};
          }
        }
      }
    }
  };

  if constexpr (!SPLIT) {
    store_output();
    break;
  } else {
    if (t_lo == 0 && t_hi == n_tiles) {
      store_output();  // the piece is the whole task
    } else {
      // ---- a piece of a task: leave it for, or fold in, the task's other pieces ----------------------------
      // Slot layout (floats): [DB * 16 accumulators][512 threads], then [512] reference maxima, then [512]
      // row-sum shares: a wave's access covers 256 consecutive bytes.  A workgroup owns two slots: its first piece
      // goes to the even one, a later piece -- which can only be its last -- to the odd one.
      // The pieces of a task run on any compute units of the device, whose L2 caches (one per die) do not see each
      // other's ordinary stores.  Partial results are therefore written and read with device-scope accesses
      // (relaxed atomics: write-through stores, loads that do not trust a die's cached copy) instead of
      // bracketing ordinary accesses with cache-wide write-backs and invalidations, which cost far more than the
      // 130 KB they would protect.
      constexpr int SLOT_F = sdpa_split_slot_floats(DP);
      const int P = a.total_blocks;
      float* slot = a.partials + (size_t)(2 * bid + (piece_no > 0 ? 1 : 0)) * SLOT_F;
#pragma unroll
      for (int db = 0; db < DB; db++)
#pragma unroll
        for (int v = 0; v < 16; v++)
          __hip_atomic_store(slot + (db * 16 + v) * 512 + tid, oacc[db][v], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(slot + DB * 16 * 512 + tid, m_ref, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      __hip_atomic_store(slot + DB * 16 * 512 + 512 + tid, l_run, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      // every wave's stores have been acknowledged before the barrier, hence before the one thread's count that
      // publishes the piece
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
      __syncthreads();
      if (tid == 0) {
        const int done = t_hi - t_lo;
        const int before = __hip_atomic_fetch_add(a.counters + task, done, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        s_last = (before + done == n_tiles) ? 1 : 0;
      }
      __syncthreads();
      if (s_last != 0) {  // uniform: every other piece of the task has been published
        const int64_t ua = (int64_t)task * n_tiles, ub = ua + n_tiles;
        // the workgroup whose run holds unit x is the largest p with p * units < (x + 1) * P
        const int p_lo = (int)(((ua + 1) * P - 1) / a.units), p_hi = (int)((ub * P - 1) / a.units);
        // The pieces are folded in the order of their workgroups, this one's own included (re-read from its slot),
        // whichever of them happens to be the one doing it: the result does not depend on the order of arrival.
        for (int p = p_lo; p <= p_hi; p++) {
          const int64_t first_unit = (int64_t)p * a.units / P;
          const float* other = a.partials + (size_t)(2 * p + (first_unit < ua ? 1 : 0)) * SLOT_F;
          auto ld = [&](int i) __attribute__((always_inline)) {
            return __hip_atomic_load(other + i * 512 + tid, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
          };
          // all of the slot's loads go out before the first of them is waited for
          const float m_o = ld(DB * 16), l_o = ld(DB * 16 + 1);
          float16_t got[DB];
#pragma unroll
          for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) got[db][v] = ld(db * 16 + v);
          __builtin_amdgcn_sched_barrier(0);
          if (p == p_lo) {
            m_ref = m_o;
            l_run = l_o;
#pragma unroll
            for (int db = 0; db < DB; db++) oacc[db] = got[db];
            continue;
          }
          const float m_new = fmaxf(m_ref, m_o);
          const float wa = fast_exp2((m_ref - m_new) * c), wb = fast_exp2((m_o - m_new) * c);
          m_ref = m_new;
          l_run = l_run * wa + l_o * wb;
#pragma unroll
          for (int db = 0; db < DB; db++)
#pragma unroll
            for (int v = 0; v < 16; v++) oacc[db][v] = oacc[db][v] * wa + got[db][v] * wb;
        }
        store_output();
      }
    }
    u += t_hi - t_lo;
    piece_no++;
  }
  }  // the workgroup's run
}

// Zeroes the per-task tile counters of a SPLIT launch (a fill kernel, so that the launch can be captured in a graph).
__global__ void sdpa_zero_counters_kernel(int32_t* counters, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) counters[i] = 0;
}

// Compute units of the calling thread's current device (cached per ordinal; 256 if the runtime cannot say).
static int compute_units() {
  static std::atomic<int> cached[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) {
    (void)hipGetLastError();
    return 256;
  }
  if (dev < 0 || dev >= 64) return 256;
  int n = cached[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) {
      (void)hipGetLastError();
      n = 256;
    }
    cached[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

bool sdpa_split_plan(int32_t B, int32_t Hq, int32_t D, int64_t Sq, int64_t Skv, SdpaSplit* plan) {
  if (B <= 0 || Hq <= 0 || D <= 0 || Sq <= 0 || Skv <= 0) return false;
  // DT_SDPA_KEY_SPLIT = "never" | "always" (whenever the launch can be cut at all; for tests and measurements);
  // anything else, or unset: decide by the estimate below.  Read at every call.
  const char* knob = getenv("DT_SDPA_KEY_SPLIT");
  const bool never = knob && knob[0] == 'n', always = knob && knob[0] == 'a';
  if (never) return false;
  const int64_t tasks = (int64_t)B * Hq * ((Sq + QROWS - 1) / QROWS);
  const int64_t n_tiles = (Skv + BKV - 1) / BKV;
  const int64_t units = tasks * n_tiles;
  if (tasks > (1 << 20) || units >= (1LL << 31)) return false;  // (the kernel counts units in 32 bits)
  const int cus = compute_units();
  // at most 8 pieces per task (the piece that arrives last folds the others in one after the other), at least
  // `min_tiles` key tiles per workgroup
  const int64_t min_tiles = always ? 2 : 8;
  int64_t wgs = cus;
  if (wgs > tasks * 8) wgs = tasks * 8;
  if (wgs > units / min_tiles) wgs = units / min_tiles;
  if (wgs < 2 || n_tiles < 2) return false;
  if (!always) {
    // Measured on this part (head size 128): the card delivers about the same attention throughput whether all of
    // its compute units are busy or only 70-85 % of them -- a compute unit runs a key tile in ~1.4 us when a third
    // of the card idles and in ~1.9 us when none does -- so a launch of 1.69 or 6.19 rounds of workgroups gains
    // nothing from being cut into equal runs (0.276 against 0.248 ms at 24 heads x 4608 tokens).  What does gain
    // is a launch that fills well under one round: there the unsplit time is one task at the fast rate, the split
    // time the mean load at the slow rate plus ~25 us of fixed cost per workgroup (counter reset, pipeline refill,
    // partial results out and in).
    const double rounds = (double)tasks / cus;
    if (rounds >= 1.0) return false;
    const double fixed = 25.0 / (1.9 * (double)n_tiles);  // in task times
    if (1.0 / 1.35 <= rounds * (double)cus / (double)wgs + fixed) return false;
  }
  if (plan) {
    plan->workgroups = (int32_t)wgs;
    plan->tasks = (int32_t)tasks;
    plan->units = units;
    plan->counter_bytes = ((size_t)tasks * 4 + 255) & ~(size_t)255;
    plan->partial_bytes = (size_t)2 * wgs * sdpa_split_slot_floats(D <= 64 ? 64 : 128) * 4;
  }
  return true;
}

template <int DP>
static dt_status launch(hipStream_t s, SdpaArgs a) {
  a.q_tiles = (int)((a.Sq + QROWS - 1) / QROWS);
  int64_t total = (int64_t)a.q_tiles * a.Hq * a.B;
  if (total > 0x7fffffff) return DT_NO_KERNEL;
  a.total_blocks = (int)total;
  const bool premul = !(a.scale_log2e > 0.f && a.scale_log2e < 1e30f);
  // one K and one V segment whose rows lie within 2 GiB of the head's first row: 32-bit offsets
  const bool oneseg = a.n_kvseg == 1 && a.k[0].ss > 0 && a.v[0].ss > 0 && a.Skv < (1 << 30) &&
                      (a.Skv + 2 * BKV) * a.k[0].ss * 2 < 0x7fffffffLL && (a.Skv + 2 * BKV) * a.v[0].ss * 2 < 0x7fffffffLL;
  dim3 block(512);
  if (a.partials) {
    // key-split launch: the counters start at zero, then one workgroup per equal run of units
    hipLaunchKernelGGL(sdpa_zero_counters_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, a.counters,
                       (int)total);
    if (const dt_status st = launch_status(); st != DT_OK) return st;
    a.total_blocks = a.split_workgroups;
    dim3 grid((unsigned)a.split_workgroups);
    if (oneseg) {
      if (premul) hipLaunchKernelGGL((sdpa_kernel<DP, true, true, true>), grid, block, 0, s, a);
      else hipLaunchKernelGGL((sdpa_kernel<DP, false, true, true>), grid, block, 0, s, a);
    } else {
      if (premul) hipLaunchKernelGGL((sdpa_kernel<DP, true, false, true>), grid, block, 0, s, a);
      else hipLaunchKernelGGL((sdpa_kernel<DP, false, false, true>), grid, block, 0, s, a);
    }
    return launch_status();
  }
  dim3 grid((unsigned)total);
  if (oneseg) {
    if (premul) hipLaunchKernelGGL((sdpa_kernel<DP, true, true, false>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((sdpa_kernel<DP, false, true, false>), grid, block, 0, s, a);
  } else {
    if (premul) hipLaunchKernelGGL((sdpa_kernel<DP, true, false, false>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((sdpa_kernel<DP, false, false, false>), grid, block, 0, s, a);
  }
  return launch_status();
}

dt_status sdpa_launch(hipStream_t s, const SdpaArgs& a) {
  if (a.B <= 0 || a.Sq <= 0) return DT_OK;
  if (a.D <= 64) return launch<64>(s, a);
  return launch<128>(s, a);
}

}  // namespace dt

// K1: Dense over palettized weights, Y = X W^T (+ bias), for gfx950.
//
// The packed weight never exists dequantized in memory: per K-tile each thread
// pulls one 32-index granule (Q dwords) of a weight row into registers,
// unpacks it with constant shifts, looks the fp16 values up in the palettes
// held in LDS, and writes the fp16 row slice into the LDS B tile that
// v_mfma_f32_32x32x16_f16 then consumes.  fp32 accumulation, one rounding.
//
// Tile: BM x BN outputs per 256-thread workgroup (4 waves as 2 x 2), BK = 32.
// LDS is double-buffered; the global loads of tile t+1 are issued before the
// MFMAs of tile t and its unpack/lookup runs after them, so one barrier per
// K-tile and the unpack VALU/LDS work overlaps the matrix pipe.
#include "dt_common.h"
#include "dt_layout.h"

namespace dt {

constexpr int kMaxWeights = 4;
constexpr int BK = 32;
constexpr int LDS_ROW = BK + 8;  // halfs; 80-byte rows keep 16-byte LDS accesses of 8 consecutive rows on distinct banks
constexpr int kPalLdsBytes = 32768;

enum PalMode : int {
  kPalShared = 0,  // palettes of every block the tile's rows touch, loaded once, slot = block - first block
  kPalRow = 1,     // nib < K, K % nib == 0: one palette per row, reloaded every nib columns
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
};

struct DenseArgs {
  const uint16_t* x;
  int64_t ldx;
  int32_t m, k;
  int32_t nib;
  int32_t n_weights;
  int32_t tiles_m, tiles_n;
  DenseWeight w[kMaxWeights];
};

__device__ __forceinline__ uint4_t ld_global_16(const void* p) {
  return *reinterpret_cast<const uint4_t*>(p);
}

template <int Q, int BM, int BN, int MODE>
__global__ void __launch_bounds__(256) dense_qx_kernel(const DenseArgs a) {
  constexpr int WM = BM / 2, WN = BN / 2;  // per-wave output tile
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int A_CHUNKS = BM * (BK / 8) / 256;  // 16-byte chunks of X per thread per K-tile
  constexpr int B_GRAN = BN / 256 > 0 ? BN / 256 : 1;  // 32-index granules per thread per K-tile
  constexpr int B_CHUNKS = BN * (BK / 8) / 256;        // plain fp16 weight: 16-byte chunks per thread
  constexpr int QW = MODE == kPlainF16 ? 1 : Q;        // dwords per granule
  static_assert(BM % 64 == 0 && BN % 64 == 0, "tile");

  __shared__ __attribute__((aligned(16))) half_t As[2][BM * LDS_ROW];
  __shared__ __attribute__((aligned(16))) half_t Bs[2][BN * LDS_ROW];
  __shared__ __attribute__((aligned(16))) uint16_t Pal[(MODE == kPalShared || MODE == kPalRow) ? kPalLdsBytes / 2 : 8];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;

  // Workgroups are dealt round-robin to the 8 XCDs; give each XCD a contiguous
  // run of tiles so the weight tiles it re-reads stay in that XCD's L2.
  const int total = a.tiles_m * a.tiles_n;
  int bid = blockIdx.x;
  {
    const int per = total / 8;
    if (bid < per * 8) bid = (bid & 7) * per + (bid >> 3);
  }
  const int tn = bid / a.tiles_m;
  const int tm = bid - tn * a.tiles_m;

  int wi = 0;
#pragma unroll
  for (int i = 1; i < kMaxWeights; i++)
    if (i < a.n_weights && tn >= a.w[i].tile_begin) wi = i;
  const DenseWeight w = a.w[wi];
  const int n0 = (tn - w.tile_begin) * BN;
  const int m0 = tm * BM;
  const int K = a.k;
  const QxLayout lay = make_layout(Q, a.nib);

  // ---- per-thread load coordinates -------------------------------------
  const uint16_t* a_src[A_CHUNKS];
  int a_dst[A_CHUNKS];
#pragma unroll
  for (int i = 0; i < A_CHUNKS; i++) {
    int c = tid + i * 256;
    int row = c >> 2, kc = c & 3;
    int gm = m0 + row;
    if (gm >= a.m) gm = a.m - 1;
    a_src[i] = a.x + (int64_t)gm * a.ldx + kc * 8;
    a_dst[i] = row * LDS_ROW + kc * 8;
  }
  // weight rows handled by this thread (palettized: one granule per row per K-tile)
  int b_row[B_GRAN];
  int64_t b_flat[B_GRAN];  // flat element index of (row, k = 0)
#pragma unroll
  for (int g = 0; g < B_GRAN; g++) {
    int row = tid + g * 256;
    b_row[g] = row;
    int gn = n0 + row;
    if (gn >= w.n) gn = w.n - 1;
    b_flat[g] = (int64_t)gn * K;
  }
  const bool b_active = (BN >= 256) || (tid < BN);
  // plain fp16 weight: same chunking as X
  const uint16_t* bf_src[B_CHUNKS];
  int bf_dst[B_CHUNKS];
  if constexpr (MODE == kPlainF16) {
#pragma unroll
    for (int i = 0; i < B_CHUNKS; i++) {
      int c = tid + i * 256;
      int row = c >> 2, kc = c & 3;
      int gn = n0 + row;
      if (gn >= w.n) gn = w.n - 1;
      bf_src[i] = reinterpret_cast<const uint16_t*>(w.data) + (int64_t)gn * K + kc * 8;
      bf_dst[i] = row * LDS_ROW + kc * 8;
    }
  }

  // ---- palettes -> LDS --------------------------------------------------
  int64_t pal_first_block = 0;
  if constexpr (MODE == kPalShared) {
    int last_row = n0 + BN - 1;
    if (last_row >= w.n) last_row = w.n - 1;
    pal_first_block = ((int64_t)n0 * K) / a.nib;
    int64_t last_block = ((int64_t)last_row * K + (K - 1)) / a.nib;
    int n_pal = (int)(last_block - pal_first_block + 1);
    const int per_pal = 1 << (Q - 1);  // dwords per palette
    for (int i = tid; i < n_pal * per_pal; i += 256) {
      int p = i / per_pal, e = i - p * per_pal;
      const uint32_t* src =
          reinterpret_cast<const uint32_t*>(w.data + palette_offset(lay, pal_first_block + p));
      reinterpret_cast<uint32_t*>(Pal)[i] = src[e];
    }
  }
  auto load_row_palettes = [&](int k0) {
    // kPalRow: block of row n at column k0 is n * (K / nib) + k0 / nib
    const int per_pal = 1 << (Q - 1);
    const int bpr = K / a.nib;
    for (int i = tid; i < BN * per_pal; i += 256) {
      int row = i / per_pal, e = i - row * per_pal;
      int gn = n0 + row;
      if (gn >= w.n) gn = w.n - 1;
      int64_t blk = (int64_t)gn * bpr + k0 / a.nib;
      const uint32_t* src = reinterpret_cast<const uint32_t*>(w.data + palette_offset(lay, blk));
      reinterpret_cast<uint32_t*>(Pal)[i] = src[e];
    }
  };
  if constexpr (MODE == kPalRow) load_row_palettes(0);

  // ---- register staging -------------------------------------------------
  uint4_t a_reg[A_CHUNKS];
  uint32_t b_raw[B_GRAN][QW];
  uint4_t bf_reg[B_CHUNKS];

  auto issue_loads = [&](int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) a_reg[i] = ld_global_16(a_src[i] + k0);
    if constexpr (MODE == kPlainF16) {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; i++) bf_reg[i] = ld_global_16(bf_src[i] + k0);
    } else {
      if (b_active) {
#pragma unroll
        for (int g = 0; g < B_GRAN; g++) {
          int64_t e = b_flat[g] + k0;
          int64_t blk = e / a.nib;
          int64_t r = e - blk * a.nib;
          const uint32_t* src = reinterpret_cast<const uint32_t*>(w.data + index_byte_offset(lay, blk, r));
#pragma unroll
          for (int i = 0; i < QW; i++) b_raw[g][i] = src[i];
        }
      }
    }
  };

  auto stage_to_lds = [&](int stage, int k0) {
#pragma unroll
    for (int i = 0; i < A_CHUNKS; i++) *reinterpret_cast<uint4_t*>(&As[stage][a_dst[i]]) = a_reg[i];
    if constexpr (MODE == kPlainF16) {
#pragma unroll
      for (int i = 0; i < B_CHUNKS; i++) *reinterpret_cast<uint4_t*>(&Bs[stage][bf_dst[i]]) = bf_reg[i];
    } else {
      if (b_active) {
#pragma unroll
        for (int g = 0; g < B_GRAN; g++) {
          uint32_t idx[32];
          unpack32<Q>(b_raw[g], idx);
          uint32_t o[16];
          if constexpr (MODE == kPalGlobal) {
            int64_t blk = (b_flat[g] + k0) / a.nib;
            const uint16_t* pal = reinterpret_cast<const uint16_t*>(w.data + palette_offset(lay, blk));
#pragma unroll
            for (int j = 0; j < 16; j++)
              o[j] = (uint32_t)pal[idx[2 * j]] | ((uint32_t)pal[idx[2 * j + 1]] << 16);
          } else {
            int slot;
            if constexpr (MODE == kPalShared)
              slot = (int)((b_flat[g] + k0) / a.nib - pal_first_block);
            else
              slot = b_row[g];
            const uint16_t* pal = Pal + (slot << Q);
#pragma unroll
            for (int j = 0; j < 16; j++)
              o[j] = (uint32_t)pal[idx[2 * j]] | ((uint32_t)pal[idx[2 * j + 1]] << 16);
          }
          uint4_t* dst = reinterpret_cast<uint4_t*>(&Bs[stage][b_row[g] * LDS_ROW]);
#pragma unroll
          for (int j = 0; j < 4; j++) dst[j] = uint4_t{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
        }
      }
    }
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; i++)
#pragma unroll
    for (int j = 0; j < TN; j++)
#pragma unroll
      for (int v = 0; v < 16; v++) acc[i][j][v] = 0.f;

  const int nk = K / BK;
  issue_loads(0);
  __syncthreads();  // palettes visible
  stage_to_lds(0, 0);
  __syncthreads();

  const int frag_row = lane & 31;
  const int frag_k = (lane >> 5) * 8;

  for (int kt = 0; kt < nk; kt++) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) issue_loads((kt + 1) * BK);

    const half_t* Ab = &As[cur][(wm * WM + frag_row) * LDS_ROW + frag_k];
    const half_t* Bb = &Bs[cur][(wn * WN + frag_row) * LDS_ROW + frag_k];
#pragma unroll
    for (int ks = 0; ks < BK / 16; ks++) {
      half8_t af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; i++) af[i] = *reinterpret_cast<const half8_t*>(Ab + i * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int j = 0; j < TN; j++) bf[j] = *reinterpret_cast<const half8_t*>(Bb + j * 32 * LDS_ROW + ks * 16);
#pragma unroll
      for (int i = 0; i < TM; i++)
#pragma unroll
        for (int j = 0; j < TN; j++)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    }

    if (more) {
      const int k1 = (kt + 1) * BK;
      if constexpr (MODE == kPalRow) {
        if (k1 % a.nib == 0) {
          // every lookup of the previous K-tile finished before the last barrier
          load_row_palettes(k1);
          __syncthreads();
        }
      }
      stage_to_lds(cur ^ 1, k1);
    }
    __syncthreads();
  }

  // ---- epilogue: bias, round once to fp16, store ------------------------
  // accumulator layout of v_mfma_f32_32x32x16: lane holds column (lane & 31),
  // rows 8 * (v / 4) + 4 * (lane / 32) + (v % 4).
#pragma unroll
  for (int j = 0; j < TN; j++) {
    const int gn = n0 + wn * WN + j * 32 + (lane & 31);
    if (gn >= w.n) continue;
    float bv = 0.f;
    if (w.bias) bv = (float)bits_to_half(w.bias[gn]);
#pragma unroll
    for (int i = 0; i < TM; i++) {
#pragma unroll
      for (int v = 0; v < 16; v++) {
        const int gm = m0 + wm * WM + i * 32 + 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
        if (gm < a.m) w.y[(int64_t)gm * w.ldy + gn] = half_to_bits((half_t)(acc[i][j][v] + bv));
      }
    }
  }
}

// Any shape / alignment: one thread per output element.  Slow; keeps odd
// shapes (K not a multiple of 32, nib not a multiple of 32, unaligned rows)
// correct rather than unsupported.
__global__ void __launch_bounds__(256) dense_qx_generic_kernel(const uint16_t* __restrict__ x, int64_t ldx, int64_t m,
                                                             int64_t n, int64_t k, const uint8_t* __restrict__ wdata,
                                                             int qbits, int nib, const uint16_t* __restrict__ bias,
                                                             uint16_t* __restrict__ y, int64_t ldy) {
  int64_t o = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (o >= m * n) return;
  int64_t mi = o / n, ni = o - mi * n;
  const uint16_t* xr = x + mi * ldx;
  float acc = 0.f;
  if (qbits == 16) {
    const uint16_t* wr = reinterpret_cast<const uint16_t*>(wdata) + ni * k;
    for (int64_t kk = 0; kk < k; kk++) acc += (float)bits_to_half(xr[kk]) * (float)bits_to_half(wr[kk]);
  } else {
    const QxLayout l = make_layout(qbits, nib);
    for (int64_t kk = 0; kk < k; kk++) {
      int64_t e = ni * k + kk;
      int64_t b = e / nib, r = e - b * nib;
      const uint8_t* base = wdata + palette_offset(l, b);
      const uint16_t* pal = reinterpret_cast<const uint16_t*>(base);
      uint16_t wv = pal[load_index(base + l.pal_bytes, r, qbits)];
      acc += (float)bits_to_half(xr[kk]) * (float)bits_to_half(wv);
    }
  }
  if (bias) acc += (float)bits_to_half(bias[ni]);
  y[mi * ldy + ni] = half_to_bits((half_t)acc);
}

template <int Q, int BM, int BN>
static dt_status launch_tiled(hipStream_t s, const DenseArgs& a, int mode) {
  dim3 grid((unsigned)(a.tiles_m * a.tiles_n)), block(256);
  switch (mode) {
    case kPalShared: hipLaunchKernelGGL((dense_qx_kernel<Q, BM, BN, kPalShared>), grid, block, 0, s, a); break;
    case kPalRow:
      if constexpr ((BN << (Q + 1)) <= kPalLdsBytes) {
        hipLaunchKernelGGL((dense_qx_kernel<Q, BM, BN, kPalRow>), grid, block, 0, s, a);
        break;
      } else {
        return DT_NO_KERNEL;  // choose_pal_mode never picks per-row palettes that do not fit
      }
    default: hipLaunchKernelGGL((dense_qx_kernel<Q, BM, BN, kPalGlobal>), grid, block, 0, s, a); break;
  }
  return launch_status();
}

template <int BM, int BN>
static dt_status launch_tiled_q(hipStream_t s, const DenseArgs& a, int qbits, int mode) {
  switch (qbits) {
    case 4: return launch_tiled<4, BM, BN>(s, a, mode);
    case 5: return launch_tiled<5, BM, BN>(s, a, mode);
    case 6: return launch_tiled<6, BM, BN>(s, a, mode);
    case 7: return launch_tiled<7, BM, BN>(s, a, mode);
    case 8: return launch_tiled<8, BM, BN>(s, a, mode);
    case 16: {
      dim3 grid((unsigned)(a.tiles_m * a.tiles_n)), block(256);
      hipLaunchKernelGGL((dense_qx_kernel<8, BM, BN, kPlainF16>), grid, block, 0, s, a);
      return launch_status();
    }
  }
  return DT_INVALID;
}

// Palette placement for a BN-row tile (see PalMode).
static int choose_pal_mode(int qbits, int nib, int64_t K, int BN) {
  if (qbits == 16) return kPlainF16;
  const int64_t pal_bytes = (int64_t)2 << qbits;
  const int64_t shared_count = ((int64_t)BN * K) / nib + 2;
  if (shared_count * pal_bytes <= kPalLdsBytes) return kPalShared;
  if (nib < K && K % nib == 0 && (int64_t)BN * pal_bytes <= kPalLdsBytes) return kPalRow;
  return kPalGlobal;
}

}  // namespace dt

DT_EXPORT dt_status dt_dense_qx_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                    const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                                    uint16_t* const* Y, const int64_t* ldy, uint32_t flags) {
  using namespace dt;
  (void)flags;
  if (M < 0 || K <= 0 || n_weights <= 0 || !W || !Y || !ldy) return DT_INVALID;
  if (M > 0x7fffffff || K > 0x7fffffff) return DT_INVALID;
  for (int i = 0; i < n_weights; i++) {
    const dt_qx_weight& w = W[i];
    if (!w.data || w.count < 0 || w.count % K != 0) return DT_INVALID;
    if (w.qbits != 16 && (w.qbits < 4 || w.qbits > 8 || w.nib <= 0)) return DT_INVALID;
    if (w.count / K > 0x7fffffff) return DT_INVALID;
    if (M > 0 && (!Y[i] || ldy[i] < w.count / K)) return DT_INVALID;
  }
  if (M == 0) return DT_OK;
  if (!X || ldx < K) return DT_INVALID;
  if (!device_ok()) return DT_NO_KERNEL;
  hipStream_t s = as_stream(stream);

  // Weights that share (qbits, nib) and meet the tiled kernel's alignment go
  // out in groups of up to kMaxWeights per launch; the rest take the generic kernel.
  const bool x_ok = (K % BK == 0) && (ldx % 8 == 0) && ((reinterpret_cast<uintptr_t>(X) & 15) == 0);
  int i = 0;
  while (i < n_weights) {
    const dt_qx_weight& w0 = W[i];
    const int64_t n_rows0 = w0.count / K;
    bool tiled = x_ok && n_rows0 > 0 && (reinterpret_cast<uintptr_t>(w0.data) & 15) == 0 &&
                 (w0.qbits == 16 || w0.nib % 32 == 0);
    if (!tiled) {
      if (n_rows0 > 0) {
        int64_t outs = M * n_rows0;
        if ((outs + 255) / 256 > 0x7fffffff) return DT_NO_KERNEL;
        hipLaunchKernelGGL(dense_qx_generic_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, s, X, ldx, M,
                           n_rows0, K, static_cast<const uint8_t*>(w0.data), w0.qbits, w0.nib,
                           bias ? bias[i] : nullptr, Y[i], ldy[i]);
        dt_status st = launch_status();
        if (st != DT_OK) return st;
      }
      i++;
      continue;
    }
    // tile shape: big tiles when there is enough work to fill 256 CUs with them
    const bool big = (M >= 1024) && (n_rows0 >= 256);
    const int BM = big ? 256 : 128, BN = big ? 256 : 128;
    DenseArgs a;
    a.x = X;
    a.ldx = ldx;
    a.m = (int32_t)M;
    a.k = (int32_t)K;
    a.nib = w0.qbits == 16 ? 32 : w0.nib;
    a.tiles_m = (int)((M + BM - 1) / BM);
    int tiles_n = 0, cnt = 0;
    while (i < n_weights && cnt < kMaxWeights) {
      const dt_qx_weight& w = W[i];
      const int64_t n_rows = w.count / K;
      if (w.qbits != w0.qbits || (w.qbits != 16 && w.nib != w0.nib) || n_rows <= 0 ||
          (reinterpret_cast<uintptr_t>(w.data) & 15) != 0)
        break;
      a.w[cnt].data = static_cast<const uint8_t*>(w.data);
      a.w[cnt].bias = bias ? bias[i] : nullptr;
      a.w[cnt].y = Y[i];
      a.w[cnt].ldy = ldy[i];
      a.w[cnt].n = (int32_t)n_rows;
      a.w[cnt].tile_begin = tiles_n;
      tiles_n += (int)((n_rows + BN - 1) / BN);
      cnt++;
      i++;
    }
    for (int j = cnt; j < kMaxWeights; j++) a.w[j] = a.w[0];
    a.n_weights = cnt;
    a.tiles_n = tiles_n;
    if ((int64_t)a.tiles_m * tiles_n > 0x7fffffff) return DT_NO_KERNEL;
    const int mode = choose_pal_mode(w0.qbits, a.nib, K, BN);
    dt_status st = big ? launch_tiled_q<256, 256>(s, a, w0.qbits, mode) : launch_tiled_q<128, 128>(s, a, w0.qbits, mode);
    if (st != DT_OK) return st;
  }
  return DT_OK;
}

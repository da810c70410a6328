// K1: Dense over palettized weights, Y = X W^T (+ bias), for gfx950.
//
// The packed weight never exists dequantized in memory: per K-tile two threads
// per weight row each pull half of a 32-index granule into registers, unpack
// it, look the fp16 values up in palettes held in LDS, and write the fp16 row
// slice into an LDS ring that v_mfma_f32_32x32x16_f16 then consumes; X (and a
// plain fp16 weight) goes from memory straight into LDS.  fp32 accumulation,
// one rounding to fp16, optional fused tails (per-head RMSNorm + RoPE, or
// activation / gate / fp32 residual).
//
// Tile: BM x BN outputs per 512-thread workgroup (8 waves, two per SIMD, each
// a BN/2 x BM/4 slice), K-tiles of 32 processed in pairs; one barrier per K-tile
// (per pair with plain fp16 weights, which no wave writes to LDS itself).
#include "dt_dense_launch.h"

namespace dt {

// Any shape / alignment: one thread per output element.  Slow; keeps odd
// shapes (K not a multiple of 32, nib not a multiple of 32, unaligned rows)
// correct rather than unsupported.
__global__ void __launch_bounds__(256) dense_qx_generic_kernel(const uint16_t* __restrict__ x, int64_t ldx, int64_t m,
                                                             int64_t n, int64_t k, const uint8_t* __restrict__ wdata,
                                                             int qbits, int nib, const uint16_t* __restrict__ bias,
                                                             uint16_t* y, int64_t ldy, float scale,
                                                             const uint16_t* add, int64_t ld_add, int act,
                                                             const uint16_t* __restrict__ gate, float* __restrict__ res,
                                                             int64_t ld_res, const float* __restrict__ gate32,
                                                             const uint16_t* mul, int64_t ld_mul) {
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
  float v = round_f16(acc);
  v = post_value(v, scale, add != nullptr, add ? (float)bits_to_half(add[mi * ld_add + ni]) : 0.f, mul != nullptr,
                 mul ? (float)bits_to_half(mul[mi * ld_mul + ni]) : 1.f, act, gate != nullptr,
                 gate ? (float)bits_to_half(gate[ni]) : 1.0f);
  if (res) {
    float pr = gate32 ? v * gate32[ni] : v;
    asm volatile("" : "+v"(pr));  // no fused multiply-add: the product is rounded first
    res[mi * ld_res + ni] += pr;
  }
  if (y) y[mi * ldy + ni] = half_to_bits((half_t)v);
}

extern template dt_status launch_dense_q<4>(hipStream_t, const DenseArgs&, int, bool, int);
extern template dt_status launch_dense_q<5>(hipStream_t, const DenseArgs&, int, bool, int);
extern template dt_status launch_dense_q<6>(hipStream_t, const DenseArgs&, int, bool, int);
extern template dt_status launch_dense_q<7>(hipStream_t, const DenseArgs&, int, bool, int);
extern template dt_status launch_dense_q<8>(hipStream_t, const DenseArgs&, int, bool, int);
extern template dt_status launch_dense_q<16>(hipStream_t, const DenseArgs&, int, bool, int);

// the kernel with the elementwise tail only when some weight of the launch asks for one
static dt_status launch_dense(hipStream_t s, const DenseArgs& a, int tile, int qbits, int mode) {
  bool post = false;
  for (int i = 0; i < kMaxWeights; i++) post = post || a.w[i].act != DT_ACT_NONE || a.w[i].gate || a.w[i].res || a.w[i].add || a.w[i].mul || a.w[i].scale != 1.0f;
  switch (qbits) {
    case 4: return launch_dense_q<4>(s, a, tile, post, mode);
    case 5: return launch_dense_q<5>(s, a, tile, post, mode);
    case 6: return launch_dense_q<6>(s, a, tile, post, mode);
    case 7: return launch_dense_q<7>(s, a, tile, post, mode);
    case 8: return launch_dense_q<8>(s, a, tile, post, mode);
    case 16: return launch_dense_q<16>(s, a, tile, post, mode);
  }
  return DT_INVALID;
}

// Palette placement for a BN-row tile (see PalMode).
static int choose_pal_mode(int qbits, int nib, int64_t K, int BM, int BN) {
  if (qbits == 16) return kPlainF16;
  const int64_t pal_bytes = (int64_t)2 << qbits;
  const int64_t budget = pal_lds_bytes(BM, BN);
  if ((int64_t)BN * pal_bytes <= budget) return kPalRow;
  const int64_t shared_count = ((int64_t)BN * K) / nib + 2;
  if (shared_count * pal_bytes <= budget) return kPalShared;
  return kPalGlobal;
}

}  // namespace dt

namespace dt {

// One Dense problem as the entry points receive it.
struct HostGroup {
  int64_t M, K;
  const uint16_t* X;
  int64_t ldx;
  const dt_qx_weight* W;
  int32_t n_weights;
  const uint16_t* const* bias;
  uint16_t* const* Y;
  const int64_t* ldy;
  const dt_head_epilogue* epi;
  const dt_dense_post* post;

  bool wants_epi(int wi) const { return epi && (epi[wi].gamma || epi[wi].rot); }
  // fused head epilogue: in the tiled kernel for 128-wide heads that start on a 16-byte aligned,
  // 8-element-strided output; otherwise the Dense runs plain and the norm / rotation pass follows
  bool fusable(int wi) const {
    return epi[wi].head_dim == 128 && (ldy[wi] % 8 == 0) && ((reinterpret_cast<uintptr_t>(Y[wi]) & 15) == 0) &&
           (!epi[wi].gamma || (reinterpret_cast<uintptr_t>(epi[wi].gamma) & 7) == 0) &&
           (!epi[wi].rot || (reinterpret_cast<uintptr_t>(epi[wi].rot) & 7) == 0) &&
           (!bias || !bias[wi] || (reinterpret_cast<uintptr_t>(bias[wi]) & 7) == 0);
  }
  // (the tiled kernel addresses X and the packed weight with 32-bit byte offsets from their bases)
  bool x_ok() const {
    return (K % (2 * BK) == 0) && (ldx % 8 == 0) && ((reinterpret_cast<uintptr_t>(X) & 15) == 0) &&
           (M == 0 || ((M - 1) * ldx + K) * 2 <= (int64_t)0xffffffff);
  }
  bool w_tiled(int wi) const {
    const dt_qx_weight& w = W[wi];
    if (!(w.count / K > 0 && (reinterpret_cast<uintptr_t>(w.data) & 15) == 0 && (w.qbits == 16 || w.nib % 32 == 0))) return false;
    const int64_t bytes = w.qbits == 16 ? w.count * 2 : dt_qx_bytes(w.qbits, w.nib, w.count);
    return bytes > 0 && bytes <= (int64_t)0xffffffff;
  }
};

static dt_status validate_group(const HostGroup& h) {
  if (h.epi && h.n_weights > 0) {
    for (int i = 0; i < h.n_weights; i++) {
      const dt_head_epilogue& e = h.epi[i];
      if (!e.gamma && !e.rot) continue;
      if (e.head_dim <= 0 || e.head_dim % 2 != 0 || e.head_dim > 128) return DT_NO_KERNEL;
      if (e.rot && e.rot_pos0 < 0) return DT_INVALID;
      if (h.Y && h.ldy && h.M > 0 && ((h.ldy[i] & 1) || (reinterpret_cast<uintptr_t>(h.Y[i]) & 3))) return DT_INVALID;
      if (e.rot && (reinterpret_cast<uintptr_t>(e.rot) & 3)) return DT_INVALID;
      if (h.W && h.K > 0 && h.W[i].count >= 0 && (h.W[i].count / h.K) % e.head_dim != 0) return DT_INVALID;
    }
  }
  if (h.M < 0 || h.K <= 0 || h.n_weights <= 0 || !h.W || !h.Y || !h.ldy) return DT_INVALID;
  if (h.post && h.epi) return DT_INVALID;
  if (h.post)
    for (int i = 0; i < h.n_weights; i++) {
      const dt_dense_post& p = h.post[i];
      if (p.activation < DT_ACT_NONE || p.activation > DT_ACT_GELU_ERF) return DT_INVALID;
      if (p.multiplicand && ((reinterpret_cast<uintptr_t>(p.multiplicand) & 1) || (h.W && h.K > 0 && p.ld_multiplicand < h.W[i].count / h.K)))
        return DT_INVALID;
      if (p.residual && ((reinterpret_cast<uintptr_t>(p.residual) & 3) || (h.W && h.K > 0 && p.ld_residual < h.W[i].count / h.K)))
        return DT_INVALID;
      if (p.addend && ((reinterpret_cast<uintptr_t>(p.addend) & 1) || (h.W && h.K > 0 && p.ld_addend < h.W[i].count / h.K)))
        return DT_INVALID;
      if (!(p.scale == p.scale) || p.scale - p.scale != 0.f) return DT_INVALID;  // NaN or infinite
      if (p.gate_f32 && (!p.residual || p.gate || (reinterpret_cast<uintptr_t>(p.gate_f32) & 3))) return DT_INVALID;
    }
  if (h.M > 0x7fffffff || h.K > 0x7fffffff) return DT_INVALID;
  for (int i = 0; i < h.n_weights; i++) {
    const dt_qx_weight& w = h.W[i];
    if (!w.data || w.count < 0 || w.count % h.K != 0) return DT_INVALID;
    if (w.qbits != 16 && (w.qbits < 4 || w.qbits > 8 || w.nib <= 0)) return DT_INVALID;
    if (w.count / h.K > 0x7fffffff) return DT_INVALID;
    const bool to_residual_only = h.post && h.post[i].residual && !h.Y[i];
    if (h.M > 0 && !to_residual_only && (!h.Y[i] || h.ldy[i] < w.count / h.K)) return DT_INVALID;
  }
  if (h.M > 0 && (!h.X || h.ldx < h.K)) return DT_INVALID;
  return DT_OK;
}

static dt_status epilogue_pass(hipStream_t s, const HostGroup& h, int wi) {
  QkPrepArgs p;
  p.src = h.Y[wi];
  p.dst = h.Y[wi];
  p.src_sb = p.dst_sb = 0;
  p.src_ss = p.dst_ss = h.ldy[wi];
  p.src_sh = p.dst_sh = h.epi[wi].head_dim;
  p.B = 1;
  p.S = h.M;
  p.H = (int32_t)((h.W[wi].count / h.K) / h.epi[wi].head_dim);
  p.D = h.epi[wi].head_dim;
  p.gamma = h.epi[wi].gamma;
  p.eps = h.epi[wi].eps;
  p.norm_per_head = 1;
  p.rot = h.epi[wi].rot;
  p.rot_pos0 = h.epi[wi].rot_pos0;
  p.post_scale = 1.0f;
  return qk_prep_launch(s, p);
}

// dt_dense_post::scale as the kernels take it: 0 (a zeroed struct) means none.
static float post_scale(const HostGroup& h, int wi) {
  return h.post && h.post[wi].scale != 0.f ? h.post[wi].scale : 1.0f;
}

// Appends weight wi of h to the launch; returns its number of N-tiles.
static int add_weight(DenseArgs& a, int slot, const HostGroup& h, int wi, int tile_begin, int BN, bool fuse) {
  const int64_t n_rows = h.W[wi].count / h.K;
  DenseWeight& d = a.w[slot];
  d.data = static_cast<const uint8_t*>(h.W[wi].data);
  d.bias = h.bias ? h.bias[wi] : nullptr;
  d.y = h.Y[wi];
  d.ldy = h.ldy[wi];
  d.n = (int32_t)n_rows;
  d.tile_begin = tile_begin;
  d.gamma = fuse ? h.epi[wi].gamma : nullptr;
  d.rot = fuse ? h.epi[wi].rot : nullptr;
  d.rot_pos0 = fuse ? h.epi[wi].rot_pos0 : 0;
  d.eps = fuse ? h.epi[wi].eps : 0.f;
  d.scale = post_scale(h, wi);
  d.add = h.post ? h.post[wi].addend : nullptr;
  d.ld_add = h.post ? h.post[wi].ld_addend : 0;
  d.act = h.post ? h.post[wi].activation : DT_ACT_NONE;
  d.gate = h.post ? h.post[wi].gate : nullptr;
  d.res = h.post ? h.post[wi].residual : nullptr;
  d.ld_res = h.post ? h.post[wi].ld_residual : 0;
  d.gate32 = h.post ? h.post[wi].gate_f32 : nullptr;
  d.mul = h.post ? h.post[wi].multiplicand : nullptr;
  d.ld_mul = h.post ? h.post[wi].ld_multiplicand : 0;
  return (int)((n_rows + BN - 1) / BN);
}

static void finish_args(DenseArgs& a, int n_groups, int n_w, int64_t K, const dt_qx_weight& w0) {
  for (int j = n_w; j < kMaxWeights; j++) a.w[j] = a.w[0];
  for (int j = n_groups; j < kMaxGroups; j++) a.g[j] = a.g[0];
  a.n_groups = n_groups;
  a.k = (int32_t)K;
  a.nib = w0.qbits == 16 ? 32 : w0.nib;
  a.pal_step = (int32_t)(std::gcd((int64_t)K, (int64_t)a.nib) / BK);
}

// One validated problem with M > 0: weights that share (qbits, nib) and meet the
// tiled kernel's alignment go out in runs of up to kMaxWeights per launch; the
// rest take the generic kernel.
// Fewer 256 x 256 tiles than this leave too many of the 256 compute units idle: such launches take 128 x 128 tiles.
constexpr int64_t kFillTiles = 192;

static dt_status run_group(hipStream_t s, const HostGroup& h) {
  const int64_t M = h.M, K = h.K;
  const bool x_ok = h.x_ok();
  int i = 0;
  while (i < h.n_weights) {
    const dt_qx_weight& w0 = h.W[i];
    const int64_t n_rows0 = w0.count / K;
    if (!(x_ok && h.w_tiled(i))) {
      if (n_rows0 > 0) {
        int64_t outs = M * n_rows0;
        if ((outs + 255) / 256 > 0x7fffffff) return DT_NO_KERNEL;
        hipLaunchKernelGGL(dense_qx_generic_kernel, dim3((unsigned)((outs + 255) / 256)), dim3(256), 0, s, h.X, h.ldx,
                           M, n_rows0, K, static_cast<const uint8_t*>(w0.data), w0.qbits, w0.nib,
                           h.bias ? h.bias[i] : nullptr, h.Y[i], h.ldy[i], post_scale(h, i),
                           h.post ? h.post[i].addend : nullptr, h.post ? h.post[i].ld_addend : 0,
                           h.post ? h.post[i].activation : DT_ACT_NONE,
                           h.post ? h.post[i].gate : nullptr, h.post ? h.post[i].residual : nullptr,
                           h.post ? h.post[i].ld_residual : 0, h.post ? h.post[i].gate_f32 : nullptr,
                           h.post ? h.post[i].multiplicand : nullptr, h.post ? h.post[i].ld_multiplicand : 0);
        dt_status st = launch_status();
        if (st != DT_OK) return st;
        if (h.wants_epi(i)) {
          st = epilogue_pass(s, h, i);
          if (st != DT_OK) return st;
        }
      }
      i++;
      continue;
    }
    // tile shape: big tiles when there is enough work to fill 256 CUs with them
    bool any_fused = false;
    for (int j = i; j < h.n_weights && j < i + kMaxWeights; j++)
      any_fused = any_fused || (h.wants_epi(j) && h.fusable(j));
    // (the fused epilogue needs the 128-feature wave slice of the big tile)
    int64_t big_tiles = 0;  // 256 x 256 tiles this launch would have
    for (int j = i, cnt = 0; j < h.n_weights && cnt < kMaxWeights; j++, cnt++) {
      const dt_qx_weight& wj = h.W[j];
      if (wj.qbits != w0.qbits || (wj.qbits != 16 && wj.nib != w0.nib) || !h.w_tiled(j)) break;
      big_tiles += ((M + 255) / 256) * ((wj.count / K + 255) / 256);
    }
    // (palettes that fit beside no big tile -- 256-entry palettes with small blocks -- would be looked up in memory:
    // the small tile holds a per-row table of them and is several times faster, unless a fused epilogue needs the big one)
    const bool pal_fits_big = choose_pal_mode(w0.qbits, w0.nib, K, 256, 256) != kPalGlobal ||
                              choose_pal_mode(w0.qbits, w0.nib, K, 128, 128) == kPalGlobal;
    const bool big = (((M >= 1024) && (n_rows0 >= 256) && big_tiles >= kFillTiles) && pal_fits_big) || any_fused;
    // few token rows: halve the token tile so that more workgroups share the work
    const bool narrow = big && M < 1024;
    // palettes that only fit beside a 128-feature tile, and enough work for tall tiles: 256 tokens x 128 features
    // (twice the MFMAs per unpacked weight of the 128 x 128 tile)
    const bool tall = !big && !pal_fits_big && (w0.qbits == 7 || w0.qbits == 8) && M >= 1024 && n_rows0 >= 128 &&
                      big_tiles * 2 >= kFillTiles;
    const int BM = big ? (narrow ? 128 : 256) : (tall ? 256 : 128), BN = big ? 256 : 128;
    DenseArgs a;
    DenseGroup& g = a.g[0];
    g.x = h.X;
    g.ldx = h.ldx;
    g.m = (int32_t)M;
    g.tiles_m = (int)((M + BM - 1) / BM);
    g.tile_begin = 0;
    g.w_begin = 0;
    int tiles_n = 0, cnt = 0;
    const int first = i;
    while (i < h.n_weights && cnt < kMaxWeights) {
      const dt_qx_weight& w = h.W[i];
      if (w.qbits != w0.qbits || (w.qbits != 16 && w.nib != w0.nib) || !h.w_tiled(i)) break;
      tiles_n += add_weight(a, cnt, h, i, tiles_n, BN, big && h.wants_epi(i) && h.fusable(i));
      cnt++;
      i++;
    }
    g.w_end = cnt;
    g.tiles_n = tiles_n;
    if ((int64_t)g.tiles_m * tiles_n > 0x7fffffff) return DT_NO_KERNEL;
    a.total_tiles = g.tiles_m * tiles_n;
    finish_args(a, 1, cnt, K, w0);
    const int mode = choose_pal_mode(w0.qbits, a.nib, K, BM, BN);
    dt_status st = launch_dense(s, a, tall ? kTile256x128 : !big ? kTile128x128 : narrow ? kTile128x256 : kTile256x256,
                                w0.qbits, mode);
    if (st != DT_OK) return st;
    for (int j = first; j < i; j++)
      if (h.wants_epi(j) && !(big && h.fusable(j))) {
        st = epilogue_pass(s, h, j);
        if (st != DT_OK) return st;
      }
  }
  return DT_OK;
}

// All problems in one launch of 256 x 256 tiles, when every X and weight meets
// the tiled kernel's alignment, they share K and the weight format, and at least
// one of them is large enough for that tile.  Returns false if they do not fit.
static bool run_groups_fused(hipStream_t s, const HostGroup* hs, int n, dt_status* status) {
  if (n < 2 || n > kMaxGroups) return false;
  const dt_qx_weight& w0 = hs[0].W[0];
  int total_w = 0;
  bool big = false;
  for (int gi = 0; gi < n; gi++) {
    const HostGroup& h = hs[gi];
    if (h.K != hs[0].K || !h.x_ok()) return false;
    for (int i = 0; i < h.n_weights; i++) {
      const dt_qx_weight& w = h.W[i];
      if (!h.w_tiled(i) || w.qbits != w0.qbits || (w.qbits != 16 && w.nib != w0.nib)) return false;
      big = big || (h.M >= 1024 && w.count / h.K >= 256);
    }
    total_w += h.n_weights;
  }
  if (!big || total_w > kMaxWeights) return false;
  if (choose_pal_mode(w0.qbits, w0.nib, hs[0].K, 256, 256) == kPalGlobal &&
      choose_pal_mode(w0.qbits, w0.nib, hs[0].K, 128, 128) != kPalGlobal)
    return false;  // problem by problem, on the small tile with its per-row palette table
  // the kernel variant with the elementwise tail has no fused head epilogue: such problems do not share a launch
  bool any_post = false, any_epi = false;
  for (int gi = 0; gi < n; gi++) {
    any_post = any_post || hs[gi].post != nullptr;
    for (int i = 0; i < hs[gi].n_weights; i++) any_epi = any_epi || hs[gi].wants_epi(i);
  }
  if (any_post && any_epi) return false;
  constexpr int BM = 256, BN = 256;
  DenseArgs a;
  int cnt = 0;
  int64_t tiles = 0;
  for (int gi = 0; gi < n; gi++) {
    const HostGroup& h = hs[gi];
    DenseGroup& g = a.g[gi];
    g.x = h.X;
    g.ldx = h.ldx;
    g.m = (int32_t)h.M;
    g.tiles_m = (int)((h.M + BM - 1) / BM);
    g.tile_begin = (int32_t)tiles;
    g.w_begin = cnt;
    int tiles_n = 0;
    for (int i = 0; i < h.n_weights; i++, cnt++)
      tiles_n += add_weight(a, cnt, h, i, tiles_n, BN, h.wants_epi(i) && h.fusable(i));
    g.w_end = cnt;
    g.tiles_n = tiles_n;
    tiles += (int64_t)g.tiles_m * tiles_n;
    if (tiles > 0x7fffffff) return false;
  }
  a.total_tiles = (int32_t)tiles;
  finish_args(a, n, cnt, hs[0].K, w0);
  const int mode = choose_pal_mode(w0.qbits, a.nib, hs[0].K, BM, BN);
  dt_status st = launch_dense(s, a, kTile256x256, w0.qbits, mode);
  for (int gi = 0; gi < n && st == DT_OK; gi++)
    for (int i = 0; i < hs[gi].n_weights && st == DT_OK; i++)
      if (hs[gi].wants_epi(i) && !hs[gi].fusable(i)) st = epilogue_pass(s, hs[gi], i);
  *status = st;
  return true;
}

}  // namespace dt

DT_EXPORT dt_status dt_dense_qx_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                    const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                                    uint16_t* const* Y, const int64_t* ldy, uint32_t flags) {
  return dt_dense_qx_heads_f16(stream, M, K, X, ldx, W, n_weights, bias, Y, ldy, nullptr, flags);
}

DT_EXPORT dt_status dt_dense_qx_heads_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                          const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                                          uint16_t* const* Y, const int64_t* ldy, const dt_head_epilogue* epi,
                                          uint32_t flags) {
  using namespace dt;
  (void)flags;
  const HostGroup h{M, K, X, ldx, W, n_weights, bias, Y, ldy, epi, nullptr};
  dt_status st = validate_group(h);
  if (st != DT_OK) return st;
  if (M == 0) return DT_OK;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  return run_group(as_stream(stream), h);
}

DT_EXPORT dt_status dt_dense_qx_post_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                         const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                                         uint16_t* const* Y, const int64_t* ldy, const dt_dense_post* post,
                                         uint32_t flags) {
  using namespace dt;
  (void)flags;
  const HostGroup h{M, K, X, ldx, W, n_weights, bias, Y, ldy, nullptr, post};
  dt_status st = validate_group(h);
  if (st != DT_OK) return st;
  if (M == 0) return DT_OK;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  return run_group(as_stream(stream), h);
}

DT_EXPORT dt_status dt_dense_qx_grouped_f16(dt_stream stream, int32_t n_groups, const dt_dense_group* groups,
                                            uint32_t flags) {
  using namespace dt;
  (void)flags;
  if (n_groups < 0 || (n_groups > 0 && !groups)) return DT_INVALID;
  if (n_groups > 64) return DT_INVALID;
  HostGroup hs[64];
  int n = 0;
  for (int i = 0; i < n_groups; i++) {
    const dt_dense_group& d = groups[i];
    const HostGroup h{d.M, d.K, d.X, d.ldx, d.W, d.n_weights, d.bias, d.Y, d.ldy, d.epi, d.post};
    dt_status st = validate_group(h);
    if (st != DT_OK) return st;
    if (h.M > 0) hs[n++] = h;
  }
  if (n == 0) return DT_OK;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  hipStream_t s = as_stream(stream);
  dt_status st = DT_OK;
  if (run_groups_fused(s, hs, n, &st)) return st;
  for (int i = 0; i < n; i++) {
    st = run_group(s, hs[i]);
    if (st != DT_OK) return st;
  }
  return DT_OK;
}

// Launchers of the tiled Dense kernels, instantiated once per index width in dt_dense_q<Q>.hip.
#pragma once
#include "dt_dense_kernel.h"

namespace dt {

// Tile shapes the host side chooses between.
// (tokens x features; 256 x 128 exists for the palettes that only fit beside a 128-feature tile -- per-row tables of
// 128 and 256 entries -- and is instantiated for those index widths only)
enum DenseTile : int { kTile128x128 = 0, kTile128x256 = 1, kTile256x256 = 2, kTile256x128 = 3 };

template <int Q, int BM, int BN, bool POST>
static dt_status launch_tiled(hipStream_t s, const DenseArgs& a, int mode) {
  dim3 grid((unsigned)a.total_tiles), block(512);
  if constexpr (Q == 16) {  // plain fp16 weight
    hipLaunchKernelGGL((dense_qx_kernel<8, BM, BN, kPlainF16, POST>), grid, block, 0, s, a);
    return launch_status();
  } else {
    switch (mode) {
      case kPalShared: hipLaunchKernelGGL((dense_qx_kernel<Q, BM, BN, kPalShared, POST>), grid, block, 0, s, a); break;
      case kPalRow:
        if constexpr ((BN << (Q + 1)) <= pal_lds_bytes(BM, BN)) {
          hipLaunchKernelGGL((dense_qx_kernel<Q, BM, BN, kPalRow, POST>), grid, block, 0, s, a);
          break;
        } else {
          return DT_NO_KERNEL;  // choose_pal_mode never picks per-row palettes that do not fit
        }
      default: hipLaunchKernelGGL((dense_qx_kernel<Q, BM, BN, kPalGlobal, POST>), grid, block, 0, s, a); break;
    }
    return launch_status();
  }
}

template <int Q, bool POST>
static dt_status launch_dense_qp(hipStream_t s, const DenseArgs& a, int tile, int mode) {
  switch (tile) {
    case kTile128x128: return launch_tiled<Q, 128, 128, POST>(s, a, mode);
    case kTile128x256: return launch_tiled<Q, 128, 256, POST>(s, a, mode);
    case kTile256x128:
      if constexpr (Q == 7 || Q == 8) {
        if (mode != kPalRow) return DT_NO_KERNEL;
        hipLaunchKernelGGL((dense_qx_kernel<Q, 256, 128, kPalRow, POST>), dim3((unsigned)a.total_tiles), dim3(512), 0, s, a);
        return launch_status();
      } else {
        return DT_NO_KERNEL;  // the host side picks this tile for 7- and 8-bit indices only
      }
    default: return launch_tiled<Q, 256, 256, POST>(s, a, mode);
  }
}

// Every tiled kernel for Q-bit indices (Q = 16: plain fp16 weights); `post` selects the variant with the
// elementwise tail.  Instantiated once per Q in dt_dense_q<Q>.hip.
template <int Q>
dt_status launch_dense_q(hipStream_t s, const DenseArgs& a, int tile, bool post, int mode) {
  return post ? launch_dense_qp<Q, true>(s, a, tile, mode) : launch_dense_qp<Q, false>(s, a, tile, mode);
}

}  // namespace dt

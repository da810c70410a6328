// K0: depalettize a packed tensor to fp16 (bit-exact table lookup).
// HBM-bound byte work: reads count*q/8 + palettes, writes 2*count bytes.
#include "dt_common.h"
#include "dt_layout.h"

namespace dt {

// One thread per 32-element granule (needs nib % 32 == 0 so that a granule
// never straddles a block and always starts on a dword of the index stream).
template <int Q>
__global__ void __launch_bounds__(256) depalettize32_kernel(const uint8_t* __restrict__ packed, int nib,
                                                          int64_t n_granules, uint16_t* __restrict__ out) {
  int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (g >= n_granules) return;
  const QxLayout l = make_layout(Q, nib);
  int64_t e = g * 32;
  int64_t b = e / nib;
  int64_t r = e - b * nib;
  const uint16_t* pal = reinterpret_cast<const uint16_t*>(packed + palette_offset(l, b));
  const uint32_t* src = reinterpret_cast<const uint32_t*>(packed + index_byte_offset(l, b, r));
  uint32_t raw[Q];
#pragma unroll
  for (int i = 0; i < Q; i++) raw[i] = src[i];
  uint32_t idx[32];
  unpack32<Q>(raw, idx);
  uint32_t o[16];
#pragma unroll
  for (int j = 0; j < 16; j++) o[j] = (uint32_t)pal[idx[2 * j]] | ((uint32_t)pal[idx[2 * j + 1]] << 16);
  uint16_t* dst = out + e;
  if ((reinterpret_cast<uintptr_t>(dst) & 15) == 0) {
    uint4_t* d4 = reinterpret_cast<uint4_t*>(dst);
#pragma unroll
    for (int j = 0; j < 4; j++) d4[j] = uint4_t{o[4 * j], o[4 * j + 1], o[4 * j + 2], o[4 * j + 3]};
  } else {
#pragma unroll
    for (int j = 0; j < 16; j++) {
      dst[2 * j] = (uint16_t)o[j];
      dst[2 * j + 1] = (uint16_t)(o[j] >> 16);
    }
  }
}

// The same granule-per-thread unpacking for blocks of 512 elements and more, with both sides of the lookup moved
// into LDS: the palettes of the (at most 8192 / nib + 2) blocks that a workgroup's 256 granules touch are loaded once,
// and the 64 bytes a thread produces go through a [thread][4 chunks] staging array, so that every store
// instruction of a wave writes 1 KB of consecutive addresses (thread-per-granule stores are 64 bytes apart per lane).
// Chunk c of thread t is staged at chunk 4 t + (c ^ (t / 4 % 4)): 16 consecutive lanes hit 16 different 16-byte
// bank groups on the way in (stride of 4 chunks) and on the way out (consecutive chunks).
constexpr int kDepalMinNib = 512;
template <int Q>
__global__ void __launch_bounds__(256) depalettize_tile_kernel(const uint8_t* __restrict__ packed, int nib,
                                                             int64_t n_granules, uint16_t* __restrict__ out) {
  constexpr int MAXP = 8192 / kDepalMinNib + 2;
  __shared__ uint16_t pal[MAXP << Q];
  __shared__ __attribute__((aligned(16))) uint4_t stage[256 * 4];
  const int t = threadIdx.x;
  const int64_t g0 = (int64_t)blockIdx.x * 256;
  const QxLayout l = make_layout(Q, nib);
  const int64_t g_last = (g0 + 255 < n_granules ? g0 + 255 : n_granules - 1);
  const int64_t b_first = g0 * 32 / nib, b_last = (g_last * 32 + 31) / nib;
  const int n_pal = (int)(b_last - b_first + 1);
  for (int i = t; i < n_pal << (Q - 1); i += 256) {
    const int p = i >> (Q - 1), e = i & ((1 << (Q - 1)) - 1);
    reinterpret_cast<uint32_t*>(pal)[i] =
        reinterpret_cast<const uint32_t*>(packed + palette_offset(l, b_first + p))[e];
  }
  __syncthreads();
  const int64_t g = g0 + t;
  if (g < n_granules) {
    const int64_t e = g * 32;
    const int64_t b = e / nib;
    const int64_t r = e - b * nib;
    const uint32_t* src = reinterpret_cast<const uint32_t*>(packed + index_byte_offset(l, b, r));
    uint32_t raw[Q];
#pragma unroll
    for (int i = 0; i < Q; i++) raw[i] = src[i];
    uint32_t idx[32];
    unpack32<Q>(raw, idx);
    const uint16_t* mine = pal + ((int)(b - b_first) << Q);
    uint32_t o[16];
#pragma unroll
    for (int j = 0; j < 16; j++) o[j] = (uint32_t)mine[idx[2 * j]] | ((uint32_t)mine[idx[2 * j + 1]] << 16);
#pragma unroll
    for (int c = 0; c < 4; c++)
      stage[4 * t + (c ^ ((t >> 2) & 3))] = uint4_t{o[4 * c], o[4 * c + 1], o[4 * c + 2], o[4 * c + 3]};
  }
  __syncthreads();
  // chunk L of the workgroup's 16 KB (L = 4 * thread + c) leaves through lane L % 256 of trip L / 256
  uint4_t* dst = reinterpret_cast<uint4_t*>(out + g0 * 32);
  const int64_t n_chunks = (g_last - g0 + 1) * 4;
#pragma unroll
  for (int j = 0; j < 4; j++) {
    const int L = j * 256 + t;
    const int src_t = L >> 2, c = L & 3;
    if (L < n_chunks) dst[L] = stage[4 * src_t + (c ^ ((src_t >> 2) & 3))];
  }
}

template <int Q>
static void launch_granules(bool tiled, dim3 grid, hipStream_t s, const uint8_t* packed, int nib, int64_t ng,
                            uint16_t* out) {
  if (tiled) hipLaunchKernelGGL(depalettize_tile_kernel<Q>, grid, dim3(256), 0, s, packed, nib, ng, out);
  else hipLaunchKernelGGL(depalettize32_kernel<Q>, grid, dim3(256), 0, s, packed, nib, ng, out);
}

// One thread per element: any nib, ragged tails.
__global__ void __launch_bounds__(256) depalettize1_kernel(const uint8_t* __restrict__ packed, int qbits, int nib,
                                                         int64_t first, int64_t count,
                                                         uint16_t* __restrict__ out) {
  int64_t e = first + (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (e >= count) return;
  const QxLayout l = make_layout(qbits, nib);
  int64_t b = e / nib;
  int64_t r = e - b * nib;
  const uint16_t* pal = reinterpret_cast<const uint16_t*>(packed + palette_offset(l, b));
  const uint8_t* idx = packed + palette_offset(l, b) + l.pal_bytes;
  out[e] = pal[load_index(idx, r, qbits)];
}

}  // namespace dt

DT_EXPORT dt_status dt_depalettize_f16(dt_stream stream, const dt_qx_weight* w, uint16_t* out) {
  using namespace dt;
  if (!w || w->count < 0) return DT_INVALID;
  if (w->count == 0) return DT_OK;
  if (!w->data || !out) return DT_INVALID;
  if (w->qbits < 4 || w->qbits > 8 || w->nib <= 0) return DT_INVALID;
  if ((reinterpret_cast<uintptr_t>(out) & 1) != 0) return DT_INVALID;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  hipStream_t s = as_stream(stream);
  const uint8_t* packed = static_cast<const uint8_t*>(w->data);
  int64_t done = 0;
  if (w->nib % 32 == 0 && (reinterpret_cast<uintptr_t>(packed) & 3) == 0) {
    int64_t ng = w->count / 32;
    if (ng > 0) {
      if ((ng + 255) / 256 > 0x7fffffff) return DT_NO_KERNEL;
      dim3 grid((unsigned)((ng + 255) / 256));
      const bool tiled = w->nib >= kDepalMinNib && (reinterpret_cast<uintptr_t>(out) & 15) == 0;
      switch (w->qbits) {
        case 4: launch_granules<4>(tiled, grid, s, packed, w->nib, ng, out); break;
        case 5: launch_granules<5>(tiled, grid, s, packed, w->nib, ng, out); break;
        case 6: launch_granules<6>(tiled, grid, s, packed, w->nib, ng, out); break;
        case 7: launch_granules<7>(tiled, grid, s, packed, w->nib, ng, out); break;
        default: launch_granules<8>(tiled, grid, s, packed, w->nib, ng, out); break;
      }
      done = ng * 32;
    }
  }
  if (done < w->count) {
    int64_t rest = w->count - done;
    if ((rest + 255) / 256 > 0x7fffffff) return DT_NO_KERNEL;
    hipLaunchKernelGGL(depalettize1_kernel, dim3((unsigned)((rest + 255) / 256)), dim3(256), 0, s, packed, w->qbits,
                       w->nib, done, w->count, out);
  }
  return launch_status();
}

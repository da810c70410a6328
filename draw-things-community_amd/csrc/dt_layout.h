// The palettized ("q4p/q5p/q6p/q7p/q8p") tensor layout, in one place.
//
//   buffer  := block_0 block_1 ... ; block b covers elements [b*nib, (b+1)*nib)
//   block_b := palette[2^qbits] fp16 (little-endian), then the block's indices
//   indices := MSB-first bit stream: index j of the block occupies bits
//              [j*q, (j+1)*q) counted from the most significant bit of byte 0
//   value[i] = palette[i / nib][index[i]]
//
// Every kernel reaches the format through these helpers only.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define DT_HD __host__ __device__ __forceinline__
#else
#define DT_HD inline
#endif

namespace dt {

struct QxLayout {
  int qbits;
  int nib;
  int64_t pal_bytes;     // 2^qbits * 2
  int64_t block_stride;  // pal_bytes + bytes of a full block's indices
};

DT_HD QxLayout make_layout(int qbits, int nib) {
  QxLayout l;
  l.qbits = qbits;
  l.nib = nib;
  l.pal_bytes = (int64_t)2 << qbits;
  l.block_stride = l.pal_bytes + ((int64_t)nib * qbits + 7) / 8;
  return l;
}

DT_HD int64_t qx_total_bytes(int qbits, int nib, int64_t count) {
  if (qbits < 4 || qbits > 8 || nib <= 0 || count < 0) return -1;
  int64_t nblocks = (count + nib - 1) / nib;
  int64_t full = count / nib;
  int64_t tail = count - full * nib;
  return nblocks * ((int64_t)2 << qbits) + full * (((int64_t)nib * qbits + 7) / 8) +
         (tail * qbits + 7) / 8;
}

// Byte offset of block b's palette.
DT_HD int64_t palette_offset(const QxLayout& l, int64_t block) { return block * l.block_stride; }

// Byte offset of the index byte holding the first bit of element r of block b.
DT_HD int64_t index_byte_offset(const QxLayout& l, int64_t block, int64_t r) {
  return block * l.block_stride + l.pal_bytes + ((r * l.qbits) >> 3);
}

#if defined(__HIPCC__)
// Index of element r (any r) of a block whose index stream starts at `idx`.
__device__ __forceinline__ uint32_t load_index(const uint8_t* idx, int64_t r, int qbits) {
  int64_t bit = r * qbits;
  const uint8_t* p = idx + (bit >> 3);
  int off = (int)(bit & 7);
  uint32_t w = (uint32_t)p[0] << 8;
  if (off + qbits > 8) w |= p[1];
  return (w >> (16 - off - qbits)) & ((1u << qbits) - 1);
}

// 32 consecutive indices from Q little-endian dwords that start on a
// 32-element boundary of the stream.  All shifts are compile-time constants,
// so each index is one v_bfe_u32, or v_alignbit_b32 + v_and_b32 when it
// straddles two dwords.
template <int Q>
__device__ __forceinline__ void unpack32(const uint32_t (&raw)[Q], uint32_t (&idx)[32]) {
  uint32_t be[Q];
#pragma unroll
  for (int i = 0; i < Q; i++) be[i] = __builtin_bswap32(raw[i]);
#pragma unroll
  for (int j = 0; j < 32; j++) {
    const int bit = j * Q;
    const int word = bit >> 5;
    const int off = bit & 31;
    if (off + Q <= 32) {
      idx[j] = (be[word] >> (32 - off - Q)) & ((1u << Q) - 1);
    } else {
      const int sh = 64 - off - Q;  // 1..31
      const int wn = word + 1 < Q ? word + 1 : word;  // always word + 1 here
      uint32_t v = __builtin_amdgcn_alignbit(be[word], be[wn], sh);
      idx[j] = v & ((1u << Q) - 1);
    }
  }
}

// Indices 16*HALF .. 16*HALF + 15 of the same 32-index granule.
template <int Q, int HALF>
__device__ __forceinline__ void unpack16(const uint32_t (&raw)[Q], uint32_t (&idx)[16]) {
  uint32_t be[Q];
#pragma unroll
  for (int i = 0; i < Q; i++) be[i] = __builtin_bswap32(raw[i]);
#pragma unroll
  for (int j = 0; j < 16; j++) {
    const int bit = (16 * HALF + j) * Q;
    const int word = bit >> 5;
    const int off = bit & 31;
    if (off + Q <= 32) {
      idx[j] = (be[word] >> (32 - off - Q)) & ((1u << Q) - 1);
    } else {
      const int sh = 64 - off - Q;
      const int wn = word + 1 < Q ? word + 1 : word;
      uint32_t v = __builtin_amdgcn_alignbit(be[word], be[wn], sh);
      idx[j] = v & ((1u << Q) - 1);
    }
  }
}

// The same 16 indices from the HW = (Q + 1) / 2 dwords that hold them: `own`
// starts at dword Q / 2 * upper of the granule, where the upper half begins at
// bit 0 (even Q) or bit 16 (odd Q).  `upper` is a run-time value, so threads
// working on either half share one instruction stream.  Two steps, so that a
// caller can spread the extractions out: own_bits() turns the dwords into one
// big-endian bit string starting at the half's first index, own_index() cuts
// index j out of it.
template <int Q, int HW>
__device__ __forceinline__ void own_bits(const uint32_t (&own)[HW], bool upper, uint32_t (&be)[HW + 1]) {
#pragma unroll
  for (int i = 0; i < HW; i++) be[i] = __builtin_bswap32(own[i]);
  be[HW] = 0;
  if constexpr (Q & 1) {
#pragma unroll
    for (int i = 0; i < HW; i++) be[i] = upper ? __builtin_amdgcn_alignbit(be[i], be[i + 1], 16) : be[i];
  }
}
// own_index() << SH | base in two instructions (shift or funnel shift, then
// v_and_or_b32); base must have no bit in common with the shifted index.
template <int Q, int HW, int SH>
__device__ __forceinline__ uint32_t own_index_at(const uint32_t (&be)[HW + 1], int j, uint32_t base) {
  const int bit = j * Q;
  const int word = bit >> 5;
  const int off = bit & 31;
  const uint32_t mask = ((1u << Q) - 1) << SH;
  uint32_t v;
  if (off + Q <= 32) {
    const int r = 32 - off - Q - SH;  // right shift that leaves the index at bit SH
    v = r >= 0 ? be[word] >> r : be[word] << -r;
  } else {
    const int r = 64 - off - Q - SH;  // > 0: the index straddles two dwords
    v = r < 32 ? __builtin_amdgcn_alignbit(be[word], be[word + 1], r) : be[word] >> (r - 32);
  }
  uint32_t out;
  asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(out) : "v"(v), "s"(mask), "v"(base));
  return out;
}
template <int Q, int HW>
__device__ __forceinline__ uint32_t own_index(const uint32_t (&be)[HW + 1], int j) {
  const int bit = j * Q;
  const int word = bit >> 5;
  const int off = bit & 31;
  if (off + Q <= 32) return (be[word] >> (32 - off - Q)) & ((1u << Q) - 1);
  return __builtin_amdgcn_alignbit(be[word], be[word + 1], 64 - off - Q) & ((1u << Q) - 1);
}
#endif

}  // namespace dt

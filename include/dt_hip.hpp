// C++ host side above the C ABI of dt_hip.h: the operator objects the reference's model builders construct --
// Dense(count:noBias:flags:name:), RMSNorm(epsilon:axis:name:), Functional.cmul(left:right:),
// ScaledDotProductAttention(scale:isCausal:hasAttentionMask:flags:multiHeadOutputProjectionFused:name:)
// (Libraries/SwiftDiffusion/Sources/Models/Flux1.swift:161-245, Models/UNet.swift:95-156, Models/Wan.swift:68-160) --
// with the same names, argument meaning and error behaviour, for hosts written in a compiled language.  Header only;
// no device-memory management of its own: tensors are device pointers that the caller owns (the graph's buffers in
// the reference), described by the plain structs of the C ABI.  Errors are thrown as dt::Error carrying the status
// code, where the Swift operators would trap or fall through to another backend.
#pragma once
#include <cmath>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "dt_hip.h"

namespace dt {

struct Error : std::runtime_error {
  dt_status status;
  Error(const std::string& what, dt_status st) : std::runtime_error(what + ": status " + std::to_string(st)), status(st) {}
};
inline void check(const char* what, dt_status st) {
  if (st != DT_OK) throw Error(what, st);
}

// Functional.GEMMFlag: permissions to compute at a precision, not requests (Models/Flux1.swift:134, 162, 229-231).
enum GEMMFlag : uint32_t { Float16 = 1, Float32 = 2, Int8 = 4 };

// A weight as store.read(codec: [.jit, .q?p]) leaves it on the device: still palettized (qbits 4-8), or plain fp16
// (qbits 16).  [rows, cols] = [out, in].
struct QxTensor {
  const void* data = nullptr;
  int32_t qbits = 16, nib = 0;
  int64_t rows = 0, cols = 0;
  dt_qx_weight c() const { return dt_qx_weight{data, qbits, nib, rows * cols}; }
  int64_t bytes() const { return qbits == 16 ? rows * cols * 2 : dt_qx_bytes(qbits, nib, rows * cols); }
};

// A row-major fp16 matrix on the device: [rows, cols] with row stride ld (elements).
struct Matrix {
  uint16_t* ptr = nullptr;
  int64_t rows = 0, cols = 0, ld = 0;
};

// Dense(count:noBias:flags:name:): y = x W^T (+ bias).  `.weight` / `.bias` are filled by the loader, as the
// reference fills them through store.read (Models/Flux1.swift:288-321).
class Dense {
 public:
  Dense(int64_t count, bool noBias = false, uint32_t flags = 0, std::string name = "")
      : count(count), noBias(noBias), flags(flags), name(std::move(name)) {}
  int64_t count;
  bool noBias;
  uint32_t flags;
  std::string name;
  QxTensor weight;
  const uint16_t* bias = nullptr;

  void operator()(dt_stream stream, const Matrix& x, const Matrix& y) const {
    if (!weight.data) throw std::runtime_error("Dense " + name + ": weight not loaded");
    if (weight.rows != count || weight.cols != x.cols || y.rows != x.rows || y.cols != count)
      throw Error("Dense " + name + ": shapes", DT_INVALID);
    if (!noBias && !bias) throw std::runtime_error("Dense " + name + ": bias not loaded");
    const dt_qx_weight w = weight.c();
    const uint16_t* b[1] = {noBias ? nullptr : bias};
    uint16_t* ys[1] = {y.ptr};
    const int64_t ldy[1] = {y.ld};
    check("dt_dense_qx_f16", dt_dense_qx_f16(stream, x.rows, x.cols, x.ptr, x.ld, &w, 1, b, ys, ldy, flags));
  }
};

// Several Dense ops that share their input in one launch (x_q / x_k / x_v, Models/Flux1.swift:174-176), optionally
// with the per-head RMSNorm and RoPE that follow Q and K fused behind the projection (epilogues[i].gamma / .rot
// NULL = none for that weight).
inline void dense_multi(dt_stream stream, const Matrix& x, const std::vector<const Dense*>& ops,
                        const std::vector<Matrix>& ys, const std::vector<dt_head_epilogue>* epilogues = nullptr) {
  const size_t n = ops.size();
  if (ys.size() != n || (epilogues && epilogues->size() != n)) throw Error("dense_multi: arguments", DT_INVALID);
  std::vector<dt_qx_weight> w(n);
  std::vector<const uint16_t*> b(n);
  std::vector<uint16_t*> yp(n);
  std::vector<int64_t> ldy(n);
  uint32_t flags = 0;
  for (size_t i = 0; i < n; i++) {
    if (!ops[i]->weight.data) throw std::runtime_error("Dense " + ops[i]->name + ": weight not loaded");
    w[i] = ops[i]->weight.c();
    b[i] = ops[i]->noBias ? nullptr : ops[i]->bias;
    yp[i] = ys[i].ptr;
    ldy[i] = ys[i].ld;
    flags |= ops[i]->flags;
  }
  if (epilogues)
    check("dt_dense_qx_heads_f16", dt_dense_qx_heads_f16(stream, x.rows, x.cols, x.ptr, x.ld, w.data(), (int32_t)n, b.data(),
                                                         yp.data(), ldy.data(), epilogues->data(), flags));
  else
    check("dt_dense_qx_f16",
          dt_dense_qx_f16(stream, x.rows, x.cols, x.ptr, x.ld, w.data(), (int32_t)n, b.data(), yp.data(), ldy.data(), flags));
}

// RMSNorm(epsilon:axis:name:) on a [B, S, H, D] view, in place: axis [3] = per head (Flux, Models/Flux1.swift:165),
// axis [2] = over the whole H * D row (Wan, Models/Wan.swift:87-91).
class RMSNorm {
 public:
  RMSNorm(float epsilon, std::vector<int> axis, std::string name = "")
      : epsilon(epsilon), axis(std::move(axis)), name(std::move(name)) {}
  float epsilon;
  std::vector<int> axis;
  std::string name;
  const uint16_t* weight = nullptr;

  void operator()(dt_stream stream, dt_view4 x, int32_t B, int64_t S, int32_t H, int32_t D) const {
    if (!weight) throw std::runtime_error("RMSNorm " + name + ": weight not loaded");
    if (axis.size() != 1 || (axis[0] != 3 && axis[0] != 2)) throw Error("RMSNorm " + name + ": axis", DT_NO_KERNEL);
    check("dt_qk_norm_rope_f16",
          dt_qk_norm_rope_f16(stream, x, B, S, H, D, weight, epsilon, axis[0] == 3 ? 1 : 0, nullptr, 0, 1.0f));
  }
};

struct Functional {
  // Functional.cmul(left:right:): complex multiply of adjacent pairs with the rotary table `right`
  // ([>= pos0 + S, D] fp16, interleaved cos / sin), in place on `left`.
  static void cmul(dt_stream stream, dt_view4 left, int32_t B, int64_t S, int32_t H, int32_t D, const uint16_t* right,
                   int64_t pos0 = 0) {
    check("dt_qk_norm_rope_f16", dt_qk_norm_rope_f16(stream, left, B, S, H, D, nullptr, 0.f, 1, right, pos0, 1.0f));
  }
};

// ScaledDotProductAttention(scale:isCausal:hasAttentionMask:flags:multiHeadOutputProjectionFused:name:).  Inputs
// are lists of [B, len, H, D] segments (a joint text || image sequence without the concat,
// Models/Flux1.swift:184-186); the output is [B, Sq, Hq, D], or [B, Sq, Hq * D] through the fused unify-heads
// projection (`.weight` [Hq * D, Hq * D] fp16, `.bias`; Models/UNet.swift:143-155).
class ScaledDotProductAttention {
 public:
  ScaledDotProductAttention(float scale, bool isCausal = false, bool hasAttentionMask = false, uint32_t flags = 0,
                            bool multiHeadOutputProjectionFused = false, std::string name = "")
      : scale(scale), flags(flags), fused(multiHeadOutputProjectionFused), name(std::move(name)) {
    if (isCausal || hasAttentionMask) throw Error("ScaledDotProductAttention(isCausal / hasAttentionMask)", DT_NO_KERNEL);
  }
  float scale;
  uint32_t flags;
  bool fused;
  std::string name;
  const uint16_t* weight = nullptr;
  const uint16_t* bias = nullptr;

  // Scratch a call may use (see dt_sdpa_workspace_bytes): the staging it needs plus, where it pays, room for the
  // key-split form of the kernel.  The caller provides it (the reference's stream workspace allocator).
  size_t workspaceBytes(int32_t B, int32_t Hq, int32_t Hk, int32_t D, int64_t Sq, int64_t Skv, bool prep = false) const {
    return dt_sdpa_workspace_bytes(B, Hq, Hk, D, Sq, Skv, prep ? 1 : 0, fused ? 1 : 0);
  }

  void operator()(dt_stream stream, int32_t B, int32_t Hq, int32_t Hk, int32_t D, const std::vector<dt_seq_segment>& q,
                  const std::vector<dt_seq_segment>& k, const std::vector<dt_seq_segment>& v, dt_view4 o,
                  void* workspace = nullptr, size_t workspace_bytes = 0, const uint16_t* rot_q = nullptr,
                  const uint16_t* rot_k = nullptr, float eps = 1e-6f) const {
    if (fused && !weight) throw std::runtime_error("ScaledDotProductAttention " + name + ": weight not loaded");
    if (k.size() != v.size()) throw Error("ScaledDotProductAttention " + name + ": key / value segments", DT_INVALID);
    check("dt_sdpa_f16", dt_sdpa_f16(stream, B, Hq, Hk, D, (int32_t)q.size(), q.data(), (int32_t)k.size(), k.data(), v.data(),
                                     rot_q, rot_k, eps, o, scale, fused ? weight : nullptr, fused ? bias : nullptr,
                                     workspace, workspace_bytes));
  }
};

// Work units of the reference's estimator (Models/InstructionCount/InstructionCount.swift:4-17).
inline int64_t DenseInstructionCount(int64_t rows, int64_t input, int64_t output) { return rows * output * input; }
inline int64_t ScaledDotProductAttentionInstructionCount(int64_t batchSize, int64_t heads, int64_t headDimension,
                                                         int64_t sequenceDimensionA, int64_t sequenceDimensionB) {
  return batchSize * heads * (2 * headDimension + 5) * sequenceDimensionA * sequenceDimensionB;
}

}  // namespace dt

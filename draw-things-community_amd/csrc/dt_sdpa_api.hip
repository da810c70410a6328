// Host side of the attention entry point: validation, segment tables, the
// optional norm/rotate staging pass and the optional fused output projection.
#include <atomic>

#include "dt_common.h"
#include "dt_qkprep.h"
#include "dt_sdpa.h"

namespace dt {

static size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

static bool view_ok(const dt_view4& v, int align_elems) {
  if (!v.ptr) return false;
  const uintptr_t mask = (uintptr_t)align_elems * 2 - 1;
  if (reinterpret_cast<uintptr_t>(v.ptr) & mask) return false;
  return v.stride_b % align_elems == 0 && v.stride_s % align_elems == 0 && v.stride_h % align_elems == 0;
}

}  // namespace dt

DT_EXPORT size_t dt_sdpa_workspace_bytes(int32_t B, int32_t Hq, int32_t Hk, int32_t D, int64_t Sq, int64_t Skv,
                                         int32_t fused_prep, int32_t fused_out_proj) {
  using namespace dt;
  if (B <= 0 || Hq <= 0 || Hk <= 0 || D <= 0 || Sq <= 0 || Skv <= 0) return 0;
  size_t bytes = 0;
  // (the queries are normalised and rotated inside the attention kernel; only K is staged)
  if (fused_prep) bytes += align256((size_t)B * Skv * Hk * D * 2);
  if (fused_out_proj) bytes += align256((size_t)B * Sq * Hq * D * 2);
  // Optional part: room for the key-split form of the kernel (partial results of the pieces and the per-task
  // counters), for launches whose workgroup count leaves a good part of the last round of compute units idle.  A
  // call that is handed less than this, but at least the staging bytes above, runs unsplit.
  SdpaSplit plan;
  if (sdpa_split_plan(B, Hq, D, Sq, Skv, &plan)) bytes += align256(plan.bytes());
  return bytes;
}

namespace dt {

// What the argument checks of an attention request establish.
struct SdpaShape {
  int64_t Sq = 0, Skv = 0;
  bool prep = false;   // some segment is normalised or rotated on the way in
  bool qprep = false;  // ... a query segment (done inside the attention kernel)
  bool kprep = false;  // ... a key segment (staged into the workspace)
  bool empty = false;  // nothing to compute (no batch or no query row)
  size_t need = 0;     // staging bytes the request cannot run without (the first part of dt_sdpa_workspace_bytes)
};

// Argument checks shared by dt_sdpa_f16 and dt_sdpa_f16_static; touches no device state.
static dt_status sdpa_validate(int32_t B, int32_t Hq, int32_t Hk, int32_t D, int32_t n_qseg,
                               const dt_seq_segment* q_seg, int32_t n_kvseg, const dt_seq_segment* k_seg,
                               const dt_seq_segment* v_seg, const uint16_t* rot_q, const uint16_t* rot_k,
                               const dt_view4& o, const uint16_t* Wo, SdpaShape& sh) {
  if (B < 0 || Hq <= 0 || Hk <= 0 || D <= 0 || Hq % Hk != 0) return DT_INVALID;
  if (n_qseg <= 0 || n_kvseg <= 0 || !q_seg || !k_seg || !v_seg) return DT_INVALID;
  if (n_qseg > kMaxSeg || n_kvseg > kMaxSeg) return DT_NO_KERNEL;
  if (D % 8 != 0 || D > 128) return DT_NO_KERNEL;
  int64_t Sq = 0, Skv = 0;
  bool qprep = rot_q != nullptr, kprep = rot_k != nullptr;
  for (int i = 0; i < n_qseg; i++) {
    if (q_seg[i].len < 0) return DT_INVALID;
    Sq += q_seg[i].len;
    qprep = qprep || q_seg[i].gamma;
  }
  for (int i = 0; i < n_kvseg; i++) {
    if (k_seg[i].len < 0 || k_seg[i].len != v_seg[i].len) return DT_INVALID;
    Skv += k_seg[i].len;
    kprep = kprep || k_seg[i].gamma;
  }
  const bool prep = qprep || kprep;
  sh.Sq = Sq;
  sh.Skv = Skv;
  sh.prep = prep;
  sh.qprep = qprep;
  sh.kprep = kprep;
  if (B == 0 || Sq == 0) {
    sh.empty = true;
    return DT_OK;
  }
  if (Skv == 0) return DT_INVALID;  // softmax over an empty set
  for (int i = 0; i < n_qseg; i++)
    if (q_seg[i].len > 0 && !view_ok(q_seg[i].view, 8)) return DT_INVALID;
  for (int i = 0; i < n_kvseg; i++)
    if (k_seg[i].len > 0 && (!view_ok(k_seg[i].view, 8) || !view_ok(v_seg[i].view, 8))) return DT_INVALID;
  if (!o.ptr || (reinterpret_cast<uintptr_t>(o.ptr) & 7) || o.stride_b % 4 || o.stride_s % 4) return DT_INVALID;
  if (!Wo && o.stride_h % 4) return DT_INVALID;
  if (kprep) sh.need += align256((size_t)B * Skv * Hk * D * 2);
  if (Wo) sh.need += align256((size_t)B * Sq * Hq * D * 2);
  return DT_OK;
}

// Enqueue of a request that sdpa_validate() has accepted.  Calls nothing that allocates.
static dt_status sdpa_enqueue(dt_stream stream, int32_t B, int32_t Hq, int32_t Hk, int32_t D, int32_t n_qseg,
                              const dt_seq_segment* q_seg, int32_t n_kvseg, const dt_seq_segment* k_seg,
                              const dt_seq_segment* v_seg, const uint16_t* rot_q, const uint16_t* rot_k, float eps,
                              dt_view4 o, float scale, const uint16_t* Wo, const uint16_t* bo, void* workspace,
                              size_t workspace_bytes, const SdpaShape& sh) {
  const int64_t Sq = sh.Sq, Skv = sh.Skv;
  if (sh.empty) return DT_OK;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;

  if (sh.need > 0) {
    if (!workspace || workspace_bytes < sh.need) return DT_OOM;
    if (reinterpret_cast<uintptr_t>(workspace) & 255) return DT_INVALID;
  }
  hipStream_t s = as_stream(stream);
  uint8_t* ws = static_cast<uint8_t*>(workspace);

  SdpaArgs a = {};
  a.B = B;
  a.Hq = Hq;
  a.Hk = Hk;
  a.group = Hq / Hk;
  a.D = D;
  a.Sq = Sq;
  a.Skv = Skv;
  a.scale_log2e = scale * 1.44269504088896340736f;

  // Queries: read in place, segment by segment; their RMSNorm and rotation happen inside the attention kernel.
  {
    int64_t pos = 0;
    int n = 0;
    for (int i = 0; i < n_qseg; i++) {
      if (q_seg[i].len == 0) continue;
      const dt_view4& v = q_seg[i].view;
      a.q_gamma[n] = q_seg[i].gamma;
      a.q[n++] = SdpaSeg{static_cast<const uint16_t*>(v.ptr), v.stride_b, v.stride_s, v.stride_h, pos};
      pos += q_seg[i].len;
    }
    a.n_qseg = n;
    for (int i = n; i < kMaxSeg; i++) {
      a.q[i] = a.q[0];
      a.q_gamma[i] = a.q_gamma[0];
    }
    a.q_rot = rot_q;
    a.q_eps = eps;
    a.q_prep = sh.qprep ? 1 : 0;
  }
  // Keys: RMSNorm -> cmul staged into one contiguous copy when asked for (the kernel moves K tiles from memory
  // straight into LDS, so there is no register stage to do it in); otherwise read in place.  V is read in place.
  const bool kprep = sh.kprep;
  if (kprep) {
    uint16_t* kw = reinterpret_cast<uint16_t*>(ws);
    ws += align256((size_t)B * Skv * Hk * D * 2);
    int64_t pos = 0;
    for (int i = 0; i < n_kvseg; i++) {
      if (k_seg[i].len == 0) continue;
      QkPrepArgs p;
      p.src = static_cast<const uint16_t*>(k_seg[i].view.ptr);
      p.src_sb = k_seg[i].view.stride_b;
      p.src_ss = k_seg[i].view.stride_s;
      p.src_sh = k_seg[i].view.stride_h;
      p.dst = kw + pos * Hk * D;
      p.dst_sb = Skv * Hk * D;
      p.dst_ss = (int64_t)Hk * D;
      p.dst_sh = D;
      p.B = B;
      p.S = k_seg[i].len;
      p.H = Hk;
      p.D = D;
      p.gamma = k_seg[i].gamma;
      p.eps = eps;
      p.norm_per_head = 1;
      p.rot = rot_k;
      p.rot_pos0 = pos;
      p.post_scale = 1.0f;
      dt_status st = qk_prep_launch(s, p);
      if (st != DT_OK) return st;
      pos += k_seg[i].len;
    }
    a.n_kvseg = 1;
    a.k[0] = SdpaSeg{kw, Skv * Hk * D, (int64_t)Hk * D, D, 0};
    for (int i = 1; i < kMaxSeg; i++) a.k[i] = a.k[0];
  } else {
    int64_t pos = 0;
    int n = 0;
    for (int i = 0; i < n_kvseg; i++) {
      if (k_seg[i].len == 0) continue;
      const dt_view4& v = k_seg[i].view;
      a.k[n++] = SdpaSeg{static_cast<const uint16_t*>(v.ptr), v.stride_b, v.stride_s, v.stride_h, pos};
      pos += k_seg[i].len;
    }
    a.n_kvseg = n;
    for (int i = n; i < kMaxSeg; i++) a.k[i] = a.k[0];
  }
  {
    int64_t pos = 0;
    int n = 0;
    for (int i = 0; i < n_kvseg; i++) {
      if (v_seg[i].len == 0) continue;
      const dt_view4& v = v_seg[i].view;
      a.v[n++] = SdpaSeg{static_cast<const uint16_t*>(v.ptr), v.stride_b, v.stride_s, v.stride_h, pos};
      pos += v_seg[i].len;
    }
    for (int i = n; i < kMaxSeg; i++) a.v[i] = a.v[0];
    if (kprep && n > 1) {
      // K was staged as one segment; the V segments keep their own table
      a.n_kvseg = n;
      for (int i = 1; i < n; i++) {
        a.k[i] = a.k[0];
        a.k[i].start = a.v[i].start;
        a.k[i].ptr = a.k[0].ptr + a.v[i].start * a.k[0].ss;
      }
    }
  }

  // What is left of the workspace behind the staging buffers takes the key-split form's partial results, if the
  // launch is one that splitting helps and the room is there.
  auto plan_split = [&](uint8_t* free_ws) {
    SdpaSplit plan;
    if (!workspace || !sdpa_split_plan(B, Hq, D, Sq, Skv, &plan)) return;
    const size_t used = (size_t)(free_ws - static_cast<uint8_t*>(workspace));
    if (workspace_bytes < used + plan.bytes() || (reinterpret_cast<uintptr_t>(workspace) & 255)) return;
    a.counters = reinterpret_cast<int32_t*>(free_ws);
    a.partials = reinterpret_cast<float*>(free_ws + plan.counter_bytes);
    a.units = plan.units;
    a.split_workgroups = plan.workgroups;
  };
  if (Wo) {
    uint16_t* ow = reinterpret_cast<uint16_t*>(ws);
    ws += align256((size_t)B * Sq * Hq * D * 2);
    plan_split(ws);
    a.o = ow;
    a.o_sb = Sq * Hq * D;
    a.o_ss = (int64_t)Hq * D;
    a.o_sh = D;
    dt_status st = sdpa_launch(s, a);
    if (st != DT_OK) return st;
    // unify-heads projection on the staged attention output: one Dense over all batches when the output's
    // batches follow each other at the row stride, else batch by batch
    const int64_t HD = (int64_t)Hq * D;
    dt_qx_weight w{Wo, 16, 0, HD * HD};
    if (B > 1 && o.stride_b == Sq * o.stride_s) {
      const uint16_t* bias_arr[1] = {bo};
      uint16_t* y_arr[1] = {static_cast<uint16_t*>(o.ptr)};
      const int64_t ldy_arr[1] = {o.stride_s};
      return dt_dense_qx_f16(stream, (int64_t)B * Sq, HD, ow, HD, &w, 1, bias_arr, y_arr, ldy_arr, 0);
    }
    for (int b = 0; b < B; b++) {
      const uint16_t* bias_arr[1] = {bo};
      uint16_t* y_arr[1] = {static_cast<uint16_t*>(o.ptr) + b * o.stride_b};
      const int64_t ldy_arr[1] = {o.stride_s};
      st = dt_dense_qx_f16(stream, Sq, HD, ow + b * a.o_sb, HD, &w, 1, bias_arr, y_arr, ldy_arr, 0);
      if (st != DT_OK) return st;
    }
    return DT_OK;
  }
  plan_split(ws);
  a.o = static_cast<uint16_t*>(o.ptr);
  a.o_sb = o.stride_b;
  a.o_ss = o.stride_s;
  a.o_sh = o.stride_h;
  return sdpa_launch(s, a);
}

// ---- the library's own scratch, for callers that cannot allocate ------------------------------------------------
// One array per GPU (every device that loads this code object holds its own copy at its own address, until the
// process ends).  In host code the array's name is only a handle for hipGetSymbolAddress; the device address it
// yields -- looked up once per device, with that device current -- is what kernels and the host side use.
static __device__ __align__(256) unsigned char scratch[DT_SDPA_STATIC_SCRATCH_BYTES];

static std::atomic<void*> g_scratch_ptr[64];

// Device address of the calling thread's current device's array (nullptr on failure).
void* sdpa_static_scratch() {
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return nullptr;
  void* p = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!p) {
    void* q = nullptr;
    if (hipGetSymbolAddress(&q, HIP_SYMBOL(scratch)) != hipSuccess || !q) {
      (void)hipGetLastError();
      return nullptr;
    }
    g_scratch_ptr[dev].store(q, std::memory_order_release);
    p = q;
  }
  return p;
}

}  // namespace dt

DT_EXPORT dt_status dt_sdpa_f16(dt_stream stream, int32_t B, int32_t Hq, int32_t Hk, int32_t D, int32_t n_qseg,
                                const dt_seq_segment* q_seg, int32_t n_kvseg, const dt_seq_segment* k_seg,
                                const dt_seq_segment* v_seg, const uint16_t* rot_q, const uint16_t* rot_k, float eps,
                                dt_view4 o, float scale, const uint16_t* Wo, const uint16_t* bo, void* workspace,
                                size_t workspace_bytes) {
  dt::SdpaShape sh;
  if (const dt_status st = dt::sdpa_validate(B, Hq, Hk, D, n_qseg, q_seg, n_kvseg, k_seg, v_seg, rot_q, rot_k, o, Wo, sh);
      st != DT_OK)
    return st;
  return dt::sdpa_enqueue(stream, B, Hq, Hk, D, n_qseg, q_seg, n_kvseg, k_seg, v_seg, rot_q, rot_k, eps, o, scale, Wo,
                          bo, workspace, workspace_bytes, sh);
}

DT_EXPORT dt_status dt_sdpa_f16_static(dt_stream stream, int32_t B, int32_t Hq, int32_t Hk, int32_t D, int32_t n_qseg,
                                       const dt_seq_segment* q_seg, int32_t n_kvseg, const dt_seq_segment* k_seg,
                                       const dt_seq_segment* v_seg, const uint16_t* rot_q, const uint16_t* rot_k,
                                       float eps, dt_view4 o, float scale, const uint16_t* Wo, const uint16_t* bo) {
  using namespace dt;
  // the same argument checks as dt_sdpa_f16, in the same order, before the size of the request is looked at
  SdpaShape sh;
  if (const dt_status st = sdpa_validate(B, Hq, Hk, D, n_qseg, q_seg, n_kvseg, k_seg, v_seg, rot_q, rot_k, o, Wo, sh);
      st != DT_OK)
    return st;
  if (sh.empty) return DT_OK;
  if (sh.need > (size_t)DT_SDPA_STATIC_SCRATCH_BYTES) return DT_OOM;  // beyond the fixed array: use dt_sdpa_f16
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  // the staging bytes are a must; the key-split form's room is used if the array still has it
  size_t give = dt_sdpa_workspace_bytes(B, Hq, Hk, D, sh.Sq, sh.Skv, sh.kprep ? 1 : 0, Wo ? 1 : 0);
  if (give > (size_t)DT_SDPA_STATIC_SCRATCH_BYTES) give = sh.need;
  void* ws = nullptr;
  if (give > 0) {
    ws = sdpa_static_scratch();
    if (!ws) return DT_DEVICE_ERROR;
  }
  return sdpa_enqueue(stream, B, Hq, Hk, D, n_qseg, q_seg, n_kvseg, k_seg, v_seg, rot_q, rot_k, eps, o, scale, Wo, bo,
                      ws, give, sh);
}

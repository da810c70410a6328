// A compiled host program above the C ABI: the C++ operator objects of include/dt_hip.hpp (Dense over a plain and over a
// palettized weight, RMSNorm, ScaledDotProductAttention over two segments) on small inputs whose results are known in
// closed form.  Built by the Makefile next to the library; run by the GPU tests.  Prints "dt_cpp_check ok" and exits 0.
#include <hip/hip_runtime.h>

#include <cmath>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

#include "../../include/dt_hip.hpp"

static uint16_t h16(float f) {
  _Float16 h = (_Float16)f;
  uint16_t b;
  std::memcpy(&b, &h, 2);
  return b;
}
static float f32(uint16_t b) {
  _Float16 h;
  std::memcpy(&h, &b, 2);
  return (float)h;
}
#define HIP_OK(x)                                                         \
  do {                                                                    \
    if ((x) != hipSuccess) {                                              \
      std::fprintf(stderr, "%s failed at line %d\n", #x, __LINE__);       \
      return 1;                                                           \
    }                                                                     \
  } while (0)
#define REQUIRE(c)                                                        \
  do {                                                                    \
    if (!(c)) {                                                           \
      std::fprintf(stderr, "check failed at line %d: %s\n", __LINE__, #c); \
      return 1;                                                           \
    }                                                                     \
  } while (0)

template <class T>
static T* to_device(const std::vector<T>& v) {
  T* p = nullptr;
  if (hipMalloc(&p, v.size() * sizeof(T) + 256) != hipSuccess) return nullptr;
  if (hipMemcpy(p, v.data(), v.size() * sizeof(T), hipMemcpyHostToDevice) != hipSuccess) return nullptr;
  return p;
}

int main() {
  if (dt_init(0) != DT_OK) {
    std::fprintf(stderr, "device 0 is not a gfx950 part\n");
    return 1;
  }
  std::mt19937 rng(5);
  std::normal_distribution<float> gauss(0.f, 1.f);

  // ---- Dense, X = identity: Y = W^T exactly, for a plain fp16 weight and for a q8p weight (nib 64) --------------
  const int K = 64, N = 48, M = 64;
  std::vector<uint16_t> eye(M * K, h16(0.f));
  for (int i = 0; i < K; i++) eye[i * K + i] = h16(1.f);
  std::vector<uint16_t> wplain(N * K);
  for (auto& w : wplain) w = h16(gauss(rng));
  // q8p: per block of 64 elements, 256 fp16 palette entries followed by 64 index bytes
  const int nib = 64, nblocks = N * K / nib;
  std::vector<uint8_t> packed((size_t)nblocks * (512 + nib));
  std::vector<uint16_t> wq8(N * K);
  for (int b = 0; b < nblocks; b++) {
    uint8_t* blk = packed.data() + (size_t)b * (512 + nib);
    for (int e = 0; e < 256; e++) {
      const uint16_t v = h16(0.02f * gauss(rng));
      std::memcpy(blk + 2 * e, &v, 2);
    }
    for (int i = 0; i < nib; i++) {
      blk[512 + i] = (uint8_t)(rng() & 255);
      std::memcpy(&wq8[(size_t)b * nib + i], blk + 2 * blk[512 + i], 2);
    }
  }
  REQUIRE(dt_qx_bytes(8, nib, (int64_t)N * K) == (int64_t)packed.size());
  uint16_t* d_eye = to_device(eye);
  uint16_t* d_wplain = to_device(wplain);
  uint8_t* d_packed = to_device(packed);
  std::vector<uint16_t> bias_h(N);
  for (auto& b : bias_h) b = h16(0.f);
  uint16_t* d_bias = to_device(bias_h);
  uint16_t* d_y = nullptr;
  HIP_OK(hipMalloc(&d_y, (size_t)M * N * 2));
  REQUIRE(d_eye && d_wplain && d_packed && d_bias);
  for (int pass = 0; pass < 2; pass++) {
    dt::Dense dense(N, /*noBias=*/pass == 0, dt::Float16, pass == 0 ? "x_q" : "x_k");
    dense.weight = pass == 0 ? dt::QxTensor{d_wplain, 16, 0, N, K} : dt::QxTensor{d_packed, 8, nib, N, K};
    dense.bias = d_bias;
    dense(nullptr, dt::Matrix{d_eye, M, K, K}, dt::Matrix{d_y, M, N, N});
    std::vector<uint16_t> y((size_t)M * N);
    HIP_OK(hipMemcpy(y.data(), d_y, y.size() * 2, hipMemcpyDeviceToHost));
    const std::vector<uint16_t>& w = pass == 0 ? wplain : wq8;
    for (int m = 0; m < M; m++)
      for (int n = 0; n < N; n++) REQUIRE(y[(size_t)m * N + n] == w[(size_t)n * K + m]);
  }
  // a Dense whose weight is not loaded refuses, as the reference's would
  try {
    dt::Dense empty(N);
    empty(nullptr, dt::Matrix{d_eye, M, K, K}, dt::Matrix{d_y, M, N, N});
    REQUIRE(false);
  } catch (const std::runtime_error&) {
  }
  // a bad shape comes back as DT_INVALID from the library
  try {
    dt::Dense dense(N, true);
    dense.weight = dt::QxTensor{d_wplain, 16, 0, N, K};
    dense(nullptr, dt::Matrix{d_eye, M, K, K - 3}, dt::Matrix{d_y, M, N, N});  // row stride below the row length
    REQUIRE(false);
  } catch (const dt::Error& e) {
    REQUIRE(e.status == DT_INVALID);
  }

  // ---- RMSNorm(axis: [3]) on a constant row: y = sign(c) * gamma / sqrt(1 + eps / c^2) ------------------------------
  const int B = 1, S = 70, H = 2, D = 64;
  std::vector<uint16_t> xc((size_t)S * H * D, h16(-3.f)), gam(D);
  for (int d = 0; d < D; d++) gam[d] = h16(1.f + 0.01f * d);
  uint16_t* d_x = to_device(xc);
  uint16_t* d_g = to_device(gam);
  REQUIRE(d_x && d_g);
  dt::RMSNorm norm(1e-6f, {3}, "x_norm_q");
  norm.weight = d_g;
  norm(nullptr, dt_view4{d_x, (int64_t)S * H * D, (int64_t)H * D, D}, B, S, H, D);
  HIP_OK(hipMemcpy(xc.data(), d_x, xc.size() * 2, hipMemcpyDeviceToHost));
  for (int i = 0; i < S * H * D; i++) REQUIRE(std::fabs(f32(xc[i]) + f32(gam[i % D])) <= 2e-3f * f32(gam[i % D]));

  // ---- attention over two segments with V constant per head: every output row is that constant ---------------------
  const int T = 40, HW = 150, Hq = 2, Dh = 128;
  auto randn = [&](size_t n) {
    std::vector<uint16_t> v(n);
    for (auto& e : v) e = h16(gauss(rng));
    return v;
  };
  std::vector<uint16_t> vconst_c((size_t)T * Hq * Dh), vconst_x((size_t)HW * Hq * Dh);
  for (size_t i = 0; i < vconst_c.size(); i++) vconst_c[i] = h16(0.25f * (float)((i % (Hq * Dh)) % 7) - 0.5f);
  for (size_t i = 0; i < vconst_x.size(); i++) vconst_x[i] = h16(0.25f * (float)((i % (Hq * Dh)) % 7) - 0.5f);
  uint16_t *qc = to_device(randn((size_t)T * Hq * Dh)), *qx = to_device(randn((size_t)HW * Hq * Dh));
  uint16_t *kc = to_device(randn((size_t)T * Hq * Dh)), *kx = to_device(randn((size_t)HW * Hq * Dh));
  uint16_t *vc = to_device(vconst_c), *vx = to_device(vconst_x);
  uint16_t* d_o = nullptr;
  HIP_OK(hipMalloc(&d_o, (size_t)(T + HW) * Hq * Dh * 2));
  REQUIRE(qc && qx && kc && kx && vc && vx);
  auto view = [&](uint16_t* p, int64_t len) { return dt_view4{p, len * Hq * Dh, (int64_t)Hq * Dh, Dh}; };
  auto seg = [&](uint16_t* p, int64_t len) { return dt_seq_segment{view(p, len), len, nullptr}; };
  dt::ScaledDotProductAttention sdpa(1.0f / std::sqrt((float)Dh), false, false, dt::Float16);
  const size_t need = sdpa.workspaceBytes(1, Hq, Hq, Dh, T + HW, T + HW);
  void* ws = nullptr;
  if (need) HIP_OK(hipMalloc(&ws, need));
  sdpa(nullptr, 1, Hq, Hq, Dh, {seg(qc, T), seg(qx, HW)}, {seg(kc, T), seg(kx, HW)}, {seg(vc, T), seg(vx, HW)},
       view(d_o, T + HW), ws, need);
  HIP_OK(hipDeviceSynchronize());
  std::vector<uint16_t> o((size_t)(T + HW) * Hq * Dh);
  HIP_OK(hipMemcpy(o.data(), d_o, o.size() * 2, hipMemcpyDeviceToHost));
  for (size_t i = 0; i < o.size(); i++) REQUIRE(std::fabs(f32(o[i]) - f32(vconst_c[i % (Hq * Dh)])) <= 2e-3f);
  // masks are not part of this path: the constructor refuses, as a backend without that kernel would
  try {
    dt::ScaledDotProductAttention causal(1.f, /*isCausal=*/true);
    REQUIRE(false);
  } catch (const dt::Error& e) {
    REQUIRE(e.status == DT_NO_KERNEL);
  }
  REQUIRE(dt::DenseInstructionCount(4608, 3072, 3072) == 4608LL * 3072 * 3072);
  REQUIRE(dt::ScaledDotProductAttentionInstructionCount(1, 24, 128, 4608, 4608) == 24LL * 261 * 4608 * 4608);
  std::printf("dt_cpp_check ok: %s\n", dt_version());
  return 0;
}

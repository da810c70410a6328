// The low-rank branch of a LoRADense in high precision: up(scale * down(float(x))) with fp32 weights, fp32
// intermediate and fp32 accumulation, rounded to fp16 once at the end (Models/LoRA.swift:117-139, highPrecision:
// `denseDown(x.to(.Float32))`, `denseUp(scale * downX).to(of: x)`).  Two small GEMMs (the rank is 8 .. 128) on the
// fp32 matrix instruction; the base projection's epilogue then adds the branch as its `addend`.
#include "dt_common.h"

namespace dt {

typedef float float16v __attribute__((ext_vector_type(16)));

// C[M, N] = alpha * A[M, K] B[N, K]^T, fp32 accumulate.  A fp16 or fp32, B fp32, C fp32 or fp16.
// 64 x 64 outputs per 256-thread workgroup, a 32 x 32 block per wave (v_mfma_f32_32x32x2_f32), K in steps of 16
// through LDS.  Any shape: rows and columns past the edge are read as zero and not written.
template <bool A_HALF, bool C_HALF>
__global__ void __launch_bounds__(256) gemm_nt_f32_kernel(int64_t M, int64_t N, int64_t K, const void* Ap, int64_t lda,
                                                          const float* B, int64_t ldb, void* Cp, int64_t ldc, float alpha) {
  constexpr int BK = 16, PAD = BK + 1;
  __shared__ float As[64 * PAD];
  __shared__ float Bs[64 * PAD];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, hi = lane >> 5;
  const int wm = wave & 1, wn = wave >> 1;
  const int64_t m0 = (int64_t)blockIdx.x * 64, n0 = (int64_t)blockIdx.y * 64;
  const int lr = tid >> 2, lc = (tid & 3) * 4;  // this thread stages 4 consecutive k of one row of each tile
  float16v acc;
#pragma unroll
  for (int v = 0; v < 16; v++) acc[v] = 0.f;
  for (int64_t k0 = 0; k0 < K; k0 += BK) {
    float a4[4] = {0.f, 0.f, 0.f, 0.f}, b4[4] = {0.f, 0.f, 0.f, 0.f};
    const int64_t am = m0 + lr, bn = n0 + lr;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      const int64_t k = k0 + lc + e;
      if (k < K) {
        if (am < M) {
          if constexpr (A_HALF) a4[e] = (float)bits_to_half(static_cast<const uint16_t*>(Ap)[am * lda + k]);
          else a4[e] = static_cast<const float*>(Ap)[am * lda + k];
        }
        if (bn < N) b4[e] = B[bn * ldb + k];
      }
    }
    __syncthreads();  // the previous step's reads are done
#pragma unroll
    for (int e = 0; e < 4; e++) {
      As[lr * PAD + lc + e] = a4[e];
      Bs[lr * PAD + lc + e] = b4[e];
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK / 2; kk++) {
      const float a = As[(wm * 32 + l32) * PAD + 2 * kk + hi];
      const float b = Bs[(wn * 32 + l32) * PAD + 2 * kk + hi];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
  }
  // lane holds column n = l32 of the block and rows m = 8 (v / 4) + 4 hi + v % 4
  const int64_t n = n0 + wn * 32 + l32;
  if (n >= N) return;
#pragma unroll
  for (int v = 0; v < 16; v++) {
    const int64_t m = m0 + wm * 32 + 8 * (v >> 2) + 4 * hi + (v & 3);
    if (m >= M) continue;
    float r = acc[v] * alpha;
    asm volatile("" : "+v"(r));  // the scale is its own fp32 multiplication, as in the graph
    if constexpr (C_HALF) static_cast<uint16_t*>(Cp)[m * ldc + n] = half_to_bits((half_t)r);
    else static_cast<float*>(Cp)[m * ldc + n] = r;
  }
}

}  // namespace dt

DT_EXPORT dt_status dt_lora_branch_f32_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                           const float* down, int32_t rank, const float* up, int64_t N, float scale,
                                           float* T, uint16_t* out, int64_t ldo) {
  using namespace dt;
  if (M < 0 || K <= 0 || rank <= 0 || N <= 0 || !down || !up) return DT_INVALID;
  if (M == 0) return DT_OK;
  if (!X || !T || !out || ldx < K || ldo < N) return DT_INVALID;
  if ((reinterpret_cast<uintptr_t>(X) & 1) || (reinterpret_cast<uintptr_t>(out) & 1) || (reinterpret_cast<uintptr_t>(T) & 3) ||
      (reinterpret_cast<uintptr_t>(down) & 3) || (reinterpret_cast<uintptr_t>(up) & 3))
    return DT_INVALID;
  if (!(scale == scale) || scale - scale != 0.f) return DT_INVALID;
  if ((M + 63) / 64 > 0x7fffffff || (N + 63) / 64 > 65535) return DT_NO_KERNEL;
  if (const dt_status ready = device_ready(); ready != DT_OK) return ready;
  hipStream_t s = as_stream(stream);
  // T = scale * float(X) down^T  [M, rank]
  hipLaunchKernelGGL((gemm_nt_f32_kernel<true, false>), dim3((unsigned)((M + 63) / 64), (unsigned)((rank + 63) / 64)), dim3(256), 0,
                     s, M, (int64_t)rank, K, X, ldx, down, K, T, (int64_t)rank, scale);
  dt_status st = launch_status();
  if (st != DT_OK) return st;
  // out = fp16(T up^T)  [M, N]
  hipLaunchKernelGGL((gemm_nt_f32_kernel<false, true>), dim3((unsigned)((M + 63) / 64), (unsigned)((N + 63) / 64)), dim3(256), 0, s,
                     M, N, (int64_t)rank, T, (int64_t)rank, up, (int64_t)rank, out, ldo, 1.0f);
  return launch_status();
}

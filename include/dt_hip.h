/*
 * dt_hip.h -- C ABI of the MI355X (gfx950) transformer-block hot path:
 * Dense over palettized weights and ScaledDotProductAttention, plus the two
 * small ops fused around them (per-head / per-row RMSNorm and the RoPE cmul).
 *
 * Plain C, no C++ or framework types cross this boundary.  Every pointer is a
 * DEVICE pointer borrowed for the duration of the enqueue (the call returns
 * once the work is queued on `stream`; it never synchronises the stream).
 * All entry points are re-entrant and stream-ordered; the library keeps no
 * mutable global state apart from a once-per-device architecture query.
 *
 * Status codes mirror the values a ccv_nnc backend `exec` returns, so a shim
 * can map DT_NO_KERNEL to "fall through to the next backend":
 *    0  DT_OK          work enqueued
 *   -1  DT_INVALID     bad shape / alignment / NULL pointer / unknown qbits
 *   -2  DT_NO_KERNEL   valid request this library has no kernel for
 *   -3  DT_OOM         workspace too small
 *   -4  DT_DEVICE_ERROR the HIP runtime already reported a fault when the call was made (a faulted kernel, a lost
 *                      device or context: left in place for its owner; nothing was enqueued), or the device failed
 *                      under the launch; no ccv counterpart: a shim maps it to CCV_NNC_EXEC_INVALID.  A stale
 *                      non-fatal code in the calling thread's error slot (hipErrorInvalidValue of a pointer probe,
 *                      hipErrorPeerAccessAlreadyEnabled, hipErrorNotSupported, ...) does not refuse the call: the
 *                      call that produced it has returned it already, and the entry point clears it
 *
 * The operator surface this replaces is the one the reference's model
 * builders call (reference paths relative to Libraries/SwiftDiffusion/Sources):
 *   Dense(count:noBias:flags:name:)                 Models/Flux1.swift:161-176, 237-245
 *   RMSNorm(epsilon:axis:name:)                     Models/Flux1.swift:165-182, Models/Wan.swift:87-91
 *   Functional.cmul(left:right:)                    Models/Flux1.swift:187-188, Models/Wan.swift:93-94
 *   ScaledDotProductAttention(scale:flags:multiHeadOutputProjectionFused:)
 *                                                   Models/Flux1.swift:228-232, Models/UNet.swift:122-155
 *   store.read(_, codec:[.q4p/.q5p/.q6p/.q8p, .jit]) Models/UNetProtocol.swift:2230-2233, 2370-2373
 */
#ifndef DT_HIP_H
#define DT_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int32_t dt_status;
#define DT_OK 0
#define DT_INVALID (-1)
#define DT_NO_KERNEL (-2)
#define DT_OOM (-3)
#define DT_DEVICE_ERROR (-4)

/* A hipStream_t passed as an opaque pointer; NULL is the default stream. */
typedef void* dt_stream;

/*
 * A weight as store.read(codec: [.jit, .q?p]) leaves it on the device
 * (Models/UNetProtocol.swift:2230-2233): still palettized.
 *   data  : packed buffer, 16-byte aligned
 *   qbits : 4, 5, 6, 7 or 8 -> per block of `nib` elements (flattened row-major
 *           [out, in] order), 2^qbits fp16 palette entries followed by that
 *           block's indices bit-packed MSB-first;
 *           16 -> plain fp16 [out, in] weight (nib ignored)
 *   nib   : elements per palette block
 *   count : number of elements = out * in
 */
typedef struct {
  const void* data;
  int32_t qbits;
  int32_t nib;
  int64_t count;
} dt_qx_weight;

/* [B, S, H, D] fp16 view, D contiguous; strides in elements. */
typedef struct {
  void* ptr;
  int64_t stride_b;
  int64_t stride_s;
  int64_t stride_h;
} dt_view4;

/* One run of consecutive sequence positions.  A joint text||image sequence
 * (Functional.concat(axis: 1, contextK, xK), Models/Flux1.swift:184-186) is
 * passed as two segments instead of a materialised concatenation.
 *   gamma : per-head RMSNorm weight [D] applied to this segment's rows before
 *           attention (c_norm_q / x_norm_q differ per segment,
 *           Models/Flux1.swift:165-182); NULL = no norm */
typedef struct {
  dt_view4 view;
  int64_t len;
  const uint16_t* gamma;
} dt_seq_segment;

/* Library identification; never NULL. */
const char* dt_version(void);

/* Makes `device` the calling thread's current device, checks that it is a gfx950 part and warms the per-device
 * query.  Optional: every entry point does the same check lazily for whichever device is current.
 * Returns DT_NO_KERNEL on any other architecture. */
dt_status dt_init(int device);

/* Bytes a palettized tensor of `count` elements occupies, palettes included;
 * -1 for an unsupported (qbits, nib). */
int64_t dt_qx_bytes(int32_t qbits, int32_t nib, int64_t count);

/*
 * out[i] = palette[i / nib][index[i]]  -- the tensor a CPU read of the same
 * key yields (store.read(name, kind: .CPU, codec: [.q6p, .q8p, ...]) followed
 * by Tensor<FloatType>(from:), LoRALoader.swift:317).  Bit-exact.
 * out: `count` fp16 values, 2-byte aligned.
 */
dt_status dt_depalettize_f16(dt_stream stream, const dt_qx_weight* w, uint16_t* out);

/*
 * Dense: Y = X W^T (+ bias), X [M, K] fp16 with row stride ldx, each W_i
 * [N_i, K] (N_i = count_i / K), Y_i [M, N_i] fp16 with row stride ldy[i];
 * fp32 accumulation, one rounding to fp16.  n_weights > 1 runs several Dense
 * ops that share X in one launch (x_q / x_k / x_v, Models/Flux1.swift:174-176).
 * The palettized weight is unpacked and looked up on chip; no dequantized
 * copy is written to memory.
 *   bias  : array of n_weights pointers, entries may be NULL (noBias: true);
 *           the array itself may be NULL when no weight has a bias
 *   flags : bit 0 = caller allows fp16 accumulation (Functional.GEMMFlag
 *           .Float16, Models/Flux1.swift:162); accepted and ignored
 * The arrays W / bias / Y / ldy are HOST arrays of n_weights entries.
 */
dt_status dt_dense_qx_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                          const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                          uint16_t* const* Y, const int64_t* ldy, uint32_t flags);

/*
 * Dense with the per-head RMSNorm and the RoPE rotation that follow it in the
 * attention blocks fused into the GEMM epilogue (Dense -> reshaped([b, s, h, k])
 * -> RMSNorm(axis: [3]) -> cmul(rot), Models/Flux1.swift:174-188): Q and K leave
 * the projection already normalised and rotated, with no extra pass over them.
 * epi: HOST array of n_weights entries, or NULL (then identical to
 * dt_dense_qx_f16).  An entry with gamma == NULL and rot == NULL leaves that
 * weight's output plain (x_v).  Each output row is treated as heads of
 * `head_dim` features; rounding happens after the Dense, after the norm and
 * after the rotation, exactly as the three separate ops round.
 *   gamma    : RMSNorm weight [head_dim] (x_norm_q / x_norm_k), or NULL
 *   eps      : RMSNorm epsilon
 *   rot      : [>= rot_pos0 + M, head_dim] fp16 table of interleaved (cos, sin), or NULL
 *   rot_pos0 : table row of X's first row (offset of this stream in the joint sequence)
 *   head_dim : 128 runs inside the GEMM epilogue; other even values <= 128 run
 *              as a separate pass after the GEMM (same results)
 */
typedef struct {
  const uint16_t* gamma;
  const uint16_t* rot;
  int64_t rot_pos0;
  float eps;
  int32_t head_dim;
} dt_head_epilogue;

dt_status dt_dense_qx_heads_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                                uint16_t* const* Y, const int64_t* ldy, const dt_head_epilogue* epi,
                                uint32_t flags);

/*
 * Dense followed by the elementwise tail of the feed-forward and residual paths
 * of a transformer block, applied in the GEMM epilogue in this order, each step
 * rounding to fp16 as the separate ops do:
 *   scale      : scalar multiplier of the result; 0 or 1 = none (configuration.scale * downX, Models/LoRA.swift:129-134)
 *   addend     : fp16 [M, N_i] with row stride ld_addend, added to the result: the low-rank branch of a
 *                LoRADense, out = dense(x) + up(down(x)) (Models/LoRA.swift:117-140); may be Y[i] itself (in place)
 *   multiplicand : fp16 [M, N_i] with row stride ld_multiplicand, multiplies the result elementwise: the gated
 *                feed-forward fc10(x) .* GELU()(fc11(x)) (Models/UNet.swift:510-513); may be Y[i] itself
 *   activation : DT_ACT_GELU_TANH  linear1(x).GELU(approximate: .tanh)  (Models/Flux1.swift:133-135, Models/Wan.swift:52-53)
 *                DT_ACT_SWISH      fc0(x).swish()                       (Models/Flux1.swift:122-123)
 *                DT_ACT_GELU_ERF   GELU()(fc11(x)), the erf form          (Models/UNet.swift:513)
 *   gate       : [N_i] fp16, multiplies every output row ((xOut .* xChunks[2]), Models/Flux1.swift:246-250)
 *   residual   : fp32 [M, N_i] with row stride ld_residual, updated in place:
 *                residual += float(result)  (x + (...).to(of: x), Models/Flux1.swift:250, 275-283)
 *   gate_f32   : [N_i] fp32, needs residual, excludes gate: residual += float(result) * gate_f32, the product
 *                formed in fp32 (x + out.to(of: x) .* chunks[2], Models/Wan.swift:159, 220-221); Y[i], if given,
 *                receives the result before the gate
 * post: HOST array of n_weights entries (NULL = plain dt_dense_qx_f16).  Y[i] may
 * be NULL when post[i].residual is given (the result is only accumulated).
 * Concurrent calls must not share a residual tensor.
 */
#define DT_ACT_NONE 0
#define DT_ACT_GELU_TANH 1
#define DT_ACT_SWISH 2
#define DT_ACT_GELU_ERF 3

typedef struct {
  int32_t activation;
  const uint16_t* gate;
  float* residual;
  int64_t ld_residual;
  float scale;
  const uint16_t* addend;
  int64_t ld_addend;
  const float* gate_f32;
  const uint16_t* multiplicand;
  int64_t ld_multiplicand;
} dt_dense_post;

dt_status dt_dense_qx_post_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                               const dt_qx_weight* W, int32_t n_weights, const uint16_t* const* bias,
                               uint16_t* const* Y, const int64_t* ldy, const dt_dense_post* post,
                               uint32_t flags);

/*
 * LayerNorm(epsilon:, axis: [last], elementwiseAffine: false) of the fp32
 * residual stream followed by the adaLN modulation and the cast to fp16: the
 * op in front of the attention and feed-forward Dense layers of a DiT block.
 *   DT_MOD_F16 : y = fp16(fp16(fp16(norm(x)) * scale) + shift), scale / shift fp16 [C]
 *                (xNorm1(x).to(.Float16) .* xChunks[1] + xChunks[0], Models/Flux1.swift:172-173, 281-282)
 *   DT_MOD_F32 : y = fp16(norm(x) * (scale + 1) + shift), scale / shift fp32 [C]
 *                ((xNorm2(out) .* (chunks[4] + 1) + chunks[3]).to(.Float16), Models/Wan.swift:217-221)
 *   DT_MOD_AFFINE_F32 : y = fp16(norm(x) * scale + shift), scale / shift fp32 [C]: LayerNorm with its
 *                elementwise affine weight and bias (xNorm3(out).to(.Float16), Models/Wan.swift:160-161)
 * norm(x) = (x - mean) / sqrt(var + eps) with the biased variance, in fp32.
 * X: [M, C] fp32 with row stride ldx; Y: [M, C] fp16 with row stride ldy; scale
 * and shift are broadcast over rows and may be NULL.  Rows that are 16-byte
 * aligned with C % 4 == 0 and C <= 8192 stay in registers (one read, one write);
 * anything else takes a three-pass kernel with the same results.
 */
/*
 * LayerNorm(epsilon:, axis: [last]) with its elementwise affine weight and bias on an fp16 tensor, fp16 out:
 * the norms of a UNet transformer block (LayerNorm(epsilon: 1e-5, axis: [2]), Models/UNet.swift:530, 544, 554).
 * Statistics and the affine step in fp32, one rounding at the end.  gamma / beta: fp16 [C], may be NULL.
 * Y may be X (in place).
 */
dt_status dt_layernorm_f16(dt_stream stream, int64_t M, int64_t C, const uint16_t* X, int64_t ldx,
                           const uint16_t* gamma, const uint16_t* beta, float eps, uint16_t* Y, int64_t ldy);

#define DT_MOD_F16 0
#define DT_MOD_F32 1
#define DT_MOD_AFFINE_F32 2

dt_status dt_layernorm_modulate_f16(dt_stream stream, int64_t M, int64_t C, const float* X, int64_t ldx,
                                    const void* scale, const void* shift, int32_t mod, float eps,
                                    uint16_t* Y, int64_t ldy);

/*
 * The low-rank branch of a LoRADense in high precision (LoRANetworkConfiguration.highPrecision,
 * Models/LoRA.swift:117-139): out = fp16(up(scale * down(float(x)))) with fp32 weights, an fp32 intermediate and
 * fp32 accumulation -- `denseDown(x.to(.Float32))`, `denseUp(configuration.scale * downX).to(of: x)`.  The caller
 * adds it to the base projection through dt_dense_post.addend (out = dense(x) + branch).
 *   X    : [M, K] fp16, row stride ldx          down : [rank, K] fp32        up : [N, rank] fp32
 *   T    : scratch for the intermediate, [M, rank] fp32
 *   out  : [M, N] fp16, row stride ldo
 */
dt_status dt_lora_branch_f32_f16(dt_stream stream, int64_t M, int64_t K, const uint16_t* X, int64_t ldx,
                                 const float* down, int32_t rank, const float* up, int64_t N, float scale,
                                 float* T, uint16_t* out, int64_t ldo);

/*
 * Several independent Dense problems (each an X with its weights, arguments as
 * for dt_dense_qx_heads_f16) enqueued together.  The context (text) and image
 * streams of a joint block apply different weights to different token sets
 * (c_q / c_k / c_v and x_q / x_k / x_v, Models/Flux1.swift:161-176; c_o and
 * x_o, 237-245); run as one launch the short text problem fills the compute
 * units that the image problem's last round of tiles leaves idle.  Problems
 * that share K and the weight format and meet the alignment of the tiled
 * kernel go out in a single launch; anything else runs problem by problem with
 * the same results.  Outputs of different problems must not overlap.
 * `groups` is a HOST array.
 */
typedef struct {
  int64_t M, K;
  const uint16_t* X;
  int64_t ldx;
  const dt_qx_weight* W;
  int32_t n_weights;
  const uint16_t* const* bias;
  uint16_t* const* Y;
  const int64_t* ldy;
  const dt_head_epilogue* epi;  /* as for dt_dense_qx_heads_f16, or NULL */
  const dt_dense_post* post;    /* as for dt_dense_qx_post_f16, or NULL; a problem has at most one of epi and post */
} dt_dense_group;

dt_status dt_dense_qx_grouped_f16(dt_stream stream, int32_t n_groups, const dt_dense_group* groups,
                                  uint32_t flags);

/*
 * In place on a [B, S, H, D] view: optional RMSNorm, then optional RoPE.
 *   gamma       : RMSNorm weight, [D] when norm_per_head != 0 (Flux:
 *                 RMSNorm(axis: [3]), Models/Flux1.swift:165), [H*D] when 0
 *                 (Wan: RMSNorm(axis: [2]) over the whole row before the head
 *                 split, Models/Wan.swift:87-91; needs stride_h == D); NULL = skip
 *   rot         : [>= rot_pos0 + S, D] fp16 table of interleaved (cos, sin)
 *                 pairs, row stride D, broadcast over batch and heads
 *                 (Functional.cmul, Models/Flux1.swift:187-188); NULL = skip
 *   rot_pos0    : table row of this view's first position (a segment of a
 *                 joint sequence starts at its offset in the joint order)
 *   post_scale  : multiplies the result (Wan's .scale1 convention scales Q and
 *                 K by D^-1/4, Models/Wan.swift:95-98); 1.0f = none
 * Rounds to fp16 after the norm, after the rotation and after the scale, as
 * the op-by-op graph does.
 */
dt_status dt_qk_norm_rope_f16(dt_stream stream, dt_view4 x, int32_t B, int64_t S, int32_t H,
                              int32_t D, const uint16_t* gamma, float eps, int32_t norm_per_head,
                              const uint16_t* rot, int64_t rot_pos0, float post_scale);

/*
 * O = softmax(scale * Q K^T) V per (batch, head); non-causal, no mask.
 *   Q rows  : concatenation of n_qseg segments (each [B, len, Hq, D])
 *   K/V rows: concatenation of n_kvseg segments (each [B, len, Hk, D]);
 *             k_seg[i].len must equal v_seg[i].len; Hk divides Hq
 *   rot_q / rot_k : optional RoPE tables [total rows, D] indexed by position
 *             in the joint order; together with the segments' gamma this is
 *             the fused form of RMSNorm -> concat -> cmul -> attention
 *             (Models/Flux1.swift:165-188, 228-232); v_seg[i].gamma is ignored
 *   o       : [B, total Q rows, Hq, D]; when Wo != NULL the unify-heads
 *             projection is fused (multiHeadOutputProjectionFused: true,
 *             Models/UNet.swift:143-155): o is then [B, Sq, Hq*D] written with
 *             o.stride_s as row stride (stride_h unused), Wo fp16 [Hq*D, Hq*D]
 *             in [out, in] order, bo [Hq*D] or NULL
 *   workspace : device scratch, 256-byte aligned; may be NULL when nothing is
 *             staged.  dt_sdpa_workspace_bytes(...) is the staging this call
 *             cannot run without (fused_prep / fused_out_proj; less than that
 *             is DT_OOM) plus, for launches that would occupy well under one
 *             round of the card's compute units, room for the key-split form of
 *             the kernel (each task's key tiles shared out over several
 *             workgroups, fp32 partial results folded in a fixed order by the
 *             piece that finishes last).  Given only the staging part, or
 *             nothing, such a launch runs unsplit: same results to within one
 *             rounding of the fp16 output, lower occupancy.
 *             Environment: DT_SDPA_KEY_SPLIT=never|always overrides the
 *             estimate (read at every call; for tests and measurements).
 * D in {40, 64, 128} (any D <= 128 that is a multiple of 8).
 * Inputs are expected to be finite.  A key whose V row holds Inf or NaN makes the output rows of its (batch, head)
 * non-finite, as in the reference (probability x Inf, and 0 x Inf = NaN where the probability underflows); it
 * reaches no other (batch, head), and the unused rows of the ragged last key tile are zeroed rather than left holding
 * an earlier tile's values.  Non-finite Q / K scores behave as in the reference (the row's output is NaN).
 */
dt_status dt_sdpa_f16(dt_stream stream, int32_t B, int32_t Hq, int32_t Hk, int32_t D,
                      int32_t n_qseg, const dt_seq_segment* q_seg, int32_t n_kvseg,
                      const dt_seq_segment* k_seg, const dt_seq_segment* v_seg,
                      const uint16_t* rot_q, const uint16_t* rot_k, float eps, dt_view4 o,
                      float scale, const uint16_t* Wo, const uint16_t* bo, void* workspace,
                      size_t workspace_bytes);

/* Scratch for dt_sdpa_f16: room for the normalised / rotated copy of K when
 * `fused_prep` != 0 (any gamma or rot given; the queries are normalised and
 * rotated inside the attention kernel and need none), for the attention output
 * when `fused_out_proj` != 0, and -- optional, see `workspace` above -- for the
 * key-split form's partial results on the calling thread's current device. */
size_t dt_sdpa_workspace_bytes(int32_t B, int32_t Hq, int32_t Hk, int32_t D, int64_t Sq,
                               int64_t Skv, int32_t fused_prep, int32_t fused_out_proj);

/*
 * dt_sdpa_f16 with the library's own scratch instead of a caller's workspace.  No counterpart in the reference:
 * it exists for callers that cannot allocate device memory around the call -- code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc.  Same arguments, validation, kernels and results as dt_sdpa_f16;
 * it calls nothing that allocates or frees.
 *   The scratch is one fixed array of DT_SDPA_STATIC_SCRATCH_BYTES per GPU, resident on every GPU the library runs
 *   on until the process ends (its device address is looked up once per device, by dt_init or by the first call
 *   with that device current).  A request whose staging exceeds it returns DT_OOM and enqueues nothing: use
 *   dt_sdpa_f16 with a workspace of the caller's then.  (The optional key-split room is used when the array still
 *   has it, exactly as dt_sdpa_f16 uses a workspace of dt_sdpa_workspace_bytes().)  The limit covers the staged K of a joint
 *   sequence of 4608 tokens x 24 heads x 128 with fused QK-norm / RoPE (28.3 MB; up to ~10900 such tokens) and the
 *   fused unify-heads staging of SD 1.5 (5.2 MB).
 *   All calls on one GPU share that GPU's array, whose contents are whatever the last call left (every byte a
 *   call reads it has written first): calls that may overlap in time on one GPU -- different streams, or different
 *   threads -- race on it and must be ordered by the caller.  Calls on one stream are ordered by the stream.
 */
#define DT_SDPA_STATIC_SCRATCH_BYTES (64u << 20)

dt_status dt_sdpa_f16_static(dt_stream stream, int32_t B, int32_t Hq, int32_t Hk, int32_t D,
                             int32_t n_qseg, const dt_seq_segment* q_seg, int32_t n_kvseg,
                             const dt_seq_segment* k_seg, const dt_seq_segment* v_seg,
                             const uint16_t* rot_q, const uint16_t* rot_k, float eps, dt_view4 o,
                             float scale, const uint16_t* Wo, const uint16_t* bo);

#ifdef __cplusplus
}
#endif
#endif /* DT_HIP_H */

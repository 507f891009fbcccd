/*
 * tf_kernels.h — C ABI of the MI355X (gfx950) implementation of TurboFieldfare's
 * quantized MoE matmul path.
 *
 * Each entry point replaces one `encode(...)` method of the reference's Swift
 * kernel wrappers (Sources/TurboFieldfare/Kernels/ **), cited per declaration as
 * file:line relative to the reference checkout.  Conventions carried over:
 *
 *   - a tensor argument is (device pointer, byte offset), the analogue of the
 *     reference's (MTLBuffer, offset) pairs (DequantInt4GEMV.swift:44-56);
 *   - weights, scales and biases of one matrix are three offsets, usually into
 *     the same allocation (Infrastructure/ModelIO/ModelTypes.swift:164-192);
 *   - int4 weights: byte k of a row holds element 2k in its low nibble and 2k+1
 *     in its high nibble; one (scale, bias) pair per 64 consecutive elements of
 *     the reduction dimension, row-major [rows, cols/64]
 *     (Metal/Quant/dequant_int4.metal:7-12);  w = float(q) * scale + bias;
 *   - scales/biases are BF16 in the reference; TF_FP16 selects IEEE half instead;
 *   - alignment contract: packed-weight offsets even, everything else 2-byte
 *     aligned (DequantInt4GEMV.swift:57-62); 16-byte aligned operands take the
 *     vector path, anything else a slower path with identical results;
 *   - calls only enqueue work on `stream` (one in-order stream = the reference's
 *     command queue); nothing blocks except tf_stream_synchronize;
 *   - the caller owns every buffer; the library never frees caller memory;
 *   - where the reference traps on a broken precondition or throws, the call
 *     returns a negative tf_status and enqueues nothing.
 *
 * A tf_ctx is thread-compatible, not thread-safe (one encoder per runner in the
 * reference, RealForwardRunner.swift:229-377).
 */
#ifndef TF_KERNELS_H
#define TF_KERNELS_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TF_GROUP_SIZE 64u          /* Quantization.swift:5 */
#define TF_MAX_STREAMED_EXPERTS 8u /* MoE.swift:32 */
#define TF_MAX_TILE_EXPERTS 16u    /* PrefillMoEGrouping.swift:107 */

typedef struct tf_ctx tf_ctx;
typedef void *tf_stream; /* hipStream_t; NULL = the default stream */

typedef enum tf_status {
    TF_OK = 0,
    TF_ERR_INVALID_ARGUMENT = -1,  /* a `precondition` of the reference wrapper failed */
    TF_ERR_UNAVAILABLE = -2,       /* MPPPrefillInt4QMM.Path.unavailable (MPPPrefillInt4QMM.swift:5-8) */
    TF_ERR_DIMENSION_MISMATCH = -3,/* SharedExpertError.dimensionMismatch (SharedExpertInt4.swift:4-19) */
    TF_ERR_SCRATCH_TOO_SMALL = -4, /* SharedExpertError.scratchTooSmall */
    TF_ERR_UNSUPPORTED_BITS = -5,  /* SharedExpertError.unsupportedWeightBits */
    TF_ERR_NO_DEVICE = -6,         /* MetalError.noDevice (MetalContext.swift:4-20) */
    TF_ERR_DEVICE = -7,            /* a HIP call failed; see tf_last_error */
    TF_ERR_OUT_OF_MEMORY = -8
} tf_status;

typedef enum tf_dtype {
    TF_BF16 = 0, /* reference-exact scale/bias type */
    TF_FP16 = 1,
    TF_FP32 = 2
} tf_dtype;

/* MoEExpertOffsets (MoE.swift:4-29) == ExpertOffsets (Metal/MoE/moe.metal:62-72): byte offsets of the nine
 * sub-tensors inside one routed-expert blob, identical for all experts of a layer. 36 bytes. */
typedef struct tf_expert_offsets {
    uint32_t gate_W_off, gate_s_off, gate_b_off;
    uint32_t up_W_off, up_s_off, up_b_off;
    uint32_t down_W_off, down_s_off, down_b_off;
} tf_expert_offsets;

/* SharedExpertProjection (SharedExpertInt8.swift:9-31). */
typedef struct tf_projection {
    const void *weights; uint64_t weights_offset;
    const void *scales;  uint64_t scales_offset;
    const void *biases;  uint64_t biases_offset;
    uint32_t rows, cols;
} tf_projection;

/* Where the routed expert blobs of one layer live.  Either
 *   (a) blobs[0..7]: eight device pointers chosen by the host — the reference's argument buffer
 *       (MoE.swift:161-178, moe.metal:74-76), `indices` NULL; or
 *   (b) resident pool: expert e starts at pool + e * pool_stride and `indices` is a DEVICE array of top_k
 *       expert ids (what tf_router_gemma4 wrote), read by the kernels themselves: no host round trip.
 *       Ids >= num_experts are clamped to num_experts - 1 (RealForwardRunner.swift:1486). */
typedef struct tf_routed_blobs {
    const void *blobs[TF_MAX_STREAMED_EXPERTS];
    const void *pool;
    uint64_t pool_stride;
    const uint32_t *indices;
    uint32_t num_experts;
} tf_routed_blobs;

/* ---- context ------------------------------------------------------------------------------------- */
/* MetalContext.init (Infrastructure/Metal/MetalContext.swift:51-125): binds a device and allocates the
 * wrapper-owned scratch the reference's kernel classes own (router logits: MoE.swift:92-99; lm_head xNormed
 * and row summaries: LMHeadChainInt4.swift:38-51). */
int32_t tf_ctx_create(int32_t device, tf_ctx **out_ctx);
void tf_ctx_destroy(tf_ctx *ctx);
/* commandBuffer.waitUntilCompleted + checkCommandBufferError (MetalContext.swift:22-26): returns TF_ERR_DEVICE if
 * anything enqueued on the stream failed. */
int32_t tf_stream_synchronize(tf_ctx *ctx, tf_stream stream);
const char *tf_status_string(int32_t status);
const char *tf_last_error(const tf_ctx *ctx);
uint32_t tf_abi_version(void);

/* ---- dequantization (bit-exact) --------------------------------------------------------------------- */
/* Quantization.dequantizeInt4Affine / dequantizeInt8Affine (Infrastructure/ModelIO/Quantization.swift:105-119,
 * 179-191) over a [m, n] matrix: out[r, c] = float(q) * scale + bias as fp32, bit-for-bit. */
int32_t tf_dequantize_int4_affine(tf_ctx *ctx, tf_stream stream,
                                  const void *weights, uint64_t weights_offset,
                                  const void *scales, uint64_t scales_offset,
                                  const void *biases, uint64_t biases_offset,
                                  void *out_f32, uint64_t out_offset,
                                  uint32_t m, uint32_t n, tf_dtype scale_dtype);
int32_t tf_dequantize_int8_affine(tf_ctx *ctx, tf_stream stream,
                                  const void *weights, uint64_t weights_offset,
                                  const void *scales, uint64_t scales_offset,
                                  const void *biases, uint64_t biases_offset,
                                  void *out_f32, uint64_t out_offset,
                                  uint32_t m, uint32_t n, tf_dtype scale_dtype);

/* ---- GEMV ---------------------------------------------------------------------------------------------- */
/* DequantInt4GEMV.encode (Kernels/Quant/DequantInt4GEMV.swift:44-87) -> dequant_int4_gemv_simd
 * (Metal/Quant/dequant_int4.metal:173-191).  y[r] = sum_c w[r,c] * x[c]; x fp16 [n]; fp32 accumulation;
 * y is fp16 (reference) or fp32 (out_dtype).  n % 64 == 0, weights_offset even. */
int32_t tf_dequant_int4_gemv(tf_ctx *ctx, tf_stream stream,
                             const void *weights, uint64_t weights_offset,
                             const void *scales, uint64_t scales_offset,
                             const void *biases, uint64_t biases_offset,
                             const void *x, uint64_t x_offset,
                             void *y, uint64_t y_offset,
                             uint32_t m, uint32_t n, tf_dtype scale_dtype, tf_dtype out_dtype);
/* DequantInt8GEMV.encode (Kernels/Quant/DequantInt8GEMV.swift) -> dequant_int8_gemv_simd
 * (Metal/Quant/dequant_int8.metal:56-97). */
int32_t tf_dequant_int8_gemv(tf_ctx *ctx, tf_stream stream,
                             const void *weights, uint64_t weights_offset,
                             const void *scales, uint64_t scales_offset,
                             const void *biases, uint64_t biases_offset,
                             const void *x, uint64_t x_offset,
                             void *y, uint64_t y_offset,
                             uint32_t m, uint32_t n, tf_dtype scale_dtype, tf_dtype out_dtype);

/* ---- primitives on the path -------------------------------------------------------------------------------- */
/* gelu_mul_fp16 (Metal/Primitives/utility.metal:6-18; dispatched at SharedExpertInt4.swift:76-86):
 * out = half(gelu_tanh(float(gate)) * float(up)). */
int32_t tf_gelu_mul_fp16(tf_ctx *ctx, tf_stream stream,
                         const void *gate, uint64_t gate_offset, const void *up, uint64_t up_offset,
                         void *out, uint64_t out_offset, uint32_t count);
/* RMSNorm.encodeBF16W (Kernels/Primitives/RMSNorm.swift:54-66) -> rmsnorm_bf16w (Metal/Primitives/rmsnorm.metal:70-93). */
int32_t tf_rmsnorm_bf16w(tf_ctx *ctx, tf_stream stream,
                         const void *x, uint64_t x_offset, const void *weight, uint64_t weight_offset,
                         void *out, uint64_t out_offset, uint32_t d, float eps);

/* ---- shared expert ------------------------------------------------------------------------------------------- */
/* SharedExpertInt4.encode (Kernels/MoE/SharedExpertInt4.swift:31-99): gate GEMV, up GEMV (fp16 out),
 * gelu_mul_fp16, down GEMV.  Scratch sizes are in BYTES (the MTLBuffer.length checks at :46-58); each must hold
 * gate.rows halves.  `weight_bits` mirrors SharedExpertRuntime (:102-113): only 4 is built, 8 returns
 * TF_ERR_UNSUPPORTED_BITS (the pinned checkpoint uses the 4-bit shared expert). */
int32_t tf_shared_expert_int4(tf_ctx *ctx, tf_stream stream,
                              const void *x, uint64_t x_offset, uint64_t x_length,
                              const tf_projection *gate, const tf_projection *up, const tf_projection *down,
                              void *y, uint64_t y_offset, uint64_t y_length,
                              void *scratch_gate, uint64_t scratch_gate_offset, uint64_t scratch_gate_length,
                              void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                              void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length,
                              uint32_t weight_bits, tf_dtype scale_dtype);

/* ---- router ----------------------------------------------------------------------------------------------------- */
/* MoE.encodeRouterGemma4 (Kernels/MoE/MoE.swift:109-159) -> router_gemv_gemma4_r4 + router_topk_select_k8
 * (Metal/MoE/moe.metal:78-185).  hidden fp16 [d] (no offset, as in the reference), effective_scale bf16 [d],
 * per_expert_scale bf16 [num_experts]; out_indices uint32[8] descending score (ties: lower index),
 * out_weights fp16[8] = softmax over the eight * per_expert_scale.  d % 64 == 0, num_experts <= 256, top_k == 8.
 * Both outputs stay on the device. */
int32_t tf_router_gemma4(tf_ctx *ctx, tf_stream stream,
                         const void *weights, uint64_t weights_offset,
                         const void *scales, uint64_t scales_offset,
                         const void *biases, uint64_t biases_offset,
                         const void *hidden,
                         const void *effective_scale, uint64_t effective_scale_offset,
                         const void *per_expert_scale, uint64_t per_expert_scale_offset,
                         void *out_indices, void *out_weights,
                         uint32_t num_experts, uint32_t d, uint32_t top_k);
/* The fp32 logits of the last tf_router_gemma4 call on this ctx (the wrapper-owned `routerLogits`, MoE.swift:92-99).
 * Device pointer to 256 floats; valid until the ctx is destroyed. */
const float *tf_router_logits(const tf_ctx *ctx);

/* ---- routed experts ------------------------------------------------------------------------------------------------- */
/* MoE.encodeRoutedPersistentPhase1U16Load (MoE.swift:180-213) -> moe_phase1_gate_up_act_u16load (moe.metal:407-423):
 * acts[slot*f + r] = half(gelu_tanh(gate_r . x) * (up_r . x)), GeGLU on the fp32 sums. */
int32_t tf_moe_phase1_gate_up_act(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed,
                                  const tf_expert_offsets *routed_offsets, const void *x, void *acts,
                                  uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype);
/* MoE.encodeRoutedPersistentPhase1SubsetU16Load (MoE.swift:215-258) -> ..._subset_u16load (moe.metal:425-444):
 * same for the slots listed in the DEVICE array active_slots[0..active_count); other slots of acts untouched;
 * active_count == 0 enqueues nothing. */
int32_t tf_moe_phase1_gate_up_act_subset(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed,
                                         const tf_expert_offsets *routed_offsets, const void *x, void *acts,
                                         const uint32_t *active_slots, uint32_t active_count,
                                         uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype);
/* MoE.encodeRoutedPersistentPhase2Reduce (MoE.swift:260-295) -> moe_phase2_down_reduce_k8 (moe.metal:446-482):
 * y[r] = half(residual[r] + sum_{slot=0..7} float(routing_w[slot]) * (down_slot[r,:] . acts[slot,:])), summed in
 * slot order.  routing_w fp16[8] on the device. */
int32_t tf_moe_phase2_down_reduce(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed,
                                  const tf_expert_offsets *routed_offsets, const void *acts, const void *routing_weights,
                                  const void *residual, void *y, uint32_t d, uint32_t f, uint32_t top_k,
                                  tf_dtype scale_dtype);

/* One routed-MoE decode step enqueued by a single call: tf_router_gemma4 -> tf_moe_phase1_gate_up_act ->
 * tf_moe_phase2_down_reduce over a resident expert pool, the selected indices flowing from kernel to kernel in device
 * memory.  It is the sequence RealForwardRunner.produceToken runs per layer (Runtime/Inference/RealForwardRunner.swift:
 * 1462-1470 router, :1652-1685 phase 1 + phase 2) without the CPU wait at :1472 and the expert fetch at :1623-1631.
 * `router_x` feeds the router, `x` the experts (router_x / routed_x of fused_post_attn_setup).  out_indices (uint32[8]),
 * out_weights (fp16[8]) and acts (fp16[8*f]) are caller-owned device buffers. */
int32_t tf_moe_decode_step(tf_ctx *ctx, tf_stream stream,
                           const void *router_weights, uint64_t router_weights_offset,
                           const void *router_scales, uint64_t router_scales_offset,
                           const void *router_biases, uint64_t router_biases_offset,
                           const void *router_x,
                           const void *effective_scale, uint64_t effective_scale_offset,
                           const void *per_expert_scale, uint64_t per_expert_scale_offset,
                           const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                           const tf_expert_offsets *routed_offsets,
                           const void *x, void *acts, const void *residual, void *y,
                           void *out_indices, void *out_weights,
                           uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype);

/* ---- lm_head ----------------------------------------------------------------------------------------------------------- */
/* LMHeadChainInt4.encodeGreedyDecode (Kernels/Fusions/LMHeadChainInt4.swift:53-122) -> rmsnorm_bf16w,
 * lm_head_greedy_int4_rows_chunk_raw, lm_head_greedy_int4_rows_reduce (Metal/Sampling/logit.metal:692-787):
 * token = argmax_r (W[r,:] . half(rmsnorm(hidden))) on the raw fp32 logits; non-finite rows are skipped; ties go to
 * the lowest row; nothing finite => 0.  out_token: one uint32 on the device.  d % 64 == 0. */
int32_t tf_lm_head_greedy_int4(tf_ctx *ctx, tf_stream stream,
                               const void *hidden, uint64_t hidden_offset,
                               const void *norm_weight, uint64_t norm_offset,
                               const void *weights, uint64_t weights_offset,
                               const void *scales, uint64_t scales_offset,
                               const void *biases, uint64_t biases_offset,
                               void *out_token, uint32_t d, uint32_t vocab, float rms_eps, tf_dtype scale_dtype);
/* The logits head (Runtime/Inference/RealForwardRunner.swift:1704-1715; Kernels/Prefill/Epilogues/
 * PrefillFinalRowHead.swift:22-65): rmsnorm_bf16w then the M = vocab GEMV.  logits are fp16 (reference) or fp32. */
int32_t tf_lm_head_logits_int4(tf_ctx *ctx, tf_stream stream,
                               const void *hidden, uint64_t hidden_offset,
                               const void *norm_weight, uint64_t norm_offset,
                               const void *weights, uint64_t weights_offset,
                               const void *scales, uint64_t scales_offset,
                               const void *biases, uint64_t biases_offset,
                               void *logits, uint64_t logits_offset,
                               uint32_t d, uint32_t vocab, float rms_eps, tf_dtype scale_dtype, tf_dtype out_dtype);

#ifdef __cplusplus
}
#endif
#endif /* TF_KERNELS_H */

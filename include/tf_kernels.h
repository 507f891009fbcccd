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
 *     command queue); nothing blocks or allocates except tf_ctx_create,
 *     tf_ctx_reserve, tf_stream_synchronize, the tf_upload_* loaders and
 *     tf_ctx_last_step_timing (which waits for the timed step's last event), so
 *     every other entry point may be recorded into a HIP graph;
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
/* The reference's wrappers size their own scratch once, in `init` (MoE.swift:92-99 routerLogits for 256 experts;
 * LMHeadChainInt4.swift:38-51 xNormed/rowSummaries for maxD/maxVocab; PrefillRouter, PrefillSharedExpert and the samplers
 * likewise).  Here that is tf_ctx_create, which sizes every wrapper buffer for the limits below, and tf_ctx_reserve,
 * which raises them (limits only grow; it waits for the device and reallocates, so call it at set-up, never while a
 * stream is being captured).  An entry point whose arguments exceed the limits returns TF_ERR_SCRATCH_TOO_SMALL and
 * enqueues nothing; no entry point allocates, frees or synchronises.  tf_ctx_create's limits are
 * {262144, 2048, 256, 2112, 16, 512, 128}. */
typedef struct tf_scratch_limits {
    uint32_t max_vocab;                  /* lm_head rows: fp32 logits of the unaligned greedy path, the samplers' cells and top-k pair buffers */
    uint32_t max_block_tokens;           /* rows of one prefill block: router logits [tokens, experts], shared-expert activations */
    uint32_t max_experts;                /* router width of the multi-token router */
    uint32_t max_shared_intermediate;    /* shared expert's intermediate size (activations [tokens, intermediate] of the block form) */
    uint32_t max_q_heads, max_head_dim;  /* decode and block attention: split-KV partial states */
    uint32_t max_attention_block_tokens; /* queries of one tf_prefill_attention_causal call */
} tf_scratch_limits;
int32_t tf_ctx_reserve(tf_ctx *ctx, const tf_scratch_limits *limits);
int32_t tf_ctx_scratch_limits(const tf_ctx *ctx, tf_scratch_limits *out_limits);
/* commandBuffer.waitUntilCompleted + checkCommandBufferError (MetalContext.swift:22-26): returns TF_ERR_DEVICE if
 * anything enqueued on the stream failed. */
int32_t tf_stream_synchronize(tf_ctx *ctx, tf_stream stream);
const char *tf_status_string(int32_t status);
const char *tf_last_error(const tf_ctx *ctx);
uint32_t tf_abi_version(void);
/* The runner's hand-rolled phase counters (totalCb1Nanos / totalCb2Nanos ..., RealForwardRunner.swift:408-419, surfaced by
 * DecodeRunnerDiagnostics), as device time: while enabled, tf_moe_decode_step brackets its router, phase-1 and phase-2
 * launches with HIP events on the call's stream, and tf_ctx_last_step_timing waits for the most recent step and returns,
 * in microseconds, out_us[0..2] = the three brackets and out_us[3] = an empty bracket (two events with nothing between
 * them: what the event packets themselves cost, to be subtracted from each of the others).  Leave it disabled while a
 * stream is being captured into a graph. */
int32_t tf_ctx_set_step_timing(tf_ctx *ctx, int32_t enabled);
int32_t tf_ctx_last_step_timing(tf_ctx *ctx, float out_us[4]);

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

/* FusedQKVGEMV.encode (Kernels/Fusions/FusedQKVGEMV.swift:38-97) -> dequant_int4_qkv_gemv_simd
 * (Metal/Quant/dequant_int4.metal:194-244): the q, k and v projections of one token in one launch;
 * q [q_rows, n], k and v [kv_rows, n] int4 group-64 with bf16/fp16 scales, x fp16[n], outputs fp16.
 * Each output equals tf_dequant_int4_gemv of its matrix bit for bit.  n % 64 == 0, even weights offsets. */
int32_t tf_fused_qkv_gemv(tf_ctx *ctx, tf_stream stream, const void *q_weights, uint64_t q_weights_offset, const void *q_scales,
                          uint64_t q_scales_offset, const void *q_biases, uint64_t q_biases_offset, const void *k_weights,
                          uint64_t k_weights_offset, const void *k_scales, uint64_t k_scales_offset, const void *k_biases,
                          uint64_t k_biases_offset, const void *v_weights, uint64_t v_weights_offset, const void *v_scales,
                          uint64_t v_scales_offset, const void *v_biases, uint64_t v_biases_offset, const void *x, void *q_out,
                          uint64_t q_out_offset, void *k_out, uint64_t k_out_offset, void *v_out, uint64_t v_out_offset, uint32_t q_rows,
                          uint32_t kv_rows, uint32_t n, tf_dtype scale_dtype);

/* RMSNorm.encodeBF16W (Kernels/Primitives/RMSNorm.swift:17-66) + FusedQKVGEMV.encode in ONE launch: the input norm of a
 * decoder layer feeds nothing but the three projections (RealForwardRunner.swift: the per-layer decode loop), so every
 * block normalises `hidden` (fp16[n], raw) with norm_weight (bf16[n]) on its way into LDS instead of a launch of its own
 * writing a normalised copy.  q_out / k_out / v_out equal tf_rmsnorm_bf16w followed by tf_fused_qkv_gemv bit for bit.
 * Shapes the one-launch kernel does not take (n <= 1024, unaligned operands) run the two steps through the context's
 * one-row buffer (n <= 16384, else TF_ERR_SCRATCH_TOO_SMALL). */
int32_t tf_fused_norm_qkv_gemv(tf_ctx *ctx, tf_stream stream, const void *norm_weight, uint64_t norm_weight_offset, float eps,
                               const void *q_weights, uint64_t q_weights_offset, const void *q_scales, uint64_t q_scales_offset,
                               const void *q_biases, uint64_t q_biases_offset, const void *k_weights, uint64_t k_weights_offset,
                               const void *k_scales, uint64_t k_scales_offset, const void *k_biases, uint64_t k_biases_offset,
                               const void *v_weights, uint64_t v_weights_offset, const void *v_scales, uint64_t v_scales_offset,
                               const void *v_biases, uint64_t v_biases_offset, const void *hidden, void *q_out, uint64_t q_out_offset,
                               void *k_out, uint64_t k_out_offset, void *v_out, uint64_t v_out_offset, uint32_t q_rows, uint32_t kv_rows,
                               uint32_t n, tf_dtype scale_dtype);
/* tf_fused_layer_tail_shared_norm of one decoder layer followed by tf_fused_norm_qkv_gemv of the next as one call: the runner
 * encodes the layers back to back (RealForwardRunner.swift:1462-1685), and the tail's output is read by nothing but the next
 * layer's input norm and the residual add after its attention.  Every block of the projection launch repeats the tail's row
 * reductions in its prologue (FusedLayerTail.swift:19-52 -> fused_layer_tail, fused.metal:271-375, with the shared expert's
 * post-norm first) and normalises the result on its way into LDS; block 0 writes it to hidden_out.  One launch fewer per decoder
 * layer; every output equals the two calls bit for bit.  hidden_out must be a different buffer from h2, shared_out and hidden
 * for the tail to be folded in; otherwise, or with operands that are not 16-byte aligned or rows the row streamer does not
 * take, the tail runs as its own launch first.  n <= 4096. */
int32_t tf_fused_layer_tail_norm_qkv_gemv(tf_ctx *ctx, tf_stream stream,
                               const void *h2, const void *shared_out, const void *hidden, void *hidden_out,
                               const void *post_ffn1_weight, uint64_t post_ffn1_weight_offset,
                               const void *post_ffn2_weight, uint64_t post_ffn2_weight_offset,
                               const void *post_ffn_weight, uint64_t post_ffn_weight_offset, float tail_eps, float layer_scalar,
                               const void *norm_weight, uint64_t norm_weight_offset, float eps,
                               const void *q_weights, uint64_t q_weights_offset, const void *q_scales, uint64_t q_scales_offset,
                               const void *q_biases, uint64_t q_biases_offset,
                               const void *k_weights, uint64_t k_weights_offset, const void *k_scales, uint64_t k_scales_offset,
                               const void *k_biases, uint64_t k_biases_offset,
                               const void *v_weights, uint64_t v_weights_offset, const void *v_scales, uint64_t v_scales_offset,
                               const void *v_biases, uint64_t v_biases_offset,
                               void *q_out, uint64_t q_out_offset, void *k_out, uint64_t k_out_offset,
                               void *v_out, uint64_t v_out_offset,
                               uint32_t q_rows, uint32_t kv_rows, uint32_t n, tf_dtype scale_dtype);

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
/* RMSNorm.encodeNoScale (RMSNorm.swift:67-87) -> rmsnorm_no_scale (rmsnorm.metal:153-175): out = half(x * inv). */
int32_t tf_rmsnorm_no_scale(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *out, uint64_t out_offset,
                            uint32_t d, float eps);
/* RMSNorm.encodeBF16WPerHead / encodeNoScalePerHead (RMSNorm.swift:89-136) -> rmsnorm_bf16w_perhead,
 * rmsnorm_no_scale_perhead (rmsnorm.metal:100-151): num_heads contiguous heads of head_dim, each normalised on its own;
 * weight bf16[head_dim] shared by the heads.  In place is allowed. */
int32_t tf_rmsnorm_bf16w_perhead(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight,
                                 uint64_t weight_offset, void *out, uint64_t out_offset, uint32_t head_dim,
                                 uint32_t num_heads, float eps);
int32_t tf_rmsnorm_no_scale_perhead(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *out,
                                    uint64_t out_offset, uint32_t head_dim, uint32_t num_heads, float eps);
/* PrefillRMSNorm.encodeBF16W (Kernels/Prefill/Primitives/PrefillPrimitives.swift:41-71) -> prefill_rmsnorm_bf16w_block
 * (Metal/Prefill/prefill.metal:86-111): `tokens` contiguous rows of d. */
int32_t tf_prefill_rmsnorm_bf16w_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight,
                                       uint64_t weight_offset, void *out, uint64_t out_offset, uint32_t tokens, uint32_t d,
                                       float eps);
/* PrefillPerHeadNorm.encodeBF16W / encodeNoScale (Kernels/Prefill/Primitives/PrefillPerHeadNorm.swift:13-84) ->
 * prefill_rmsnorm_bf16w_perhead_block, prefill_rmsnorm_no_scale_perhead_block (prefill.metal:113-176): head h of token t at
 * t * token_stride_elements + h * head_dim in x and in out; elements between token rows are untouched.  Every row equals
 * the single-row call on that row, bit for bit (the reference suite's own check, PrefillPerHeadNormTests.swift:90,144). */
int32_t tf_prefill_rmsnorm_bf16w_perhead_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset,
                                               const void *weight, uint64_t weight_offset, void *out, uint64_t out_offset,
                                               uint32_t query_count, uint32_t head_dim, uint32_t num_heads,
                                               uint32_t token_stride_elements, float eps);
int32_t tf_prefill_rmsnorm_no_scale_perhead_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *out,
                                                  uint64_t out_offset, uint32_t query_count, uint32_t head_dim,
                                                  uint32_t num_heads, uint32_t token_stride_elements, float eps);

/* ---- the stages either side of the MoE block ------------------------------------------------------------------- */
/* FusedPostAttentionSetup.encode (Kernels/Fusions/FusedPostAttentionSetup.swift:19-56) -> fused_post_attn_setup
 * (Metal/Fusions/fused.metal:190-269).  All activations fp16[d], weights bf16[d], d <= 4096:
 *   hidden   <- half(hidden + half(attn * rsqrt(mean(attn^2) + eps) * post_attention_weight))      (in place)
 *   h         = hidden * rsqrt(mean(hidden^2) + eps)
 *   dense_x   = half(h * pre_ffn_weight),  routed_x = half(h * pre_ffn2_weight),  router_x = half(h). */
int32_t tf_fused_post_attn_setup(tf_ctx *ctx, tf_stream stream, void *hidden, const void *attn, void *dense_x, void *routed_x,
                                 void *router_x, const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                 const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset, const void *pre_ffn2_weight,
                                 uint64_t pre_ffn2_weight_offset, uint32_t d, float eps);
/* PrefillPostAttentionSetup.encode (Kernels/Prefill/Epilogues/PrefillPostAttentionSetup.swift:11-74) ->
 * prefill_post_attn_setup_block (Metal/Prefill/prefill.metal:178-253): the same for query_count rows, row r of each
 * operand at r * its stride (in elements, >= d); bytes between rows are left untouched. */
int32_t tf_prefill_post_attn_setup_block(tf_ctx *ctx, tf_stream stream, void *hidden, uint64_t hidden_offset, const void *attn,
                                         uint64_t attn_offset, void *dense_x, uint64_t dense_x_offset, void *routed_x,
                                         uint64_t routed_x_offset, void *router_x, uint64_t router_x_offset,
                                         const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                         const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset, const void *pre_ffn2_weight,
                                         uint64_t pre_ffn2_weight_offset, uint32_t query_count, uint32_t d,
                                         uint32_t hidden_stride_elements, uint32_t attn_stride_elements,
                                         uint32_t dense_stride_elements, uint32_t routed_stride_elements,
                                         uint32_t router_stride_elements, float eps);
/* FusedLayerTail.encode (Kernels/Fusions/FusedLayerTail.swift:19-52) -> fused_layer_tail (Metal/Fusions/fused.metal:271-375):
 *   h12     = half(h1 + half(h2 * rsqrt(mean(h2^2) + eps) * post_ffn2_weight))
 *   hidden <- half(half(hidden + half(h12 * rsqrt(mean(h12^2) + eps) * post_ffn_weight)) * half(layer_scalar))   (in place) */
int32_t tf_fused_layer_tail(tf_ctx *ctx, tf_stream stream, const void *h2, const void *h1, void *hidden, const void *post_ffn2_weight,
                            uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset, uint32_t d,
                            float eps, float layer_scalar);
/* RMSNorm.encodeBF16W of the shared expert's output (RealForwardRunner.swift: h1 = rmsnorm(shared, post_ffn1)) + FusedLayerTail.encode
 * in ONE launch: shared_out is the shared expert's raw output, h1 = half(shared_out * rsqrt(mean(shared_out^2) + eps) *
 * post_ffn1_weight) is formed in registers and the tail proceeds as tf_fused_layer_tail.  Equal to the two calls up to the
 * order in which the squares of shared_out are summed (a last-bit difference of 1/rms can move an fp16 rounding on a tie). */
int32_t tf_fused_layer_tail_shared_norm(tf_ctx *ctx, tf_stream stream, const void *h2, const void *shared_out, void *hidden,
                                        const void *post_ffn1_weight, uint64_t post_ffn1_weight_offset, const void *post_ffn2_weight,
                                        uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset,
                                        uint32_t d, float eps, float layer_scalar);
/* PrefillLayerTail.encode (Kernels/Prefill/Epilogues/PrefillLayerTail.swift:11-60) -> prefill_layer_tail_block
 * (Metal/Prefill/prefill.metal:255-334): the same for query_count strided rows. */
int32_t tf_prefill_layer_tail_block(tf_ctx *ctx, tf_stream stream, const void *h2, uint64_t h2_offset, const void *h1,
                                    uint64_t h1_offset, void *hidden, uint64_t hidden_offset, const void *post_ffn2_weight,
                                    uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset,
                                    uint32_t query_count, uint32_t d, uint32_t h2_stride_elements, uint32_t h1_stride_elements,
                                    uint32_t hidden_stride_elements, float eps, float layer_scalar);

/* ---- shared expert ------------------------------------------------------------------------------------------- */
/* SharedExpertInt4.encode (Kernels/MoE/SharedExpertInt4.swift:31-99): gate GEMV, up GEMV (fp16 out),
 * gelu_mul_fp16, down GEMV.  Scratch sizes are in BYTES (the MTLBuffer.length checks at :46-58); each must hold
 * gate.rows halves.  `weight_bits` mirrors SharedExpertRuntime (:96-137): 4 runs this chain, 8 hands over to
 * tf_shared_expert_int8 (which uses scratch_act only), anything else returns TF_ERR_UNSUPPORTED_BITS. */
int32_t tf_shared_expert_int4(tf_ctx *ctx, tf_stream stream,
                              const void *x, uint64_t x_offset, uint64_t x_length,
                              const tf_projection *gate, const tf_projection *up, const tf_projection *down,
                              void *y, uint64_t y_offset, uint64_t y_length,
                              void *scratch_gate, uint64_t scratch_gate_offset, uint64_t scratch_gate_length,
                              void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                              void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length,
                              uint32_t weight_bits, tf_dtype scale_dtype);
/* SharedExpertInt8.encode / encodePhase1 / encodeDown (Kernels/MoE/SharedExpertInt8.swift:67-170) ->
 * shared_int8_gate_up_act_simd (Metal/Quant/dequant_int8.metal:100-157) then dequant_int8_gemv_simd: 8-bit affine group-64
 * projections (one byte per weight), act = half(gelu_tanh(half(gate)) * half(up)) into scratch_act (gate.rows halves), then
 * the down GEMV.  Lengths in bytes; SharedExpertInt8Error.dimensionMismatch -> TF_ERR_DIMENSION_MISMATCH, .scratchTooSmall ->
 * TF_ERR_SCRATCH_TOO_SMALL. */
int32_t tf_shared_expert_int8(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, uint64_t x_length,
                              const tf_projection *gate, const tf_projection *up, const tf_projection *down, void *y,
                              uint64_t y_offset, uint64_t y_length, void *scratch_act, uint64_t scratch_act_offset,
                              uint64_t scratch_act_length, tf_dtype scale_dtype);
int32_t tf_shared_expert_int8_phase1(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, uint64_t x_length,
                                     const tf_projection *gate, const tf_projection *up, void *scratch_act,
                                     uint64_t scratch_act_offset, uint64_t scratch_act_length, tf_dtype scale_dtype);
int32_t tf_shared_expert_int8_down(tf_ctx *ctx, tf_stream stream, const tf_projection *down, void *y, uint64_t y_offset,
                                   uint64_t y_length, const void *scratch_act, uint64_t scratch_act_offset,
                                   uint64_t scratch_act_length, tf_dtype scale_dtype);

/* PrefillSharedExpert.encodeBlock (Kernels/Prefill/MoE/PrefillSharedExpert.swift:11-58): the shared expert for
 * query_count rows of x (row stride x_stride_elements halves) into query_count rows of y.  The reference runs the
 * single-row chain once per row through the same one-row scratch buffers; so does this entry for fewer than 8 rows and
 * for operands the matrix-core path cannot take (weights or x rows not 16-byte aligned, intermediate % 64 != 0, the scale
 * or the bias arrays of gate and up more than 2 GiB apart).
 * Otherwise the rows go through the matrix cores: gate and up in one pass with both sums rounded to fp16 before GeGLU
 * (the chain's stage boundary), activations in a buffer the context owns, then the down projection; weights are
 * expanded to fp16 half(q*s+b) per group as in tf_int4_qmm, so results agree with the row chain within the shared
 * expert's tolerance, not bit for bit, and the caller's scratch (still validated: one row each, lengths in BYTES) is
 * left untouched.  weight_bits == 8 (PrefillSharedExpert's default): up to 15 rows in groups against each weight row,
 * bit-identical to repeated tf_shared_expert_int8; from 16 aligned rows on on the matrix cores with every weight
 * rounded to fp16 first, within the 8-bit shared expert's tolerance of the row chain (scales keep their precision
 * down to 2^-24; a weight below fp16's normal range, 6e-5, is kept to 6e-8).  query_count == 0 is a no-op.  d, intermediate > 0,
 * strides >= d (TF_ERR_INVALID_ARGUMENT); gate/up = (intermediate, d), down = (d, intermediate) or
 * TF_ERR_DIMENSION_MISMATCH. */
int32_t tf_prefill_shared_expert_int4_block(tf_ctx *ctx, tf_stream stream,
                                            const void *x, uint64_t x_offset, void *y, uint64_t y_offset,
                                            const tf_projection *gate, const tf_projection *up, const tf_projection *down,
                                            void *scratch_gate, uint64_t scratch_gate_offset, uint64_t scratch_gate_length,
                                            void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                                            void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length,
                                            uint32_t query_count, uint32_t d, uint32_t intermediate,
                                            uint32_t x_stride_elements, uint32_t y_stride_elements,
                                            uint32_t weight_bits, tf_dtype scale_dtype);

/* ---- decode attention (next in line after the quantized matmuls: the step between the QKV and the O projection) --- */
/* Attention.encodeSWA / encodeFull (Kernels/Attention/Attention.swift:150-214) -> attention_decode_partial,
 * attention_decode_gqa_swa_partial, attention_decode_combine (Metal/Attention/attention.metal:135-377): one query token,
 * q fp16 [num_q_heads, head_dim], k and v fp16 [rows, num_kv_heads, head_dim], out fp16 [num_q_heads, head_dim];
 * query head h reads kv head h / (num_q_heads / num_kv_heads).  Split-KV online softmax in fp32: un-normalized partial
 * states per chunk of positions, then a merge; the number of chunks is chosen for this GPU, not the reference's 8 / 16
 * (which only changes fp32 rounding of the partial sums, as the reference notes at :128-133).  scale <= 0 selects
 * 1 / sqrt(head_dim) (the reference's nil).  SWA attends to [max(0, seq_len - window), seq_len); ring_capacity != 0:
 * position p lives in row p % ring_capacity and the window must fit the ring.  Preconditions as the reference's:
 * num_q_heads % num_kv_heads == 0, head_dim <= 512, num_q_heads <= 16, (full) seq_len > 0 -> TF_ERR_INVALID_ARGUMENT.
 * An empty SWA range writes zeros.  Partial states live in scratch owned by the context, as in the reference. */
int32_t tf_attention_swa(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k, uint64_t k_offset,
                         const void *v, uint64_t v_offset, void *out, uint64_t out_offset, uint32_t head_dim,
                         uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len, uint32_t window, float scale,
                         uint32_t ring_capacity);
int32_t tf_attention_full(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k, uint64_t k_offset,
                          const void *v, uint64_t v_offset, void *out, uint64_t out_offset, uint32_t head_dim,
                          uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len, float scale);

/* RoPE.encodeDefaultNeox / encodeProportionalNeox (Kernels/Primitives/RoPE.swift:27-90) -> rope_default_neox,
 * rope_proportional_neox (Metal/Primitives/rope.metal:33-96): data fp16 [num_tokens, num_heads, head_dim], in place; the
 * pairs (x[i], x[i + head_dim/2]), i < rotated_pairs (default: head_dim / 2), rotate by position * theta^(-2i/head_dim);
 * every token of the block gets the same position, as in the reference.  head_dim even, rotated_pairs * 2 <= head_dim. */
int32_t tf_rope_default_neox(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t position,
                             uint32_t head_dim, uint32_t num_heads, uint32_t num_tokens, float theta);
int32_t tf_rope_proportional_neox(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t position,
                                  uint32_t head_dim, uint32_t num_heads, uint32_t num_tokens, uint32_t rotated_pairs,
                                  float theta);

/* FusedQKVEpilogue.encode (Kernels/Fusions/FusedQKVEpilogue.swift:43-99) -> fused_qkv_epilogue
 * (Metal/Fusions/fused.metal:84-173): in place, per head, q [num_q_heads, head_dim] and k [num_kv_heads, head_dim]:
 * RMSNorm with the bf16 weight [head_dim] shared by the heads, rounded to fp16, then NeoX RoPE on the first
 * rotated_pairs pairs; v [num_kv_heads, head_dim]: RMSNorm without weight.  head_dim <= 512 and even,
 * rotated_pairs * 2 <= head_dim. */
int32_t tf_fused_qkv_epilogue(tf_ctx *ctx, tf_stream stream, void *q, uint64_t q_offset, void *k, uint64_t k_offset,
                              void *v, uint64_t v_offset, const void *q_weight, uint64_t q_weight_offset,
                              const void *k_weight, uint64_t k_weight_offset, uint32_t head_dim, uint32_t num_q_heads,
                              uint32_t num_kv_heads, uint32_t position, float theta, uint32_t rotated_pairs, float eps);
/* PrefillRoPE.encodeDefaultNeox / encodeProportionalNeox (Kernels/Prefill/Primitives/PrefillRoPE.swift:13-88) ->
 * prefill_rope_default_neox_block, prefill_rope_proportional_neox_block (Metal/Prefill/prefill.metal:709-775): token t of
 * the block (row t, token_stride_elements apart) is rotated for position start_position + t, in place. */
int32_t tf_prefill_rope_default_neox_block(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset,
                                           uint32_t start_position, uint32_t query_count, uint32_t head_dim,
                                           uint32_t num_heads, uint32_t token_stride_elements, float theta);
int32_t tf_prefill_rope_proportional_neox_block(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset,
                                                uint32_t start_position, uint32_t query_count, uint32_t head_dim,
                                                uint32_t num_heads, uint32_t rotated_pairs, uint32_t token_stride_elements,
                                                float theta);
/* PrefillQKVEpilogue.encode (Kernels/Prefill/Epilogues/PrefillQKVEpilogue.swift:13-121): per token of the block the
 * per-head norms of q, k (bf16 weight) and v (no scale), then the rotation of q and k for position start_position + t; one
 * launch here, the reference's five.  Each token equals tf_fused_qkv_epilogue on its rows, bit for bit. */
int32_t tf_prefill_qkv_epilogue_block(tf_ctx *ctx, tf_stream stream, void *q, uint64_t q_offset, void *k, uint64_t k_offset,
                                      void *v, uint64_t v_offset, const void *q_weight, uint64_t q_weight_offset,
                                      const void *k_weight, uint64_t k_weight_offset, uint32_t start_position,
                                      uint32_t query_count, uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                                      uint32_t q_token_stride_elements, uint32_t kv_token_stride_elements, float theta,
                                      uint32_t rotated_pairs, float eps);

/* PrefillAttentionParams (Kernels/Attention/PrefillAttention.swift:4-40; Metal/Prefill/prefill.metal:775-788): 44 bytes. */
typedef struct tf_prefill_attention_params {
    uint32_t start_position, query_count, head_dim, num_q_heads, num_kv_heads, kv_valid_count, sliding_window;
    uint32_t kv_token_stride_elements, q_token_stride_elements, o_token_stride_elements;
    float scale;
} tf_prefill_attention_params;
/* PrefillAttention.encodeCausal (PrefillAttention.swift:56-118) -> attention_prefill_causal_tiled (prefill.metal:835-902):
 * query t of the block (row t of q, stride q_token_stride_elements) sits at position start_position + t and attends to
 * the keys [first, last): first = position + 1 - sliding_window when a window is set and exceeded, else 0;
 * last = min(kv_valid_count, position + 1).  k, v rows at kv_token_stride_elements (row p % kv_ring_capacity when a
 * ring is given); out row t at o_token_stride_elements; query head h reads kv head h / (num_q_heads / num_kv_heads);
 * a query that sees no key gets zeros; bytes between rows are untouched.  Preconditions as PrefillAttention.validate
 * (:120-136) -> TF_ERR_INVALID_ARGUMENT.  The reference's choice between its tiled and tensor-op pipelines (`path`) has
 * no counterpart: 16-byte aligned rows with head_dim in {64,128,256,512} run on the matrix cores, everything else on a
 * kernel of the reference's own shape. */
int32_t tf_prefill_attention_causal(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k,
                                    uint64_t k_offset, const void *v, uint64_t v_offset, void *out, uint64_t out_offset,
                                    const tf_prefill_attention_params *params, uint32_t kv_ring_capacity);

/* AttentionSplitGeometry / Attention.splitGeometry (Attention.swift:5-11,128-147): the reference's own dispatch shape for
 * a range, kept for callers that report it; pure host function, no context. */
typedef struct tf_attention_split_geometry_t {
    int32_t effective_length, num_chunks, chunk_length, partial_threadgroups, use_swa_grouped_partial;
} tf_attention_split_geometry_t;
void tf_attention_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len, uint32_t kv_start,
                                 int32_t prefer_gqa_swa, tf_attention_split_geometry_t *out);

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
/* The same for the block router: [query_count, num_experts] fp32 logits of the most recent
 * tf_prefill_router_gemma4_block call on this context (NULL before the first call). */
const float *tf_prefill_router_logits(const tf_ctx *ctx);

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

/* No counterpart in the reference.  tf_moe_decode_step for callers that cannot allocate or wait for an allocation
 * (code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc): same arguments, same kernels,
 * bit-identical results, but the router logits between the launches live in a load-time device array of 256 floats (one
 * copy per GPU, held until the process ends) instead of the context's buffer, and the call neither allocates, frees nor
 * records timing events.  num_experts > 256 returns TF_ERR_SCRATCH_TOO_SMALL.  Every call on a GPU shares that GPU's
 * array: calls that overlap on one GPU (two streams, two contexts) race; calls on one stream do not.  Nothing in the
 * array needs clearing between calls: a call writes logits[0..num_experts) before it reads them and reads nothing beyond. */
int32_t tf_moe_decode_step_static(tf_ctx *ctx, tf_stream stream,
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

/* tf_moe_decode_step with the layer's shared expert (tf_shared_expert_int4, 4-bit weights) riding along: the reference commits
 * the shared expert on a command buffer of its own, beside the router and the routed experts
 * (RealForwardRunner.swift:1570-1594); here its gate / up rows run as extra blocks of the router launch and its down rows as
 * extra blocks of the routed phase 1, so the decoder layer has two launches fewer.  shared_x fp16[shared_gate->cols] ->
 * shared_y fp16[shared_down->rows]; the three scratch vectors (fp16[shared_gate->rows] each) receive gate, up and the
 * activation as tf_shared_expert_int4 leaves them.  Every output of either part equals the two separate calls bit for bit.
 * Shapes whose rows do not take the shared tile shape (the production widths 2816 / 2112 do), or operands that are not 16-byte
 * aligned, run the shared expert as its own launches first.  One scale_dtype for routed and shared weights. */
int32_t tf_moe_decode_step_shared(tf_ctx *ctx, tf_stream stream,
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
                                  uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                  const void *shared_x, const tf_projection *shared_gate, const tf_projection *shared_up,
                                  const tf_projection *shared_down, void *shared_y, void *shared_scratch_gate,
                                  void *shared_scratch_up, void *shared_scratch_act);
/* tf_fused_post_attn_setup followed by tf_moe_decode_step_shared as one call: FusedPostAttentionSetup.encode
 * (FusedPostAttentionSetup.swift:19-56) makes the three vectors the MoE block reads - router_x for the router, routed_x for the
 * routed experts, dense_x for the shared expert - and nothing else runs between it and them (RealForwardRunner.swift:1462-1594).
 * Here every block of the first launch (router logits + shared gate / up) repeats the setup's two row reductions in its own
 * prologue instead of waiting for a launch of them, one launch fewer per decoder layer; block 0 writes hidden_out (the new
 * residual stream), dense_x, routed_x and router_x as the stand-alone call does.  Every output equals the two calls bit for
 * bit.  hidden_out must be a different buffer from hidden (other blocks are still reading it) for the setup to be folded in;
 * with hidden_out == hidden, operands that are not 16-byte aligned or a step that does not take the shared launches, the
 * setup runs as its own launch first.  d <= 4096; the shared expert reads d values. */
int32_t tf_moe_decode_step_shared_post_attn(tf_ctx *ctx, tf_stream stream,
                                  const void *hidden, const void *attn, void *hidden_out,
                                  const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                  const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset,
                                  const void *pre_ffn2_weight, uint64_t pre_ffn2_weight_offset, float eps,
                                  const void *router_weights, uint64_t router_weights_offset,
                                  const void *router_scales, uint64_t router_scales_offset,
                                  const void *router_biases, uint64_t router_biases_offset,
                                  void *router_x,
                                  const void *effective_scale, uint64_t effective_scale_offset,
                                  const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                  const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                  const tf_expert_offsets *routed_offsets,
                                  void *routed_x, void *acts, const void *residual, void *y,
                                  void *out_indices, void *out_weights,
                                  uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                  void *dense_x, const tf_projection *shared_gate, const tf_projection *shared_up,
                                  const tf_projection *shared_down, void *shared_y,
                                  void *shared_scratch_gate, void *shared_scratch_up, void *shared_scratch_act);

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

/* ---- prefill / multi-token path --------------------------------------------------------------------------------------- */
/* PrefillTokenExpertPair (Kernels/Prefill/MoE/PrefillRouter.swift:5-28): 16 bytes, fields at 0/4/8/12; the low 16 bits of
 * weight_bits_and_reserved hold the fp16 routing weight. */
typedef struct tf_prefill_pair { uint32_t token, expert, rank, weight_bits_and_reserved; } tf_prefill_pair;
/* PrefillMoEGroup / PrefillMoETile (Kernels/Prefill/MoE/PrefillMoEGrouping.swift:4-29). */
typedef struct tf_prefill_group { uint32_t expert, pair_start, pair_count; } tf_prefill_group;
typedef struct tf_prefill_tile { uint32_t group_start, group_count, pair_start, pair_count; } tf_prefill_tile;
/* PrefillGroupedRoutedMoEStreamedParams (Kernels/Prefill/MoE/PrefillGroupedRoutedMoE.swift:104-183): 128 bytes, field
 * offsets 0,4,...,24, local_expert[0] at 28, local_expert[15] at 88, gate_W_off at 92, down_b_off at 124.  Unused
 * local_expert slots hold 0xFFFFFFFF. */
typedef struct tf_prefill_streamed_params {
    uint32_t pair_start, pair_count, d, routed_intermediate, top_k, hidden_stride_elements, live_expert_count;
    uint32_t local_expert[TF_MAX_TILE_EXPERTS];
    uint32_t gate_W_off, gate_s_off, gate_b_off, up_W_off, up_s_off, up_b_off, down_W_off, down_s_off, down_b_off;
} tf_prefill_streamed_params;

/* PrefillMoEGroupingError (PrefillMoEGrouping.swift:52-63), as negative statuses of the grouping call. */
#define TF_ERR_GROUP_INVALID_QUERY_COUNT (-101)
#define TF_ERR_GROUP_INVALID_TOP_K (-102)
#define TF_ERR_GROUP_INVALID_NUM_EXPERTS (-103)
#define TF_ERR_GROUP_INVALID_TILE_EXPERT_COUNT (-104)
#define TF_ERR_GROUP_PAIR_COUNT_MISMATCH (-105)
#define TF_ERR_GROUP_TOKEN_OUT_OF_RANGE (-106)
#define TF_ERR_GROUP_RANK_OUT_OF_RANGE (-107)
#define TF_ERR_GROUP_EXPERT_OUT_OF_RANGE (-108)
#define TF_ERR_GROUP_DUPLICATE_TOKEN_RANK (-109)
#define TF_ERR_GROUP_SORT_KEY_COUNT_MISMATCH (-110)

/* PrefillRouter.encodeGemma4Block (PrefillRouter.swift:37-89) -> prefill_router_gemma4_block (Metal/Prefill/prefill.metal:
 * 478-573): per token row t, logits over num_experts, top_k (1...64) by (score desc, index asc), softmax over the selected,
 * times per_expert_scale.  hidden rows are hidden_stride_elements apart.  out_indices uint32[T, top_k], out_weights
 * fp16[T, top_k].  query_count > 0, num_experts <= 256, d % 64 == 0, hidden_stride_elements >= d. */
int32_t tf_prefill_router_gemma4_block(tf_ctx *ctx, tf_stream stream,
                                       const void *weights, uint64_t weights_offset,
                                       const void *scales, uint64_t scales_offset,
                                       const void *biases, uint64_t biases_offset,
                                       const void *hidden, uint64_t hidden_offset,
                                       const void *effective_scale, uint64_t effective_scale_offset,
                                       const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                       void *out_indices, uint64_t out_indices_offset,
                                       void *out_weights, uint64_t out_weights_offset,
                                       uint32_t query_count, uint32_t num_experts, uint32_t d, uint32_t top_k,
                                       uint32_t hidden_stride_elements);

/* PrefillRouter.makeTokenExpertPairs (PrefillRouter.swift:91-111).  HOST arrays; pure CPU. */
int32_t tf_prefill_make_token_expert_pairs(const uint32_t *indices, const uint16_t *weights_f16, int32_t query_count,
                                           int32_t top_k, tf_prefill_pair *pairs);
/* PrefillMoEGrouping.groupTokenExpertPairs (PrefillMoEGrouping.swift:90-193).  HOST arrays; pure CPU.  Validates, sorts by
 * (sort key?, expert, token, rank), run-length groups, tiles of <= tile_expert_count experts.  expert_sort_keys may be NULL.
 * per_expert_offsets/per_expert_counts: num_experts entries (offset 0xFFFFFFFF = expert unused); groups/tiles: capacity
 * min(num_experts, pair_count) each.  Returns TF_OK or one of TF_ERR_GROUP_*. */
int32_t tf_prefill_group_token_expert_pairs(const tf_prefill_pair *pairs, uint64_t pair_count, int32_t query_count,
                                            int32_t top_k, int32_t num_experts, int32_t tile_expert_count,
                                            const uint64_t *expert_sort_keys, uint64_t expert_sort_key_count,
                                            tf_prefill_pair *sorted_pairs, uint32_t *per_expert_offsets,
                                            uint32_t *per_expert_counts, tf_prefill_group *groups, uint32_t *group_count,
                                            tf_prefill_tile *tiles, uint32_t *tile_count);
/* The same grouping (no sort keys) done on the DEVICE straight from the router's outputs, so a resident-expert pipeline
 * needs no host round trip: sorted_pairs[T*top_k] ordered by (expert, token, rank), per_expert_offsets / per_expert_counts
 * [num_experts], and a work list `chunks` (runs of <= 128 sorted pairs sharing one expert) with its length in chunk_count[0].
 * chunks capacity: num_experts + T*top_k/128 entries.  Expert ids are clamped to num_experts - 1
 * (RealForwardRunner.swift:955); the experts of one token must be distinct (the router guarantees it). */
int32_t tf_prefill_group_pairs_device(tf_ctx *ctx, tf_stream stream, const void *indices, const void *weights,
                                      uint32_t query_count, uint32_t top_k, uint32_t num_experts,
                                      void *sorted_pairs, void *per_expert_offsets, void *per_expert_counts,
                                      void *chunks, void *chunk_count);

/* PrefillGroupedRoutedMoE.encodeStreamedBatched (PrefillGroupedRoutedMoE.swift:386-461) -> prefill_grouped_routed_moe_
 * batched_phase1 / _down (prefill.metal:598-670): for the sorted pairs [pair_start, pair_start + pair_count) of one tile,
 * route_partials[(token*top_k + rank)*d + c] = half(down_c . half(gelu(gate . x) * (up . x))), unweighted.  `blobs`: HOST array
 * of live_expert_count device pointers bound to params->local_expert[i].  `tile_groups`: HOST array, the groups of this tile
 * (PrefillMoEGroupedRoutes.groups[tile.groupStart ..< tile.groupStart + tile.groupCount]).  Pairs are processed in
 * micro-batches of pair_microbatch_rows (reference default 32) so that gate_up_act_scratch needs 3 * rows * F halves and
 * down_scratch rows * d halves, as in the reference; *out_microbatches (may be NULL) receives the micro-batch count.
 * Pairs whose expert is not bound are skipped. */
int32_t tf_prefill_grouped_routed_moe_streamed(tf_ctx *ctx, tf_stream stream,
                                               const void *hidden, uint64_t hidden_offset,
                                               const void *sorted_pairs, uint64_t sorted_pairs_offset,
                                               void *route_partials, uint64_t route_partials_offset,
                                               void *gate_up_act_scratch, uint64_t gate_up_act_scratch_offset,
                                               void *down_scratch, uint64_t down_scratch_offset,
                                               const void *const *blobs, const tf_prefill_streamed_params *params,
                                               const tf_prefill_group *tile_groups, uint32_t tile_group_count,
                                               int32_t pair_microbatch_rows, int32_t *out_microbatches, tf_dtype scale_dtype);
/* tf_prefill_router_gemma4_block followed by tf_prefill_group_pairs_device on its outputs, as one call with every output of
 * both (PrefillRouter.encodeGemma4Block, PrefillRouter.swift:37-89, then makeTokenExpertPairs + groupTokenExpertPairs,
 * PrefillRouter.swift:91-111 and PrefillMoEGrouping.swift:90-193, which the reference runs on the host between two command
 * buffers).  For up to 32 token rows and top_k <= 8 the selection and the grouping share one launch; results are bit-identical
 * to the two calls, which larger calls are forwarded to. */
int32_t tf_prefill_router_group_block(tf_ctx *ctx, tf_stream stream,
                                      const void *weights, uint64_t weights_offset,
                                      const void *scales, uint64_t scales_offset,
                                      const void *biases, uint64_t biases_offset,
                                      const void *hidden, uint64_t hidden_offset,
                                      const void *effective_scale, uint64_t effective_scale_offset,
                                      const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                      void *out_indices, uint64_t out_indices_offset,
                                      void *out_weights, uint64_t out_weights_offset,
                                      uint32_t query_count, uint32_t num_experts, uint32_t d, uint32_t top_k,
                                      uint32_t hidden_stride_elements,
                                      void *sorted_pairs, void *per_expert_offsets, void *per_expert_counts,
                                      void *chunks, void *chunk_count);
/* A few token rows (multi-token verification: up to 32, top_k == 8, experts in a resident pool) through the whole routed path
 * as ONE call: tf_prefill_router_group_block, tf_prefill_grouped_routed_moe_resident and tf_prefill_moe_reduce_token_major
 * (PrefillRouter.encodeGemma4Block, PrefillRouter.swift:37-89; the host grouping, PrefillMoEGrouping.swift:90-193;
 * PrefillGroupedRoutedMoE.encodeStreamedBatched, PrefillGroupedRoutedMoE.swift:386-461; PrefillMoE.encodeReduceTokenMajor,
 * PrefillMoE.swift:11-38; in RealForwardRunner.swift:922-1156 the router reads routerX and the experts routedX, hence the two
 * hidden arguments).  Outputs: out_indices uint32[T, 8], out_weights fp16[T, 8] (the router's), route_partials fp16[T, 8, d]
 * (unweighted, as the grouped call leaves them), h2 fp16[T, d].  acts_scratch: T * 8 * f halves.
 * Up to five rows (at most 128 experts, a multiple of 4; d in (1024, 4096]; f <= 1024; 16-byte aligned operands, strides
 * multiples of 8) take three launches of their own, in which nothing is sorted: every block of the gate / up launch repeats
 * its token's selection and finds the other tokens that chose its expert by counting, the first such token's blocks read the
 * expert's rows once for all of them; the down launch reads each expert in use once and adds a token's eight partial results
 * in rank order itself.  Same arithmetic as the three calls (fp16 activations and partials, fused multiply-adds in rank order);
 * sums inside a dot product are taken in another order, so these rows agree with the three calls to rounding, not bit for bit.
 * More rows, and shapes the three launches do not take, go through the three calls themselves (from six rows on their
 * persistent kernels are faster), with the grouping's outputs kept in the context: bit-identical to making the calls.
 * Returns TF_ERR_UNAVAILABLE, with nothing enqueued, for more than 32 rows or another top_k. */
int32_t tf_prefill_routed_moe_few_tokens(tf_ctx *ctx, tf_stream stream,
                                         const void *weights, uint64_t weights_offset,
                                         const void *scales, uint64_t scales_offset,
                                         const void *biases, uint64_t biases_offset,
                                         const void *hidden, uint64_t hidden_offset,
                                         const void *effective_scale, uint64_t effective_scale_offset,
                                         const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                         void *out_indices, uint64_t out_indices_offset,
                                         void *out_weights, uint64_t out_weights_offset,
                                         uint32_t query_count, uint32_t num_experts, uint32_t d, uint32_t top_k,
                                         uint32_t hidden_stride_elements,
                                         const void *routed_hidden, uint64_t routed_hidden_offset,
                                         uint32_t routed_hidden_stride_elements,
                                         const void *expert_pool, uint64_t expert_pool_stride,
                                         const tf_expert_offsets *routed_offsets,
                                         void *acts_scratch, void *route_partials, void *h2, uint64_t h2_offset,
                                         uint32_t f, tf_dtype scale_dtype);
/* Resident-pool form of the same computation over ALL sorted pairs of a chunk of tokens in one go: experts are
 * pool + expert * pool_stride, the work list comes from tf_prefill_group_pairs_device, nothing is read by the host.  Groups
 * of a few pairs stream each expert row once and apply it to every routed token (weight-read bound, the small-M regime);
 * large groups run as a grouped GEMM on the matrix cores (weights expanded to fp16 in LDS, fp32 accumulation).
 * hidden holds pair_count / top_k token rows and every (token, rank) combination appears once among the pairs.
 * acts_scratch: pair_count * f halves.  max_chunks: capacity of `chunks`. */
int32_t tf_prefill_grouped_routed_moe_resident(tf_ctx *ctx, tf_stream stream,
                                               const void *hidden, uint64_t hidden_offset, uint32_t hidden_stride_elements,
                                               const void *sorted_pairs, const void *chunks, const void *chunk_count,
                                               uint32_t max_chunks, uint32_t pair_count,
                                               const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                               const tf_expert_offsets *routed_offsets,
                                               void *acts_scratch, void *route_partials,
                                               uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype);
/* tf_prefill_grouped_routed_moe_resident and tf_prefill_shared_expert_int4_block of the same token rows as one call
 * (the reference encodes them back to back in one command buffer: the routed stages of PrefillGroupedRoutedMoE.swift:386-461,
 * then PrefillSharedExpert.encodeBlock, PrefillSharedExpert.swift:12-67).  Neither reads what the other writes, so the
 * shared expert's matrix-core tiles are placed ahead of the routed tiles in the same two launches (gate / up / GeGLU, then
 * down) instead of under-filling the chip in launches of their own; results are bit-identical to the two calls.
 * Applies when the routed pairs go to the matrix-core tile kernels and the shared expert is 4-bit with at least 8 rows and
 * 16-byte aligned operands; otherwise the two calls are made one after the other.  Arguments: those of the routed call, then
 * those of the shared call (its d is the routed d, its scale dtype the routed one; query_count token rows). */
int32_t tf_prefill_grouped_routed_moe_resident_shared(tf_ctx *ctx, tf_stream stream,
                                               const void *hidden, uint64_t hidden_offset, uint32_t hidden_stride_elements,
                                               const void *sorted_pairs, const void *chunks, const void *chunk_count,
                                               uint32_t max_chunks, uint32_t pair_count,
                                               const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                               const tf_expert_offsets *routed_offsets,
                                               void *acts_scratch, void *route_partials,
                                               uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                               const void *shared_x, uint64_t shared_x_offset,
                                               void *shared_y, uint64_t shared_y_offset,
                                               const tf_projection *shared_gate, const tf_projection *shared_up,
                                               const tf_projection *shared_down,
                                               void *scratch_gate, uint64_t scratch_gate_offset, uint64_t scratch_gate_length,
                                               void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                                               void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length,
                                               uint32_t query_count, uint32_t shared_intermediate,
                                               uint32_t shared_x_stride_elements, uint32_t shared_y_stride_elements,
                                               uint32_t shared_weight_bits);
/* PrefillMoE.encodeReduceTokenMajor (Kernels/Prefill/MoE/PrefillMoE.swift:11-38) -> prefill_moe_reduce_token_major
 * (prefill.metal:575-596): h2[t, c] = half(sum_r float(w[t, r]) * float(partial[t, r, c])), r ascending, fused multiply-adds. */
int32_t tf_prefill_moe_reduce_token_major(tf_ctx *ctx, tf_stream stream,
                                          const void *route_partials, uint64_t route_partials_offset,
                                          const void *route_weights, uint64_t route_weights_offset,
                                          void *h2, uint64_t h2_offset, uint32_t query_count, uint32_t top_k, uint32_t d);

/* MPPPrefillInt4QMM.encode (Kernels/TensorCore/MPPPrefillInt4QMM.swift:34-77) -> mpp_prefill_affine_threadgroup_f16
 * (Metal/TensorCore/tensorops.metal:13-105): y[m, n] fp16 [M, N] = x[M, K] . W[N, K]^T, weights expanded to fp16
 * half(q*s+b) per K group, fp32 accumulation on the matrix cores.  Returns TF_ERR_UNAVAILABLE (the reference's
 * Path.unavailable) when m, n, k <= 0, k % 64 != 0, an operand is not 16-byte aligned or the matrix has fewer than six
 * groups in all (n * k / 64 < 6: the tiles stage scales six at a time); nothing is enqueued then. */
int32_t tf_int4_qmm(tf_ctx *ctx, tf_stream stream,
                    const void *weights, uint64_t weights_offset,
                    const void *scales, uint64_t scales_offset,
                    const void *biases, uint64_t biases_offset,
                    const void *x, uint64_t x_offset, void *y, uint64_t y_offset,
                    int32_t m, int32_t n, int32_t k, tf_dtype scale_dtype);
/* PrefillInt4QMM.encode (Kernels/Prefill/Primitives/PrefillPrimitives.swift:73-109) -> prefill_dequant_int4_qmm_f16_block
 * (prefill.metal:672-709): the same product with fp32 weights q*s+b (no fp16 rounding of the weight): every token row
 * goes through the GEMV arithmetic, so QMM == repeated GEMV.  Any 2-byte alignment. */
int32_t tf_prefill_int4_qmm(tf_ctx *ctx, tf_stream stream,
                            const void *weights, uint64_t weights_offset,
                            const void *scales, uint64_t scales_offset,
                            const void *biases, uint64_t biases_offset,
                            const void *x, uint64_t x_offset, void *y, uint64_t y_offset,
                            int32_t t, int32_t n, int32_t k, tf_dtype scale_dtype);

/* ---- neighbours of the output head --------------------------------------------------------------------------- */
/* EmbedLookupInt4.encode (Kernels/Quant/EmbedLookupInt4.swift:11-41) -> embed_lookup_int4
 * (Metal/Quant/dequant_int4.metal:63-83): out[i] = half((q_i * s + b) * out_scale) for row token_id of the tied int4
 * table [table_rows, d/2], scales/biases bf16 [table_rows, d/64]; d % 64 == 0.  table_rows has no counterpart in the
 * Metal wrapper (which cannot check the token): a token outside the table is rejected here instead of read. */
int32_t tf_embed_lookup_int4(tf_ctx *ctx, tf_stream stream, const void *table, uint64_t table_offset, const void *scales,
                             uint64_t scales_offset, const void *biases, uint64_t biases_offset, void *out, uint64_t out_offset,
                             uint32_t token_id, uint32_t d, float out_scale, uint32_t table_rows);
/* PrefillEmbedLookupInt4.encode (Kernels/Prefill/Primitives/PrefillPrimitives.swift:11-38) -> prefill_embed_lookup_int4_block
 * (Metal/Prefill/prefill.metal:26-52): the same for t tokens read from the DEVICE array tokens[t] (uint32), out [t, d].
 * A token >= table_rows reads the last row. */
int32_t tf_prefill_embed_lookup_int4_block(tf_ctx *ctx, tf_stream stream, const void *table, uint64_t table_offset, const void *scales,
                                           uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *tokens,
                                           uint64_t tokens_offset, void *out, uint64_t out_offset, uint32_t t, uint32_t d, float out_scale,
                                           uint32_t table_rows);
/* LogitSoftcapSoftmax.encode (Kernels/Sampling/LogitOutput.swift:11-30) -> logit_softcap_softmax
 * (Metal/Sampling/logit.metal:52-124): probs[i] = half(softmax_i(softcap * tanh(logits / softcap))), probs fp16[v].
 * logits_dtype: TF_FP16 (the reference's) or TF_FP32 (what tf_lm_head_logits_int4 can write). */
int32_t tf_logit_softcap_softmax(tf_ctx *ctx, tf_stream stream, const void *logits, void *probs, uint32_t v, float softcap,
                                 tf_dtype logits_dtype);
/* Sample.encode (Kernels/Sampling/LogitOutput.swift:40-71) -> sample (Metal/Sampling/logit.metal:183-447).
 * probs fp16[v] -> out_token uint32[1].  temperature <= 0: argmax (lowest index on ties).  top_k == 0 and top_p outside
 * (0, 1): Gumbel-max draw from p^(1/T) with counter-based noise keyed by (seed, position, index).  Otherwise: the
 * min(top_k or v, 256) most probable, cut where their cumulative mass reaches top_p, reweighted by p^(1/T), one
 * inverse-CDF draw with xorshift64* seeded by `seed` (which must be non-zero). */
int32_t tf_sample(tf_ctx *ctx, tf_stream stream, const void *probs, void *out_token, uint32_t v, float temperature, uint32_t top_k,
                  float top_p, uint64_t seed, uint32_t position);
/* SampleTopK64.encode (Kernels/Sampling/LogitOutput.swift:150-206) -> sample_topk64_stage1 / _reduce / _final
 * (Metal/Sampling/logit.metal:449-606): the top-64 sampler through sorted 1024-entry tiles; same token as
 * tf_sample(..., top_k = 64, ...).  vocab in 1...262144 (SampleTopK64Error.unsupportedVocabulary otherwise). */
int32_t tf_sample_topk64(tf_ctx *ctx, tf_stream stream, const void *probs, void *out_token, uint32_t vocab, float temperature, float top_p,
                         uint64_t seed);

/* ---- resident experts ------------------------------------------------------------------------------------------ */
/* Fills a caller-owned device pool [num_experts, expert_stride] from one packed-experts layer file
 * (packed_experts/layer_XX.bin: num_experts blobs of expert_stride bytes), placing LOGICAL expert e, stored at position
 * physical_rank[e] of the file (host array; NULL = identity), at pool + e * expert_stride.  Replaces the reference's SSD
 * streamer + slot cache (Runtime/Inference/ModelExpertIO.swift:45-110, Infrastructure/Streaming/PreadExpertStreamer.swift) with one
 * upload per layer; the layout comes from packed_experts/layout.json (GTurboPackedExpertsLayoutV1.swift).
 * Blocks until the upload is complete.  The file must be a regular file of exactly num_experts * expert_stride bytes
 * (TF_ERR_DIMENSION_MISMATCH otherwise). */
int32_t tf_upload_packed_experts_layer(tf_ctx *ctx, tf_stream stream, const char *layer_file_path, uint64_t expert_stride,
                                       uint32_t num_experts, const uint32_t *physical_rank, void *device_pool);

/* ResidentBuffer.init (Infrastructure/ModelIO/ResidentBuffer.swift:15-78) for a discrete GPU: where the reference maps
 * [file_offset, file_offset + bytes) of model_weights.bin into one shared MTLBuffer, this copies the range into
 * `device_dst` (bytes long, caller-owned) through two pinned staging buffers.  The path must be a regular file that
 * holds the whole range (TF_ERR_DIMENSION_MISMATCH otherwise).  Blocks until the copy is complete.  The index that
 * says which tensor lives where inside the range is read on the host (tf::gturbo::loadResidentIndex). */
int32_t tf_upload_file_region(tf_ctx *ctx, tf_stream stream, const char *file_path, uint64_t file_offset, uint64_t bytes,
                              void *device_dst);

#ifdef __cplusplus
}
#endif
#endif /* TF_KERNELS_H */

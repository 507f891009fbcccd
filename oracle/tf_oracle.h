/*
 * tf_oracle.h — CPU restatement of the reference's FP32 validation path.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing in the product (the HIP library, its C ABI,
 * the host mirror) may include, link or call anything declared here.  The only
 * legitimate callers are the test suite, the smoke check and the benchmark's
 * CPU-baseline leg, and there only as the checker / the thing timed beside the
 * GPU path — never as a fallback.
 *
 * Every function restates one piece of the reference (Swift); the citation after
 * each declaration names the reference file and lines it follows.  Paths are
 * relative to the reference checkout:
 *   Q   = Sources/TurboFieldfare/Infrastructure/ModelIO/Quantization.swift
 *   VS  = Sources/TurboFieldfareValidation/Support
 *   T   = Tests/TurboFieldfare/Core
 *   M   = Sources/TurboFieldfare/Metal
 *
 * Arithmetic the reference delegates to Apple Accelerate (vDSP_dotpr,
 * vDSP_svesq, vDSP_vmul, vDSP_vsmul, vDSP_vadd — closed source, unavailable on
 * Linux) is restated as a plain sequential fp32 loop; the reference's own tests
 * pin that substitution at 1e-5 relative
 * (T/Validation/Reference/DequantInt4GEMVReferenceTests.swift:32-53,
 *  T/Validation/Reference/RMSNormReferenceTests.swift:28-43).
 *
 * Parity pinning status (see tests/test_oracle_*.py for the checks):
 *   every function below is pinned by a known answer, a library routine or a
 *   brute-force/closed-form check EXCEPT the summation order inside Accelerate
 *   and the ulp behaviour of Metal's fast::exp/tanh/rsqrt/simd_sum, which no
 *   test here can pin; the tfo_k_* "kernel order" restatements are pinned only
 *   against the tfo_*_ref functions within fp16 tolerance (they exist to tighten
 *   GPU comparisons, not to define parity).
 */
#ifndef TF_ORACLE_H
#define TF_ORACLE_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { TFO_GROUP_SIZE = 64 }; /* Q:5 */

/* ---- scalar codecs ------------------------------------------------------- */
uint16_t tfo_bf16_bits(float x);            /* Q:17-23  round-half-even, no NaN special case */
float    tfo_bf16_to_float(uint16_t bits);  /* Q:25-28 */
uint16_t tfo_f16_bits(float x);             /* Swift Float16(Float): IEEE RNE (VS/Buffers/Fp16Buffer.swift:8) */
float    tfo_f16_to_float(uint16_t bits);   /* Swift Float(Float16)  (VS/Buffers/Fp16Buffer.swift:47-53) */

/* ---- seeded streams ------------------------------------------------------ */
uint64_t tfo_splitmix64_next(uint64_t *state);                      /* VS/PRNG/SplitMix64.swift:11-17 */
float    tfo_splitmix64_uniform(uint64_t *state, float lo, float hi); /* VS/PRNG/SplitMix64.swift:20-23 */
uint64_t tfo_seedtree_key(uint64_t root, const char *label);        /* VS/PRNG/SeedTree.swift:12-19; returns the child's initial state */
void     tfo_fill_uniform(uint64_t *state, float lo, float hi, float *out, int64_t n);

/* ---- affine quantizer (test-fixture quantizer of the reference) ----------- */
void tfo_quantize_int4_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases);     /* Q:51-103 */
void tfo_dequantize_int4_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int n, float *out); /* Q:105-119 */
void tfo_quantize_int8_affine(const float *row, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases);     /* Q:137-177 */
void tfo_dequantize_int8_affine(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int n, float *out); /* Q:179-191 */
/* row-major [m, n] convenience wrappers around the four above */
void tfo_quantize_int4_matrix(const float *w, int m, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases);
void tfo_quantize_int8_matrix(const float *w, int m, int n, uint8_t *packed, uint16_t *scales, uint16_t *biases);
void tfo_dequantize_int4_matrix(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int m, int n, float *out);
void tfo_dequantize_int8_matrix(const uint8_t *packed, const uint16_t *scales, const uint16_t *biases, int m, int n, float *out);

/* ---- error metrics -------------------------------------------------------- */
float tfo_rel_error(const float *actual, const float *reference, int64_t n);            /* VS/Tolerance/RelError.swift:7-16 */
float tfo_max_abs_diff(const float *a, const float *b, int64_t n);                      /* VS/Tolerance/RelError.swift:18-25 */
float tfo_bounded_rel(const float *actual, const float *reference, int64_t n, float abs_floor); /* VS/Tolerance/RelError.swift:30-43 */

/* ---- GEMV references ("the Swift CPU path") ------------------------------- */
/* y[r] = dot(dequant(W[r,:]), x): bulk-dequantise one row into a scratch fp32
 * row, then an fp32 dot.  threads<=1: serial (what the reference is);
 * threads>1: OpenMP over rows (same per-row arithmetic, identical results). */
void tfo_int4_gemv_ref(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x,
                       float *y, int64_t m, int n, int threads);   /* VS/Reference/Quant/DequantInt4Gemv.swift:12-43 */
void tfo_int8_gemv_ref(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x,
                       float *y, int64_t m, int n, int threads);   /* VS/Reference/Quant/DequantInt8Gemv.swift:12-41 */
/* same sums carried in double: the "truth" both fp32 orders are judged against (not in the reference) */
void tfo_int4_gemv_f64(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x,
                       double *y, int64_t m, int n);
void tfo_int8_gemv_f64(const uint8_t *W, const uint16_t *S, const uint16_t *B, const float *x,
                       double *y, int64_t m, int n);

/* ---- primitives ------------------------------------------------------------ */
void tfo_gelu_tanh(const float *x, float *y, int64_t n);                       /* VS/Reference/MoE/Moe.swift:22-30 */
void tfo_rmsnorm_ref(const float *x, const float *weight, float eps, float *y, int d); /* VS/Reference/Primitives/RmsNorm.swift:14-45 */

/* ---- MoE references --------------------------------------------------------- */
/* The nine byte offsets inside one expert blob (Sources/TurboFieldfare/Kernels/MoE/MoE.swift:4-29). */
typedef struct tfo_expert_offsets {
    uint32_t gate_W_off, gate_s_off, gate_b_off;
    uint32_t up_W_off, up_s_off, up_b_off;
    uint32_t down_W_off, down_s_off, down_b_off;
} tfo_expert_offsets;

/* down(gelu(gate x) * up x), everything fp32 */
void tfo_moe_run_ffn(const uint8_t *blob, const tfo_expert_offsets *off, const float *x,
                     float *y, int d, int f);                                  /* VS/Reference/MoE/Moe.swift:34-53 */
/* y = residual + sum_slot w[slot] * ffn(blobs[slot], x); blobs[slot] already selected by the caller */
void tfo_moe_apply_streamed_routed(const uint8_t *const *blobs, const tfo_expert_offsets *off,
                                   const float *x, const float *residual, const float *routing_w,
                                   int n_slots, float *y, int d, int f, int threads); /* VS/Reference/MoE/Moe.swift:60-89 */
/* Router reference: logits = int8 gemv(hidden*effective_scale); top-k by (value desc, index asc);
 * softmax over the selected; weight = p * expert_scale[idx]. */
void tfo_router_reference(const uint8_t *W, const uint16_t *S, const uint16_t *B,
                          const float *hidden, const float *effective_scale, const float *expert_scale,
                          int num_experts, int d, int top_k,
                          uint32_t *out_indices, float *out_weights, float *out_logits /* may be NULL */);
                                                                               /* T/Kernels/MoE/RouterTopKTests.swift:72-97 */
/* Shared expert reference: gate/up fp32, GeGLU via double tanh, act rounded to fp16, down fp32. */
void tfo_shared_expert_ref(const uint8_t *gW, const uint16_t *gS, const uint16_t *gB,
                           const uint8_t *uW, const uint16_t *uS, const uint16_t *uB,
                           const uint8_t *dW, const uint16_t *dS, const uint16_t *dB,
                           const float *x, float *y, int d, int f, int threads);
                                                                               /* T/Kernels/MoE/SharedExpertInt4Tests.swift:19-28 */

/* ---- lm_head ------------------------------------------------------------------ */
/* RMSNorm (bf16 weight) -> fp16 -> per-row dequant+dot -> strict-greater argmax (first max wins,
 * NaN never wins, nothing wins => 0).  logits_out may be NULL. */
uint32_t tfo_lm_head_cpu_greedy(const uint16_t *hidden_f16, const uint16_t *norm_w_bf16,
                                const uint8_t *W, const uint16_t *S, const uint16_t *B,
                                int d, int64_t v, float eps, float *logits_out, int threads);
                                                                               /* T/Kernels/Fusions/LMHeadChainInt4Tests.swift:10-39 */

/* ---- prefill ---------------------------------------------------------------------- */
typedef struct tfo_pair {           /* Sources/TurboFieldfare/Kernels/Prefill/MoE/PrefillRouter.swift:5-28 (16 bytes) */
    uint32_t token, expert, rank, weight_bits_and_reserved;
} tfo_pair;
typedef struct tfo_group { uint32_t expert, pair_start, pair_count; } tfo_group;   /* .../PrefillMoEGrouping.swift:4-14 */
typedef struct tfo_tile  { uint32_t group_start, group_count, pair_start, pair_count; } tfo_tile; /* :17-29 */

/* error codes of tfo_prefill_group_pairs = the reference's PrefillMoEGroupingError cases (:52-63) */
enum {
    TFO_GROUP_OK = 0,
    TFO_GROUP_INVALID_QUERY_COUNT = 1, TFO_GROUP_INVALID_TOP_K = 2, TFO_GROUP_INVALID_NUM_EXPERTS = 3,
    TFO_GROUP_INVALID_TILE_EXPERT_COUNT = 4, TFO_GROUP_PAIR_COUNT_MISMATCH = 5, TFO_GROUP_TOKEN_OUT_OF_RANGE = 6,
    TFO_GROUP_RANK_OUT_OF_RANGE = 7, TFO_GROUP_EXPERT_OUT_OF_RANGE = 8, TFO_GROUP_DUPLICATE_TOKEN_RANK = 9,
    TFO_GROUP_SORT_KEY_COUNT_MISMATCH = 10
};
/* sorted_pairs[pair_count]; offsets/counts[num_experts]; groups/tiles sized by caller to >= min(num_experts, pairs).
 * expert_sort_keys may be NULL (sort_key_count ignored then). */
int tfo_prefill_group_pairs(const tfo_pair *pairs, int64_t pair_count, int query_count, int top_k, int num_experts,
                            int tile_expert_count, const uint64_t *expert_sort_keys, int sort_key_count,
                            tfo_pair *sorted_pairs, uint32_t *per_expert_offsets, uint32_t *per_expert_counts,
                            tfo_group *groups, int *n_groups, tfo_tile *tiles, int *n_tiles);
                                                                               /* .../PrefillMoEGrouping.swift:90-193 */
void tfo_prefill_make_pairs(const uint32_t *indices, const uint16_t *weights_f16, int query_count, int top_k,
                            tfo_pair *pairs);                                  /* .../PrefillRouter.swift:91-111 */
/* acc += (q*scale+bias)*x over one row of a blob-resident matrix */
float tfo_prefill_cpu_int4_dot(const uint8_t *bytes, int64_t base, int64_t w_off, int64_t s_off, int64_t b_off,
                               int row, int n, const float *x);               /* T/Kernels/Prefill/PrefillGroupedRoutedMoETests.swift:275-303 */
/* per (token, rank): act = f16(gelu(gate)*up), partial = f16(down . act); out pre-filled with fill_f16 */
void tfo_prefill_route_partials(const tfo_pair *sorted_pairs, int64_t pair_count, int query_count,
                                const uint16_t *hidden_f16, int hidden_stride,
                                const uint8_t *pool, int64_t pool_stride, const tfo_expert_offsets *off,
                                int top_k, int d, int f, uint16_t fill_f16, uint16_t *out_f16, int threads);
                                                                               /* T/Kernels/Prefill/PrefillGroupedRoutedMoETests.swift:229-273 */
void tfo_prefill_reduce_token_major(const uint16_t *partials_f16, const uint16_t *weights_f16,
                                    int rows, int top_k, int d, uint16_t *out_f16); /* T/Kernels/Prefill/PrefillMoETests.swift:46-64 */
/* Y[t, r] = f16( fma-chain over k of (q*s+b) * x[t,k] ), returned as fp32 of that fp16 */
void tfo_qmm_cpu_reference(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *x_f16,
                           int m, int n, int k, float *out, int threads);     /* T/Kernels/TensorCore/MPPPrefillInt4QMMTests.swift:80-105 */

/* ---- kernel-order restatements (follow the Metal kernels' rounding points) -------------------
 * Lane-parallel sums are taken lane 0..31 in order; the hardware reduction tree is not specified
 * by the reference, so these agree with the device only to fp32 rounding. */
void tfo_k_int4_gemv(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *x_f16,
                     float *y_f32, int64_t m, int n);                          /* M/Quant/dequant_int4.metal:93-171 (value before the final half()) */
void tfo_k_router_logits(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *hidden_f16,
                         const uint16_t *eff_scale_bf16, float *logits, int num_experts, int d); /* M/MoE/moe.metal:78-117 */
void tfo_k_router_topk(const float *logits, const uint16_t *per_expert_scale_bf16, int num_experts, int top_k,
                       uint32_t *out_indices, uint16_t *out_weights_f16);       /* M/MoE/moe.metal:135-185 (top_k==8) and M/Prefill/prefill.metal:527-572 (generic) */
void tfo_k_moe_phase1(const uint8_t *const *blobs, const tfo_expert_offsets *off, const uint16_t *x_f16,
                      uint16_t *acts_f16, int d, int f, int top_k);            /* M/MoE/moe.metal:339-369 */
void tfo_k_moe_phase2(const uint8_t *const *blobs, const tfo_expert_offsets *off, const uint16_t *acts_f16,
                      const uint16_t *routing_w_f16, const uint16_t *residual_f16, uint16_t *y_f16,
                      int d, int f);                                            /* M/MoE/moe.metal:446-482 */
void tfo_k_gelu_mul_fp16(const uint16_t *gate_f16, const uint16_t *up_f16, uint16_t *out_f16, int n); /* M/Primitives/utility.metal:6-18 */
void tfo_embed_lookup_int4(const uint8_t *table, const uint16_t *S, const uint16_t *B, uint32_t token, int d, float out_scale, float *out); /* VS/Reference/Quant/EmbedLookup.swift:41-68 */
void tfo_logit_softcap_softmax_ref(const float *x, int v, float softcap, float *out); /* VS/Reference/Sampling/LogitSoftcapSoftmax.swift:12-48 */
uint64_t tfo_sampler_xorshift64(uint64_t *state);                                      /* M/Sampling/logit.metal:148-153 */
float tfo_sampler_gumbel(uint64_t seed, uint32_t position, uint32_t row);              /* M/Sampling/logit.metal:165-181 */
uint32_t tfo_sample(const uint16_t *probs_f16, uint32_t v, float temperature, uint32_t top_k, float top_p, uint64_t seed, uint32_t position); /* M/Sampling/logit.metal:183-447 */
uint32_t tfo_sample_topk64(const uint16_t *probs_f16, uint32_t v, float temperature, float top_p, uint64_t seed); /* M/Sampling/logit.metal:449-606 */
void tfo_k_post_attn_setup(uint16_t *hidden_f16, const uint16_t *attn_f16, const uint16_t *w_post_attn_bf16,
                           const uint16_t *w_pre_ffn_bf16, const uint16_t *w_pre_ffn2_bf16, float eps, uint16_t *dense_f16,
                           uint16_t *routed_f16, uint16_t *router_f16, int d); /* M/Fusions/fused.metal:190-269 */
void tfo_k_layer_tail(const uint16_t *h2_f16, const uint16_t *h1_f16, uint16_t *hidden_f16, const uint16_t *w_postffn2_bf16,
                      const uint16_t *w_postffn_bf16, float eps, float layer_scalar, int d); /* M/Fusions/fused.metal:271-375 */
void tfo_layer_tail_ref(const uint16_t *h2_f16, const uint16_t *h1_f16, const uint16_t *hidden_f16, const uint16_t *w_postffn2_bf16,
                        const uint16_t *w_postffn_bf16, float eps, float layer_scalar, float *out, int d); /* T/Core/Kernels/Fusions/FusedLayerTailTests.swift:76-92 */
void tfo_k_rmsnorm_bf16w(const uint16_t *x_f16, const uint16_t *w_bf16, float eps, uint16_t *out_f16, int d); /* M/Primitives/rmsnorm.metal:32-93 */
void tfo_k_rmsnorm_rows(const uint16_t *x_f16, const uint16_t *w_bf16, float eps, uint16_t *out_f16, int tokens, int heads, int d,
                        int token_stride); /* M/Primitives/rmsnorm.metal:100-175, M/Prefill/prefill.metal:86-176 */
void tfo_k_prefill_router_logits(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *hidden_f16,
                                 const uint16_t *eff_scale_bf16, float *logits, int num_experts, int d); /* M/Prefill/prefill.metal:503-525 */
float tfo_k_prefill_int4_row(const uint8_t *W, const uint16_t *S, const uint16_t *B, const uint16_t *x_f16,
                             int row, int n);                                  /* M/Prefill/prefill.metal:406-440 */

/* decode attention: AttentionRef.apply, the kernel-order split-KV path, Attention.splitGeometry */
void tfo_attention_ref(const float *q, const float *k, const float *v, int head_dim, int num_q_heads, int num_kv_heads, int seq_len,
                       int window, float scale, float *out);
void tfo_k_attention_split(const uint16_t *q_f16, const uint16_t *k_f16, const uint16_t *v_f16, int head_dim, int num_q_heads,
                           int num_kv_heads, int seq_len, int kv_start, int chunk_len, int num_chunks, float scale, int ring_capacity,
                           uint16_t *out_f16);
void tfo_attention_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len, uint32_t kv_start, int prefer_gqa_swa,
                                  int32_t *out5);

/* causal attention of a block of query tokens (prefill): the test-embedded reference and the kernel-order path */
void tfo_prefill_attention_ref(const float *q, const float *k, const float *v, int start, int chunk, int head_dim, int q_heads, int kv_heads,
                               int kv_valid, int window, int q_stride, int kv_stride, float scale, float *out);
void tfo_k_prefill_attention(const uint16_t *q_f16, const uint16_t *k_f16, const uint16_t *v_f16, uint16_t *out_f16, int start, int chunk,
                             int head_dim, int q_heads, int kv_heads, int kv_valid, int window, int q_stride, int kv_stride, int o_stride,
                             float scale, int ring_capacity);

/* RoPE (NeoX pairs) and the fused per-head Q/K/V epilogue */
void tfo_rope_neox_ref(const float *input, int num_tokens, int num_heads, int head_dim, int rotated_pairs, int position, float theta,
                       float *out);
void tfo_k_rope_neox(uint16_t *data_f16, int num_tokens, int num_heads, int head_dim, int rotated_pairs, uint32_t position, float theta);
void tfo_k_fused_qkv_epilogue(uint16_t *q_f16, uint16_t *k_f16, uint16_t *v_f16, const uint16_t *q_weight_bf16, const uint16_t *k_weight_bf16,
                              int head_dim, int num_q_heads, int num_kv_heads, uint32_t position, float theta, int rotated_pairs, float eps);

#ifdef __cplusplus
}
#endif
#endif /* TF_ORACLE_H */

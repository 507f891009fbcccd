// Rotary position embedding (NeoX pairing) and the per-head Q/K/V epilogue: RMSNorm per head (q and k with a bf16 weight
// shared by all heads, v without), then rotation of the first `rotated_pairs` pairs of q and k, in place.  For one token
// (decode) and for a block of tokens at consecutive positions with padded token rows (prefill): the same kernels, so a block
// equals its tokens done one by one, bit for bit.
#include <math.h>

#include "tf_common.hpp"
#include "tf_context.hpp"

using namespace tfk;

namespace {

constexpr uint32_t kEpilogueMaxHeadDim = 512;   // the reference's threadgroup scratch (fused.metal kFusedMaxHeadDim)

// (x0, x1) rotated by angle position * theta^(-2 pair / head_dim); accurate sine / cosine: angles reach position itself
__device__ __forceinline__ void rope_pair(float &x0, float &x1, uint32_t pair, uint32_t head_dim, float position, float theta) {
    const float exponent = -(float)(2u * pair) / (float)head_dim;
    const float angle = position * powf(theta, exponent);
    float sn, c;
    sincosf(angle, &sn, &c);
    const float r0 = x0 * c - x1 * sn, r1 = x0 * sn + x1 * c;
    x0 = r0;
    x1 = r1;
}

// grid (pair blocks, heads, tokens): head h of token t starts at t * token_stride + h * head_dim and sits at position
// position + t * position_step
__global__ __launch_bounds__(256) void rope_neox_kernel(half_t *data, uint32_t position, uint32_t position_step, uint32_t head_dim,
                                                        uint32_t token_stride, float theta, uint32_t rotated_pairs) {
    const uint32_t pair = blockIdx.x * blockDim.x + threadIdx.x;
    if (pair >= rotated_pairs) return;
    const uint32_t half_dim = head_dim / 2;
    half_t *head = data + (size_t)blockIdx.z * token_stride + (size_t)blockIdx.y * head_dim;
    float x0 = (float)head[pair], x1 = (float)head[half_dim + pair];
    rope_pair(x0, x1, pair, head_dim, (float)(position + blockIdx.z * position_step), theta);
    head[pair] = (half_t)x0;
    head[half_dim + pair] = (half_t)x1;
}

// one block per head and token (grid (heads, tokens)): q heads, then k heads, then v heads; token t at position + t
__global__ __launch_bounds__(256) void qkv_epilogue_kernel(half_t *q, half_t *k, half_t *v, const uint16_t *q_weight, const uint16_t *k_weight,
                                                           uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t position,
                                                           float theta, uint32_t rotated_pairs, float eps, uint32_t q_token_stride,
                                                           uint32_t kv_token_stride) {
    __shared__ half_t normed[kEpilogueMaxHeadDim];
    __shared__ float partial[4];
    const uint32_t hg = blockIdx.x, t = blockIdx.y;
    position += t;
    const bool is_q = hg < num_q_heads, is_k = !is_q && hg < num_q_heads + num_kv_heads;
    half_t *dst = is_q ? q + (size_t)t * q_token_stride + (size_t)hg * head_dim
                       : (is_k ? k + (size_t)t * kv_token_stride + (size_t)(hg - num_q_heads) * head_dim
                               : v + (size_t)t * kv_token_stride + (size_t)(hg - num_q_heads - num_kv_heads) * head_dim);
    const uint16_t *w = is_q ? q_weight : k_weight;
    float acc = 0.0f;
    for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x) {
        const float xv = (float)dst[i];
        acc = fmaf(xv, xv, acc);
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float inv = 1.0f / sqrtf(((partial[0] + partial[1]) + (partial[2] + partial[3])) / (float)head_dim + eps);
    for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x) {
        float xv = (float)dst[i] * inv;
        if (is_q || is_k) xv *= bf16_to_f32(w[i]);
        asm volatile("" : "+v"(xv));   // the fp32 product is rounded to half, not fused into the conversion
        normed[i] = (half_t)xv;
    }
    __syncthreads();
    if (!is_q && !is_k) {
        for (uint32_t i = threadIdx.x; i < head_dim; i += blockDim.x) dst[i] = normed[i];
        return;
    }
    const uint32_t half_dim = head_dim / 2;
    for (uint32_t pair = threadIdx.x; pair < half_dim; pair += blockDim.x) {
        float x0 = (float)normed[pair], x1 = (float)normed[half_dim + pair];
        if (pair < rotated_pairs) rope_pair(x0, x1, pair, head_dim, (float)position, theta);
        dst[pair] = (half_t)x0;
        dst[half_dim + pair] = (half_t)x1;
    }
}

int32_t launch_rope(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t position, uint32_t position_step, uint32_t head_dim,
                    uint32_t num_heads, uint32_t num_tokens, uint32_t token_stride, float theta, uint32_t rotated_pairs, const char *who) {
    TF_REQUIRE(ctx, ctx && data, TF_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    TF_REQUIRE(ctx, head_dim % 2 == 0, TF_ERR_INVALID_ARGUMENT, "%s: head_dim must be even", who);
    TF_REQUIRE(ctx, (uint64_t)rotated_pairs * 2 <= head_dim, TF_ERR_INVALID_ARGUMENT, "%s: rotatedPairs * 2 must not exceed head_dim", who);
    TF_REQUIRE(ctx, data_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT, "%s: offsets must be 2-byte aligned", who);
    TF_REQUIRE(ctx, num_heads <= 65535 && num_tokens <= 65535, TF_ERR_INVALID_ARGUMENT, "%s: more than 65535 heads or tokens", who);
    if (rotated_pairs == 0 || num_heads == 0 || num_tokens == 0) return TF_OK;
    const dim3 grid((rotated_pairs + 255) / 256, num_heads, num_tokens);
    hipLaunchKernelGGL(rope_neox_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), reinterpret_cast<half_t *>(at(data, data_offset)),
                       position, position_step, head_dim, token_stride, theta, rotated_pairs);
    return check_launch(ctx, who);
}

int32_t launch_qkv_epilogue(tf_ctx *ctx, tf_stream stream, void *q, uint64_t q_offset, void *k, uint64_t k_offset, void *v, uint64_t v_offset,
                            const void *q_weight, uint64_t q_weight_offset, const void *k_weight, uint64_t k_weight_offset, uint32_t head_dim,
                            uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t position, uint32_t tokens, uint32_t q_token_stride,
                            uint32_t kv_token_stride, float theta, uint32_t rotated_pairs, float eps, const char *who) {
    TF_REQUIRE(ctx, ctx && q && k && v && q_weight && k_weight, TF_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    TF_REQUIRE(ctx, head_dim > 0 && head_dim <= kEpilogueMaxHeadDim, TF_ERR_INVALID_ARGUMENT, "headDim > 512 exceeds the fused QKV epilogue scratch");
    TF_REQUIRE(ctx, head_dim % 2 == 0, TF_ERR_INVALID_ARGUMENT, "%s: head_dim must be even", who);
    TF_REQUIRE(ctx, (uint64_t)rotated_pairs * 2 <= head_dim, TF_ERR_INVALID_ARGUMENT, "rotatedPairs must fit inside one NeoX head");
    TF_REQUIRE(ctx, q_offset % 2 == 0 && k_offset % 2 == 0 && v_offset % 2 == 0 && q_weight_offset % 2 == 0 && k_weight_offset % 2 == 0,
               TF_ERR_INVALID_ARGUMENT, "%s: offsets must be 2-byte aligned", who);
    TF_REQUIRE(ctx, tokens <= 65535, TF_ERR_INVALID_ARGUMENT, "%s: more than 65535 tokens", who);
    const uint32_t groups = num_q_heads + 2 * num_kv_heads;
    if (groups == 0 || tokens == 0) return TF_OK;
    hipLaunchKernelGGL(qkv_epilogue_kernel, dim3(groups, tokens), dim3(256), 0, static_cast<hipStream_t>(stream),
                       reinterpret_cast<half_t *>(at(q, q_offset)), reinterpret_cast<half_t *>(at(k, k_offset)), reinterpret_cast<half_t *>(at(v, v_offset)),
                       reinterpret_cast<const uint16_t *>(at(q_weight, q_weight_offset)), reinterpret_cast<const uint16_t *>(at(k_weight, k_weight_offset)),
                       head_dim, num_q_heads, num_kv_heads, position, theta, rotated_pairs, eps, q_token_stride, kv_token_stride);
    return check_launch(ctx, who);
}

}  // namespace

extern "C" {

int32_t tf_rope_default_neox(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t position, uint32_t head_dim,
                             uint32_t num_heads, uint32_t num_tokens, float theta) {
    return launch_rope(ctx, stream, data, data_offset, position, 0, head_dim, num_heads, num_tokens, num_heads * head_dim, theta, head_dim / 2,
                       "rope_default_neox");
}

int32_t tf_rope_proportional_neox(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t position, uint32_t head_dim,
                                  uint32_t num_heads, uint32_t num_tokens, uint32_t rotated_pairs, float theta) {
    return launch_rope(ctx, stream, data, data_offset, position, 0, head_dim, num_heads, num_tokens, num_heads * head_dim, theta, rotated_pairs,
                       "rope_proportional_neox");
}

int32_t tf_prefill_rope_default_neox_block(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t start_position,
                                           uint32_t query_count, uint32_t head_dim, uint32_t num_heads, uint32_t token_stride_elements, float theta) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "prefill_rope_default_neox_block: null context");
    TF_REQUIRE(ctx, query_count > 0, TF_ERR_INVALID_ARGUMENT, "queryCount must be positive");
    TF_REQUIRE(ctx, (uint64_t)token_stride_elements >= (uint64_t)num_heads * head_dim, TF_ERR_INVALID_ARGUMENT, "token stride is too small");
    return launch_rope(ctx, stream, data, data_offset, start_position, 1, head_dim, num_heads, query_count, token_stride_elements, theta, head_dim / 2,
                       "prefill_rope_default_neox_block");
}

int32_t tf_prefill_rope_proportional_neox_block(tf_ctx *ctx, tf_stream stream, void *data, uint64_t data_offset, uint32_t start_position,
                                                uint32_t query_count, uint32_t head_dim, uint32_t num_heads, uint32_t rotated_pairs,
                                                uint32_t token_stride_elements, float theta) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "prefill_rope_proportional_neox_block: null context");
    TF_REQUIRE(ctx, query_count > 0, TF_ERR_INVALID_ARGUMENT, "queryCount must be positive");
    TF_REQUIRE(ctx, (uint64_t)token_stride_elements >= (uint64_t)num_heads * head_dim, TF_ERR_INVALID_ARGUMENT, "token stride is too small");
    return launch_rope(ctx, stream, data, data_offset, start_position, 1, head_dim, num_heads, query_count, token_stride_elements, theta, rotated_pairs,
                       "prefill_rope_proportional_neox_block");
}

int32_t tf_fused_qkv_epilogue(tf_ctx *ctx, tf_stream stream, void *q, uint64_t q_offset, void *k, uint64_t k_offset, void *v, uint64_t v_offset,
                              const void *q_weight, uint64_t q_weight_offset, const void *k_weight, uint64_t k_weight_offset, uint32_t head_dim,
                              uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t position, float theta, uint32_t rotated_pairs, float eps) {
    return launch_qkv_epilogue(ctx, stream, q, q_offset, k, k_offset, v, v_offset, q_weight, q_weight_offset, k_weight, k_weight_offset, head_dim,
                               num_q_heads, num_kv_heads, position, 1, 0, 0, theta, rotated_pairs, eps, "fused_qkv_epilogue");
}

int32_t tf_prefill_qkv_epilogue_block(tf_ctx *ctx, tf_stream stream, void *q, uint64_t q_offset, void *k, uint64_t k_offset, void *v,
                                      uint64_t v_offset, const void *q_weight, uint64_t q_weight_offset, const void *k_weight,
                                      uint64_t k_weight_offset, uint32_t start_position, uint32_t query_count, uint32_t head_dim,
                                      uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t q_token_stride_elements,
                                      uint32_t kv_token_stride_elements, float theta, uint32_t rotated_pairs, float eps) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "prefill_qkv_epilogue_block: null context");
    // PrefillQKVEpilogue.encode's preconditions (PrefillQKVEpilogue.swift:34-43)
    TF_REQUIRE(ctx, query_count > 0, TF_ERR_INVALID_ARGUMENT, "queryCount must be positive");
    TF_REQUIRE(ctx, head_dim > 0 && head_dim % 2 == 0, TF_ERR_INVALID_ARGUMENT, "headDim must be positive and even");
    TF_REQUIRE(ctx, num_q_heads > 0, TF_ERR_INVALID_ARGUMENT, "numQHeads must be positive");
    TF_REQUIRE(ctx, num_kv_heads > 0, TF_ERR_INVALID_ARGUMENT, "numKVHeads must be positive");
    TF_REQUIRE(ctx, rotated_pairs > 0, TF_ERR_INVALID_ARGUMENT, "rotatedPairs must be positive");
    TF_REQUIRE(ctx, (uint64_t)rotated_pairs * 2 <= head_dim, TF_ERR_INVALID_ARGUMENT, "rotatedPairs must fit inside one head");
    TF_REQUIRE(ctx, (uint64_t)q_token_stride_elements >= (uint64_t)num_q_heads * head_dim, TF_ERR_INVALID_ARGUMENT, "Q token stride is too small");
    TF_REQUIRE(ctx, (uint64_t)kv_token_stride_elements >= (uint64_t)num_kv_heads * head_dim, TF_ERR_INVALID_ARGUMENT, "KV token stride is too small");
    return launch_qkv_epilogue(ctx, stream, q, q_offset, k, k_offset, v, v_offset, q_weight, q_weight_offset, k_weight, k_weight_offset, head_dim,
                               num_q_heads, num_kv_heads, start_position, query_count, q_token_stride_elements, kv_token_stride_elements, theta,
                               rotated_pairs, eps, "prefill_qkv_epilogue_block");
}

}  // extern "C"

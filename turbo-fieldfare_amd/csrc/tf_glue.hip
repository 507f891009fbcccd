// The two element-wise/normalisation stages that bracket the MoE block of a decoder layer, for one token or a block of
// token rows: post-attention setup (produces the three inputs of the FFN sandwich) and the layer tail (folds the two FFN
// branches back into the residual stream).  One 256-thread block per row; a row (at most 4096 values) lives in registers
// between its two reductions, so each operand is read once and each result written once.
#include "tf_context.hpp"
#include "tf_rowdot.hpp"

using namespace tfk;

namespace {

constexpr uint32_t kGlueMaxD = 4096;   // the reference's threadgroup scratch (fused.metal kFusedMaxD, prefill.metal kPrefillPostMaxD)
constexpr int kPerThread = 16;         // kGlueMaxD / 256

// fp32 -> fp16 -> fp32.  The empty asm pins the operand as an fp32 value first: without it the compiler may fold the
// multiply that produced it into the conversion (v_fma_mixlo_f16: one rounding of the exact product), which is not what
// the reference computes (an fp32 product, then rounded to half) and differs from it near ties.
__device__ __forceinline__ float round_half(float v) {
    asm volatile("" : "+v"(v));
    return (float)(half_t)v;
}

// The elements of a row owned by one thread: two runs of 8 consecutive elements.  VEC moves a run with one 16-byte access
// (d % 8 == 0 and every row base 16-byte aligned); otherwise element by element (any even alignment, any d).  Ownership,
// and with it the order of every sum, is the same in both forms, so results do not depend on alignment or row stride.
template <bool VEC>
struct RowSlice {
    uint32_t d;

    __device__ __forceinline__ uint32_t index(int j) const {
        return (threadIdx.x + 256u * (uint32_t)(j >> 3)) * 8u + (uint32_t)(j & 7);
    }
    __device__ __forceinline__ bool live(int j) const { return index(j) < d; }

    // 16-bit elements widened by `widen` (fp16 or bf16 -> fp32); elements past the row read as 0
    template <typename F>
    __device__ __forceinline__ void load(const uint16_t *row, float *v, F widen) const {
        if constexpr (VEC) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                u32x4 r = {0u, 0u, 0u, 0u};
                if (live(8 * p)) r = load16(row + index(8 * p));
#pragma unroll
                for (int j = 0; j < 8; ++j) v[8 * p + j] = widen((uint16_t)(r[j >> 1] >> (16 * (j & 1))));
            }
        } else {
#pragma unroll
            for (int j = 0; j < kPerThread; ++j) v[j] = live(j) ? widen(row[index(j)]) : 0.0f;
        }
    }
    __device__ __forceinline__ void load_f16(const half_t *row, float *v) const {
        load(reinterpret_cast<const uint16_t *>(row), v, [](uint16_t b) { return f16_to_f32(b); });
    }
    __device__ __forceinline__ void load_bf16(const uint16_t *row, float *v) const {
        load(row, v, [](uint16_t b) { return bf16_to_f32(b); });
    }
    // v holds values already rounded to fp16 precision
    __device__ __forceinline__ void store_f16(half_t *row, const float *v) const {
        if constexpr (VEC) {
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                if (!live(8 * p)) continue;
                u32x4 r;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const half2_t h = {(half_t)v[8 * p + 2 * j], (half_t)v[8 * p + 2 * j + 1]};
                    r[j] = as_u32(h);
                }
                *reinterpret_cast<u32x4 *>(row + index(8 * p)) = r;
            }
        } else {
#pragma unroll
            for (int j = 0; j < kPerThread; ++j)
                if (live(j)) row[index(j)] = (half_t)v[j];
        }
    }
};

// 1 / sqrt(mean(v^2) + eps) over the block's row; partial: 4 floats of LDS not in use by another reduction in flight
__device__ __forceinline__ float block_inv_rms(const float *v, uint32_t d, float eps, float *partial) {
    float acc = 0.0f;
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) acc = fmaf(v[j], v[j], acc);
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    return 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)d + eps);
}

struct PostAttnArgs {
    half_t *hidden;
    const half_t *attn;
    half_t *dense_x, *routed_x, *router_x;
    const uint16_t *w_post_attn, *w_pre_ffn, *w_pre_ffn2;
    uint32_t rows, d;
    uint32_t hidden_stride, attn_stride, dense_stride, routed_stride, router_stride;
    float eps;
};

// hidden <- half(hidden + half(attn * inv_rms(attn) * w_post_attn));  with h = hidden * inv_rms(hidden):
// dense_x = half(h * w_pre_ffn), routed_x = half(h * w_pre_ffn2), router_x = half(h).
template <bool VEC>
__global__ __launch_bounds__(256) void post_attn_setup_kernel(PostAttnArgs a) {
    __shared__ float partial[2][4];
    const uint32_t row = blockIdx.x;
    const RowSlice<VEC> rs{a.d};
    float at[kPerThread], w[kPerThread], h[kPerThread], w2[kPerThread], w3[kPerThread];
    rs.load_f16(a.attn + (size_t)row * a.attn_stride, at);
    rs.load_bf16(a.w_post_attn, w);
    rs.load_f16(a.hidden + (size_t)row * a.hidden_stride, h);
    rs.load_bf16(a.w_pre_ffn, w2);
    rs.load_bf16(a.w_pre_ffn2, w3);
    const float attn_inv = block_inv_rms(at, a.d, a.eps, partial[0]);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) h[j] = round_half(h[j] + round_half(at[j] * attn_inv * w[j]));
    rs.store_f16(a.hidden + (size_t)row * a.hidden_stride, h);
    const float hidden_inv = block_inv_rms(h, a.d, a.eps, partial[1]);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const float hn = h[j] * hidden_inv;
        w2[j] = round_half(hn * w2[j]);
        w3[j] = round_half(hn * w3[j]);
        h[j] = round_half(hn);
    }
    rs.store_f16(a.dense_x + (size_t)row * a.dense_stride, w2);
    rs.store_f16(a.routed_x + (size_t)row * a.routed_stride, w3);
    rs.store_f16(a.router_x + (size_t)row * a.router_stride, h);
}

struct LayerTailArgs {
    const half_t *h2, *h1;
    half_t *hidden;
    const uint16_t *w_postffn2, *w_postffn;
    const uint16_t *w_postffn1;   // not null: h1 is the shared expert's raw output and is normalised here first
    uint32_t rows, d;
    uint32_t h2_stride, h1_stride, hidden_stride;
    float eps, layer_scalar;
};

// h12 = half(h1 + half(h2 * inv_rms(h2) * w_postffn2));
// hidden <- half(half(hidden + half(h12 * inv_rms(h12) * w_postffn)) * half(layer_scalar)).
// NORM_H1: h1 <- half(h1 * inv_rms(h1) * w_postffn1) first (rmsnorm_bf16w of the shared expert's output, otherwise a launch
// of its own between the shared expert and this kernel).
template <bool VEC, bool NORM_H1>
__global__ __launch_bounds__(256) void layer_tail_kernel(LayerTailArgs a) {
    __shared__ float partial[3][4];
    const uint32_t row = blockIdx.x;
    const RowSlice<VEC> rs{a.d};
    float x[kPerThread], w[kPerThread], h1[kPerThread], wp[kPerThread], hid[kPerThread];
    rs.load_f16(a.h2 + (size_t)row * a.h2_stride, x);
    rs.load_bf16(a.w_postffn2, w);
    rs.load_f16(a.h1 + (size_t)row * a.h1_stride, h1);
    rs.load_bf16(a.w_postffn, wp);
    rs.load_f16(a.hidden + (size_t)row * a.hidden_stride, hid);
    if constexpr (NORM_H1) {
        float w1[kPerThread];
        rs.load_bf16(a.w_postffn1, w1);
        const float inv_h1 = block_inv_rms(h1, a.d, a.eps, partial[2]);
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) h1[j] = round_half(h1[j] * inv_h1 * w1[j]);
    }
    const float inv_h2 = block_inv_rms(x, a.d, a.eps, partial[0]);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) x[j] = round_half(h1[j] + round_half(x[j] * inv_h2 * w[j]));
    const float inv_h12 = block_inv_rms(x, a.d, a.eps, partial[1]);
    const float scale = round_half(a.layer_scalar);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) hid[j] = round_half(round_half(hid[j] + round_half(x[j] * inv_h12 * wp[j])) * scale);
    rs.store_f16(a.hidden + (size_t)row * a.hidden_stride, hid);
}

bool rows_vectorizable(const void *base, uint32_t stride, uint32_t rows) {
    return aligned16(base) && (rows == 1 || stride % 8 == 0);
}

int32_t post_attn_setup_entry(tf_ctx *ctx, tf_stream stream, const char *who, void *hidden, uint64_t hidden_offset, const void *attn,
                              uint64_t attn_offset, void *dense_x, uint64_t dense_offset, void *routed_x, uint64_t routed_offset,
                              void *router_x, uint64_t router_offset, const void *w_post, uint64_t w_post_offset, const void *w_pre,
                              uint64_t w_pre_offset, const void *w_pre2, uint64_t w_pre2_offset, uint32_t rows, uint32_t d,
                              uint32_t hidden_stride, uint32_t attn_stride, uint32_t dense_stride, uint32_t routed_stride,
                              uint32_t router_stride, float eps) {
    TF_REQUIRE(ctx, ctx && hidden && attn && dense_x && routed_x && router_x && w_post && w_pre && w_pre2, TF_ERR_INVALID_ARGUMENT,
               "%s: null argument", who);
    TF_REQUIRE(ctx, rows > 0, TF_ERR_INVALID_ARGUMENT, "%s: queryCount must be positive", who);
    TF_REQUIRE(ctx, d > 0 && d <= kGlueMaxD, TF_ERR_INVALID_ARGUMENT, "%s: D must be in 1...4096, got %u", who, d);
    TF_REQUIRE(ctx, hidden_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: hidden stride is too small", who);
    TF_REQUIRE(ctx, attn_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: attention stride is too small", who);
    TF_REQUIRE(ctx, dense_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: dense stride is too small", who);
    TF_REQUIRE(ctx, routed_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: routed stride is too small", who);
    TF_REQUIRE(ctx, router_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: router stride is too small", who);
    PostAttnArgs a;
    a.hidden = reinterpret_cast<half_t *>(at(hidden, hidden_offset));
    a.attn = reinterpret_cast<const half_t *>(at(attn, attn_offset));
    a.dense_x = reinterpret_cast<half_t *>(at(dense_x, dense_offset));
    a.routed_x = reinterpret_cast<half_t *>(at(routed_x, routed_offset));
    a.router_x = reinterpret_cast<half_t *>(at(router_x, router_offset));
    a.w_post_attn = reinterpret_cast<const uint16_t *>(at(w_post, w_post_offset));
    a.w_pre_ffn = reinterpret_cast<const uint16_t *>(at(w_pre, w_pre_offset));
    a.w_pre_ffn2 = reinterpret_cast<const uint16_t *>(at(w_pre2, w_pre2_offset));
    TF_REQUIRE(ctx, aligned(a.hidden, 2) && aligned(a.attn, 2) && aligned(a.dense_x, 2) && aligned(a.routed_x, 2) && aligned(a.router_x, 2) &&
                   aligned(a.w_post_attn, 2) && aligned(a.w_pre_ffn, 2) && aligned(a.w_pre_ffn2, 2),
               TF_ERR_INVALID_ARGUMENT, "%s: misaligned operand", who);
    a.rows = rows;
    a.d = d;
    a.hidden_stride = hidden_stride;
    a.attn_stride = attn_stride;
    a.dense_stride = dense_stride;
    a.routed_stride = routed_stride;
    a.router_stride = router_stride;
    a.eps = eps;
    const bool vec = d % 8 == 0 && rows_vectorizable(a.hidden, hidden_stride, rows) && rows_vectorizable(a.attn, attn_stride, rows) &&
                     rows_vectorizable(a.dense_x, dense_stride, rows) && rows_vectorizable(a.routed_x, routed_stride, rows) &&
                     rows_vectorizable(a.router_x, router_stride, rows) && aligned16(a.w_post_attn) && aligned16(a.w_pre_ffn) &&
                     aligned16(a.w_pre_ffn2);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec) hipLaunchKernelGGL(post_attn_setup_kernel<true>, dim3(rows), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(post_attn_setup_kernel<false>, dim3(rows), dim3(256), 0, st, a);
    return check_launch(ctx, who);
}

int32_t layer_tail_entry(tf_ctx *ctx, tf_stream stream, const char *who, const void *h2, uint64_t h2_offset, const void *h1,
                         uint64_t h1_offset, void *hidden, uint64_t hidden_offset, const void *w_postffn1, uint64_t w_postffn1_offset,
                         const void *w_postffn2, uint64_t w_postffn2_offset,
                         const void *w_postffn, uint64_t w_postffn_offset, uint32_t rows, uint32_t d, uint32_t h2_stride,
                         uint32_t h1_stride, uint32_t hidden_stride, float eps, float layer_scalar) {
    TF_REQUIRE(ctx, ctx && h2 && h1 && hidden && w_postffn2 && w_postffn, TF_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    TF_REQUIRE(ctx, rows > 0, TF_ERR_INVALID_ARGUMENT, "%s: queryCount must be positive", who);
    TF_REQUIRE(ctx, d > 0 && d <= kGlueMaxD, TF_ERR_INVALID_ARGUMENT, "%s: D must be in 1...4096, got %u", who, d);
    TF_REQUIRE(ctx, h2_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: h2 stride is too small", who);
    TF_REQUIRE(ctx, h1_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: h1 stride is too small", who);
    TF_REQUIRE(ctx, hidden_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: hidden stride is too small", who);
    LayerTailArgs a;
    a.h2 = reinterpret_cast<const half_t *>(at(h2, h2_offset));
    a.h1 = reinterpret_cast<const half_t *>(at(h1, h1_offset));
    a.hidden = reinterpret_cast<half_t *>(at(hidden, hidden_offset));
    a.w_postffn2 = reinterpret_cast<const uint16_t *>(at(w_postffn2, w_postffn2_offset));
    a.w_postffn = reinterpret_cast<const uint16_t *>(at(w_postffn, w_postffn_offset));
    a.w_postffn1 = w_postffn1 ? reinterpret_cast<const uint16_t *>(at(w_postffn1, w_postffn1_offset)) : nullptr;
    TF_REQUIRE(ctx, aligned(a.h2, 2) && aligned(a.h1, 2) && aligned(a.hidden, 2) && aligned(a.w_postffn2, 2) && aligned(a.w_postffn, 2) &&
                   aligned(a.w_postffn1, 2),
               TF_ERR_INVALID_ARGUMENT, "%s: misaligned operand", who);
    a.rows = rows;
    a.d = d;
    a.h2_stride = h2_stride;
    a.h1_stride = h1_stride;
    a.hidden_stride = hidden_stride;
    a.eps = eps;
    a.layer_scalar = layer_scalar;
    const bool vec = d % 8 == 0 && rows_vectorizable(a.h2, h2_stride, rows) && rows_vectorizable(a.h1, h1_stride, rows) &&
                     rows_vectorizable(a.hidden, hidden_stride, rows) && aligned16(a.w_postffn2) && aligned16(a.w_postffn) &&
                     aligned16(a.w_postffn1);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (a.w_postffn1) {
        if (vec) hipLaunchKernelGGL((layer_tail_kernel<true, true>), dim3(rows), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((layer_tail_kernel<false, true>), dim3(rows), dim3(256), 0, st, a);
    } else {
        if (vec) hipLaunchKernelGGL((layer_tail_kernel<true, false>), dim3(rows), dim3(256), 0, st, a);
        else hipLaunchKernelGGL((layer_tail_kernel<false, false>), dim3(rows), dim3(256), 0, st, a);
    }
    return check_launch(ctx, who);
}

}  // namespace

extern "C" {

int32_t tf_fused_post_attn_setup(tf_ctx *ctx, tf_stream stream, void *hidden, const void *attn, void *dense_x, void *routed_x,
                                 void *router_x, const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                 const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset, const void *pre_ffn2_weight,
                                 uint64_t pre_ffn2_weight_offset, uint32_t d, float eps) {
    return post_attn_setup_entry(ctx, stream, "fused_post_attn_setup", hidden, 0, attn, 0, dense_x, 0, routed_x, 0, router_x, 0,
                                 post_attention_weight, post_attention_weight_offset, pre_ffn_weight, pre_ffn_weight_offset,
                                 pre_ffn2_weight, pre_ffn2_weight_offset, 1, d, d, d, d, d, d, eps);
}

int32_t tf_prefill_post_attn_setup_block(tf_ctx *ctx, tf_stream stream, void *hidden, uint64_t hidden_offset, const void *attn,
                                         uint64_t attn_offset, void *dense_x, uint64_t dense_x_offset, void *routed_x,
                                         uint64_t routed_x_offset, void *router_x, uint64_t router_x_offset,
                                         const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                         const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset, const void *pre_ffn2_weight,
                                         uint64_t pre_ffn2_weight_offset, uint32_t query_count, uint32_t d,
                                         uint32_t hidden_stride_elements, uint32_t attn_stride_elements,
                                         uint32_t dense_stride_elements, uint32_t routed_stride_elements,
                                         uint32_t router_stride_elements, float eps) {
    return post_attn_setup_entry(ctx, stream, "prefill_post_attn_setup_block", hidden, hidden_offset, attn, attn_offset, dense_x,
                                 dense_x_offset, routed_x, routed_x_offset, router_x, router_x_offset, post_attention_weight,
                                 post_attention_weight_offset, pre_ffn_weight, pre_ffn_weight_offset, pre_ffn2_weight,
                                 pre_ffn2_weight_offset, query_count, d, hidden_stride_elements, attn_stride_elements,
                                 dense_stride_elements, routed_stride_elements, router_stride_elements, eps);
}

int32_t tf_fused_layer_tail(tf_ctx *ctx, tf_stream stream, const void *h2, const void *h1, void *hidden, const void *post_ffn2_weight,
                            uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset, uint32_t d,
                            float eps, float layer_scalar) {
    return layer_tail_entry(ctx, stream, "fused_layer_tail", h2, 0, h1, 0, hidden, 0, nullptr, 0, post_ffn2_weight, post_ffn2_weight_offset,
                            post_ffn_weight, post_ffn_weight_offset, 1, d, d, d, d, eps, layer_scalar);
}

int32_t tf_fused_layer_tail_shared_norm(tf_ctx *ctx, tf_stream stream, const void *h2, const void *shared_out, void *hidden,
                                        const void *post_ffn1_weight, uint64_t post_ffn1_weight_offset, const void *post_ffn2_weight,
                                        uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset,
                                        uint32_t d, float eps, float layer_scalar) {
    TF_REQUIRE(ctx, ctx && post_ffn1_weight, TF_ERR_INVALID_ARGUMENT, "fused_layer_tail_shared_norm: null argument");
    return layer_tail_entry(ctx, stream, "fused_layer_tail_shared_norm", h2, 0, shared_out, 0, hidden, 0, post_ffn1_weight,
                            post_ffn1_weight_offset, post_ffn2_weight, post_ffn2_weight_offset, post_ffn_weight, post_ffn_weight_offset, 1, d,
                            d, d, d, eps, layer_scalar);
}

int32_t tf_prefill_layer_tail_block(tf_ctx *ctx, tf_stream stream, const void *h2, uint64_t h2_offset, const void *h1,
                                    uint64_t h1_offset, void *hidden, uint64_t hidden_offset, const void *post_ffn2_weight,
                                    uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset,
                                    uint32_t query_count, uint32_t d, uint32_t h2_stride_elements, uint32_t h1_stride_elements,
                                    uint32_t hidden_stride_elements, float eps, float layer_scalar) {
    return layer_tail_entry(ctx, stream, "prefill_layer_tail_block", h2, h2_offset, h1, h1_offset, hidden, hidden_offset, nullptr, 0,
                            post_ffn2_weight, post_ffn2_weight_offset, post_ffn_weight, post_ffn_weight_offset, query_count, d,
                            h2_stride_elements, h1_stride_elements, hidden_stride_elements, eps, layer_scalar);
}

}  // extern "C"

// The two element-wise/normalisation stages that bracket the MoE block of a decoder layer, for one token or a block of
// token rows: post-attention setup (produces the three inputs of the FFN sandwich) and the layer tail (folds the two FFN
// branches back into the residual stream).  One 256-thread block per row; a row (at most 4096 values) lives in registers
// between its two reductions, so each operand is read once and each result written once.
#include "tf_context.hpp"
#include "tf_rowslice.hpp"

using namespace tfk;

namespace {

struct PostAttnArgs {
    const half_t *hidden;
    half_t *hidden_out;      // may be `hidden` (in place)
    const half_t *attn;
    half_t *dense_x, *routed_x, *router_x;
    const uint16_t *w_post_attn, *w_pre_ffn, *w_pre_ffn2;
    uint32_t rows, d;
    uint32_t hidden_stride, hidden_out_stride, attn_stride, dense_stride, routed_stride, router_stride;
    float eps;
};

// hidden_out <- half(hidden + half(attn * inv_rms(attn) * w_post_attn));  with h = hidden_out * inv_rms(hidden_out):
// dense_x = half(h * w_pre_ffn), routed_x = half(h * w_pre_ffn2), router_x = half(h).
template <bool VEC>
__global__ __launch_bounds__(256) void post_attn_setup_kernel(PostAttnArgs a) {
    __shared__ float partial[8];
    const uint32_t row = blockIdx.x;
    const RowSlice<VEC> rs{a.d};
    float at[kPerThread], w[kPerThread], w2[kPerThread], w3[kPerThread];
    PostAttnRow<VEC> pr;
    rs.load_f16(a.attn + (size_t)row * a.attn_stride, at);
    rs.load_bf16(a.w_post_attn, w);
    rs.load_f16(a.hidden + (size_t)row * a.hidden_stride, pr.h);
    rs.load_bf16(a.w_pre_ffn, w2);
    rs.load_bf16(a.w_pre_ffn2, w3);
    pr.finish(rs, at, w, a.eps, partial);
    rs.store_f16(a.hidden_out + (size_t)row * a.hidden_out_stride, pr.h);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) {
        const float hn = pr.h[j] * pr.inv;
        w2[j] = round_half(hn * w2[j]);
        w3[j] = round_half(hn * w3[j]);
        pr.h[j] = round_half(hn);
    }
    rs.store_f16(a.dense_x + (size_t)row * a.dense_stride, w2);
    rs.store_f16(a.routed_x + (size_t)row * a.routed_stride, w3);
    rs.store_f16(a.router_x + (size_t)row * a.router_stride, pr.h);
}

struct LayerTailArgs {
    const half_t *h2, *h1;
    const half_t *hidden;
    half_t *hidden_out;            // may be `hidden` (in place)
    const uint16_t *w_postffn2, *w_postffn;
    const uint16_t *w_postffn1;   // not null: h1 is the shared expert's raw output and is normalised here first
    uint32_t rows, d;
    uint32_t h2_stride, h1_stride, hidden_stride;
    float eps, layer_scalar;
};

// layer_tail_row over one row per block.  NORM_H1: the norm of the shared expert's output (otherwise a launch of its own between
// the shared expert and this kernel) runs here first.
template <bool VEC, bool NORM_H1>
__global__ __launch_bounds__(256) void layer_tail_kernel(LayerTailArgs a) {
    __shared__ float partial[12];
    const uint32_t row = blockIdx.x;
    const RowSlice<VEC> rs{a.d};
    float x[kPerThread], w[kPerThread], h1[kPerThread], wp[kPerThread], hid[kPerThread], w1[kPerThread];
    rs.load_f16(a.h2 + (size_t)row * a.h2_stride, x);
    rs.load_bf16(a.w_postffn2, w);
    rs.load_f16(a.h1 + (size_t)row * a.h1_stride, h1);
    rs.load_bf16(a.w_postffn, wp);
    rs.load_f16(a.hidden + (size_t)row * a.hidden_stride, hid);
    if constexpr (NORM_H1) rs.load_bf16(a.w_postffn1, w1);
    layer_tail_row<NORM_H1>(a.d, x, w, h1, wp, hid, w1, a.eps, a.layer_scalar, partial);
    rs.store_f16(a.hidden_out + (size_t)row * a.hidden_stride, hid);
}

bool rows_vectorizable(const void *base, uint32_t stride, uint32_t rows) {
    return aligned16(base) && (rows == 1 || stride % 8 == 0);
}

int32_t post_attn_setup_entry(tf_ctx *ctx, tf_stream stream, const char *who, void *hidden_out, const void *hidden, uint64_t hidden_offset, const void *attn,
                              uint64_t attn_offset, void *dense_x, uint64_t dense_offset, void *routed_x, uint64_t routed_offset,
                              void *router_x, uint64_t router_offset, const void *w_post, uint64_t w_post_offset, const void *w_pre,
                              uint64_t w_pre_offset, const void *w_pre2, uint64_t w_pre2_offset, uint32_t rows, uint32_t d,
                              uint32_t hidden_stride, uint32_t attn_stride, uint32_t dense_stride, uint32_t routed_stride,
                              uint32_t router_stride, float eps) {
    TF_REQUIRE(ctx, ctx && hidden && hidden_out && attn && dense_x && routed_x && router_x && w_post && w_pre && w_pre2, TF_ERR_INVALID_ARGUMENT,
               "%s: null argument", who);
    TF_REQUIRE(ctx, rows > 0, TF_ERR_INVALID_ARGUMENT, "%s: queryCount must be positive", who);
    TF_REQUIRE(ctx, d > 0 && d <= kGlueMaxD, TF_ERR_INVALID_ARGUMENT, "%s: D must be in 1...4096, got %u", who, d);
    TF_REQUIRE(ctx, hidden_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: hidden stride is too small", who);
    TF_REQUIRE(ctx, attn_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: attention stride is too small", who);
    TF_REQUIRE(ctx, dense_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: dense stride is too small", who);
    TF_REQUIRE(ctx, routed_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: routed stride is too small", who);
    TF_REQUIRE(ctx, router_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: router stride is too small", who);
    PostAttnArgs a;
    a.hidden = reinterpret_cast<const half_t *>(at(hidden, hidden_offset));
    a.hidden_out = reinterpret_cast<half_t *>(at(hidden_out, hidden_offset));
    a.attn = reinterpret_cast<const half_t *>(at(attn, attn_offset));
    a.dense_x = reinterpret_cast<half_t *>(at(dense_x, dense_offset));
    a.routed_x = reinterpret_cast<half_t *>(at(routed_x, routed_offset));
    a.router_x = reinterpret_cast<half_t *>(at(router_x, router_offset));
    a.w_post_attn = reinterpret_cast<const uint16_t *>(at(w_post, w_post_offset));
    a.w_pre_ffn = reinterpret_cast<const uint16_t *>(at(w_pre, w_pre_offset));
    a.w_pre_ffn2 = reinterpret_cast<const uint16_t *>(at(w_pre2, w_pre2_offset));
    TF_REQUIRE(ctx, aligned(a.hidden, 2) && aligned(a.hidden_out, 2) && aligned(a.attn, 2) && aligned(a.dense_x, 2) && aligned(a.routed_x, 2) && aligned(a.router_x, 2) &&
                   aligned(a.w_post_attn, 2) && aligned(a.w_pre_ffn, 2) && aligned(a.w_pre_ffn2, 2),
               TF_ERR_INVALID_ARGUMENT, "%s: misaligned operand", who);
    a.rows = rows;
    a.d = d;
    a.hidden_stride = hidden_stride;
    a.hidden_out_stride = hidden_stride;
    a.attn_stride = attn_stride;
    a.dense_stride = dense_stride;
    a.routed_stride = routed_stride;
    a.router_stride = router_stride;
    a.eps = eps;
    const bool vec = d % 8 == 0 && rows_vectorizable(a.hidden, hidden_stride, rows) && rows_vectorizable(a.hidden_out, hidden_stride, rows) &&
                     rows_vectorizable(a.attn, attn_stride, rows) &&
                     rows_vectorizable(a.dense_x, dense_stride, rows) && rows_vectorizable(a.routed_x, routed_stride, rows) &&
                     rows_vectorizable(a.router_x, router_stride, rows) && aligned16(a.w_post_attn) && aligned16(a.w_pre_ffn) &&
                     aligned16(a.w_pre_ffn2);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (vec) hipLaunchKernelGGL(post_attn_setup_kernel<true>, dim3(rows), dim3(256), 0, st, a);
    else hipLaunchKernelGGL(post_attn_setup_kernel<false>, dim3(rows), dim3(256), 0, st, a);
    return check_launch(ctx, who);
}

int32_t layer_tail_entry(tf_ctx *ctx, tf_stream stream, const char *who, const void *h2, uint64_t h2_offset, const void *h1,
                         uint64_t h1_offset, void *hidden_out, const void *hidden, uint64_t hidden_offset, const void *w_postffn1, uint64_t w_postffn1_offset,
                         const void *w_postffn2, uint64_t w_postffn2_offset,
                         const void *w_postffn, uint64_t w_postffn_offset, uint32_t rows, uint32_t d, uint32_t h2_stride,
                         uint32_t h1_stride, uint32_t hidden_stride, float eps, float layer_scalar) {
    TF_REQUIRE(ctx, ctx && h2 && h1 && hidden && hidden_out && w_postffn2 && w_postffn, TF_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    TF_REQUIRE(ctx, rows > 0, TF_ERR_INVALID_ARGUMENT, "%s: queryCount must be positive", who);
    TF_REQUIRE(ctx, d > 0 && d <= kGlueMaxD, TF_ERR_INVALID_ARGUMENT, "%s: D must be in 1...4096, got %u", who, d);
    TF_REQUIRE(ctx, h2_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: h2 stride is too small", who);
    TF_REQUIRE(ctx, h1_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: h1 stride is too small", who);
    TF_REQUIRE(ctx, hidden_stride >= d, TF_ERR_INVALID_ARGUMENT, "%s: hidden stride is too small", who);
    LayerTailArgs a;
    a.h2 = reinterpret_cast<const half_t *>(at(h2, h2_offset));
    a.h1 = reinterpret_cast<const half_t *>(at(h1, h1_offset));
    a.hidden = reinterpret_cast<const half_t *>(at(hidden, hidden_offset));
    a.hidden_out = reinterpret_cast<half_t *>(at(hidden_out, hidden_offset));
    a.w_postffn2 = reinterpret_cast<const uint16_t *>(at(w_postffn2, w_postffn2_offset));
    a.w_postffn = reinterpret_cast<const uint16_t *>(at(w_postffn, w_postffn_offset));
    a.w_postffn1 = w_postffn1 ? reinterpret_cast<const uint16_t *>(at(w_postffn1, w_postffn1_offset)) : nullptr;
    TF_REQUIRE(ctx, aligned(a.h2, 2) && aligned(a.h1, 2) && aligned(a.hidden, 2) && aligned(a.hidden_out, 2) && aligned(a.w_postffn2, 2) && aligned(a.w_postffn, 2) &&
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
                     rows_vectorizable(a.hidden, hidden_stride, rows) && rows_vectorizable(a.hidden_out, hidden_stride, rows) && aligned16(a.w_postffn2) && aligned16(a.w_postffn) &&
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

namespace tfk {

// tf_fused_post_attn_setup with the new residual stream written to hidden_out instead of over hidden
int32_t post_attn_setup_to(tf_ctx *ctx, tf_stream stream, const void *hidden, void *hidden_out, const void *attn, void *dense_x, void *routed_x,
                           void *router_x, const void *w_post, uint64_t w_post_offset, const void *w_pre, uint64_t w_pre_offset,
                           const void *w_pre2, uint64_t w_pre2_offset, uint32_t d, float eps) {
    return post_attn_setup_entry(ctx, stream, "fused_post_attn_setup", hidden_out, hidden, 0, attn, 0, dense_x, 0, routed_x, 0, router_x, 0, w_post,
                                 w_post_offset, w_pre, w_pre_offset, w_pre2, w_pre2_offset, 1, d, d, d, d, d, d, eps);
}

// tf_fused_layer_tail_shared_norm with the layer's output written to hidden_out instead of over hidden
int32_t layer_tail_shared_norm_to(tf_ctx *ctx, tf_stream stream, const void *h2, const void *shared_out, const void *hidden, void *hidden_out,
                                  const void *w_postffn1, uint64_t w_postffn1_offset, const void *w_postffn2, uint64_t w_postffn2_offset,
                                  const void *w_postffn, uint64_t w_postffn_offset, uint32_t d, float eps, float layer_scalar) {
    TF_REQUIRE(ctx, ctx && w_postffn1, TF_ERR_INVALID_ARGUMENT, "fused_layer_tail_shared_norm: null argument");
    return layer_tail_entry(ctx, stream, "fused_layer_tail_shared_norm", h2, 0, shared_out, 0, hidden_out, hidden, 0, w_postffn1, w_postffn1_offset,
                            w_postffn2, w_postffn2_offset, w_postffn, w_postffn_offset, 1, d, d, d, d, eps, layer_scalar);
}

}  // namespace tfk

extern "C" {

int32_t tf_fused_post_attn_setup(tf_ctx *ctx, tf_stream stream, void *hidden, const void *attn, void *dense_x, void *routed_x,
                                 void *router_x, const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                 const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset, const void *pre_ffn2_weight,
                                 uint64_t pre_ffn2_weight_offset, uint32_t d, float eps) {
    return post_attn_setup_entry(ctx, stream, "fused_post_attn_setup", hidden, hidden, 0, attn, 0, dense_x, 0, routed_x, 0, router_x, 0,
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
    return post_attn_setup_entry(ctx, stream, "prefill_post_attn_setup_block", hidden, hidden, hidden_offset, attn, attn_offset, dense_x,
                                 dense_x_offset, routed_x, routed_x_offset, router_x, router_x_offset, post_attention_weight,
                                 post_attention_weight_offset, pre_ffn_weight, pre_ffn_weight_offset, pre_ffn2_weight,
                                 pre_ffn2_weight_offset, query_count, d, hidden_stride_elements, attn_stride_elements,
                                 dense_stride_elements, routed_stride_elements, router_stride_elements, eps);
}

int32_t tf_fused_layer_tail(tf_ctx *ctx, tf_stream stream, const void *h2, const void *h1, void *hidden, const void *post_ffn2_weight,
                            uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset, uint32_t d,
                            float eps, float layer_scalar) {
    return layer_tail_entry(ctx, stream, "fused_layer_tail", h2, 0, h1, 0, hidden, hidden, 0, nullptr, 0, post_ffn2_weight, post_ffn2_weight_offset,
                            post_ffn_weight, post_ffn_weight_offset, 1, d, d, d, d, eps, layer_scalar);
}

int32_t tf_fused_layer_tail_shared_norm(tf_ctx *ctx, tf_stream stream, const void *h2, const void *shared_out, void *hidden,
                                        const void *post_ffn1_weight, uint64_t post_ffn1_weight_offset, const void *post_ffn2_weight,
                                        uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset,
                                        uint32_t d, float eps, float layer_scalar) {
    TF_REQUIRE(ctx, ctx && post_ffn1_weight, TF_ERR_INVALID_ARGUMENT, "fused_layer_tail_shared_norm: null argument");
    return layer_tail_entry(ctx, stream, "fused_layer_tail_shared_norm", h2, 0, shared_out, 0, hidden, hidden, 0, post_ffn1_weight,
                            post_ffn1_weight_offset, post_ffn2_weight, post_ffn2_weight_offset, post_ffn_weight, post_ffn_weight_offset, 1, d,
                            d, d, d, eps, layer_scalar);
}

int32_t tf_prefill_layer_tail_block(tf_ctx *ctx, tf_stream stream, const void *h2, uint64_t h2_offset, const void *h1,
                                    uint64_t h1_offset, void *hidden, uint64_t hidden_offset, const void *post_ffn2_weight,
                                    uint64_t post_ffn2_weight_offset, const void *post_ffn_weight, uint64_t post_ffn_weight_offset,
                                    uint32_t query_count, uint32_t d, uint32_t h2_stride_elements, uint32_t h1_stride_elements,
                                    uint32_t hidden_stride_elements, float eps, float layer_scalar) {
    return layer_tail_entry(ctx, stream, "prefill_layer_tail_block", h2, h2_offset, h1, h1_offset, hidden, hidden, hidden_offset, nullptr, 0,
                            post_ffn2_weight, post_ffn2_weight_offset, post_ffn_weight, post_ffn_weight_offset, query_count, d,
                            h2_stride_elements, h1_stride_elements, hidden_stride_elements, eps, layer_scalar);
}

}  // extern "C"

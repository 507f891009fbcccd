// Declarations shared between the translation units of the kernel library.
#pragma once

#include <algorithm>

#include "tf_context.hpp"
#include "tf_rowdot.hpp"

namespace tfk {

// inv = 1 / sqrt(mean(x^2) + eps) over d fp16 values, computed by one 256-thread block; every thread gets it.
// `partial` is 4 floats of LDS.
__device__ __forceinline__ float block_rms_inv(const half_t *x, uint32_t d, float eps, float *partial) {
    float acc = 0.0f;
    for (uint32_t i = threadIdx.x; i < d; i += blockDim.x) {
        const float v = (float)x[i];
        acc = fmaf(v, v, acc);
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    float total = 0.0f;
    for (uint32_t w = 0; w < (blockDim.x >> 6); ++w) total += partial[w];
    return 1.0f / sqrtf(total / (float)d + eps);
}

// largest hidden size the row streamers normalise and stage themselves (XNormStage)
constexpr int kMaxFusedNormD = XStage::kMaxK;

int32_t launch_gemv4(tf_ctx *ctx, hipStream_t st, const uint8_t *w, const uint8_t *s, const uint8_t *b, const void *x,
                     void *y, uint32_t m, uint32_t n, tf_dtype sd, tf_dtype od, const void *norm_w = nullptr, float eps = 0.0f);
bool gemv4_can_fuse_norm(const uint8_t *w, const void *x, const void *norm_w, uint32_t n);
int32_t launch_rmsnorm_bf16w(tf_ctx *ctx, hipStream_t st, const void *x, const void *w, void *out, uint32_t d, float eps);
int32_t launch_gelu_mul(tf_ctx *ctx, hipStream_t st, const void *gate, const void *up, void *out, uint32_t count);
int32_t validate_gemv(tf_ctx *ctx, const char *who, const void *weights, uint64_t wo, const void *scales, uint64_t so,
                      const void *biases, uint64_t bo, const void *x, uint64_t xo, const void *y, uint64_t yo,
                      uint32_t m, uint32_t n, tf_dtype sd, tf_dtype od, unsigned weights_align);

// tf_fused_post_attn_setup with the new residual stream written to hidden_out instead of over hidden (tf_glue.hip)
int32_t post_attn_setup_to(tf_ctx *ctx, tf_stream stream, const void *hidden, void *hidden_out, const void *attn, void *dense_x, void *routed_x,
                           void *router_x, const void *w_post, uint64_t w_post_offset, const void *w_pre, uint64_t w_pre_offset,
                           const void *w_pre2, uint64_t w_pre2_offset, uint32_t d, float eps);
// tf_fused_layer_tail_shared_norm with the layer's output written to hidden_out instead of over hidden (tf_glue.hip)
int32_t layer_tail_shared_norm_to(tf_ctx *ctx, tf_stream stream, const void *h2, const void *shared_out, const void *hidden, void *hidden_out,
                                  const void *w_postffn1, uint64_t w_postffn1_offset, const void *w_postffn2, uint64_t w_postffn2_offset,
                                  const void *w_postffn, uint64_t w_postffn_offset, uint32_t d, float eps, float layer_scalar);

}  // namespace tfk

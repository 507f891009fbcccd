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

// rmsnorm_bf16w computed by one 256-thread block straight into LDS: xn[i] = half(x[i] * inv * w[i]).
// k % 8 == 0, k <= 8192, x and w 16-byte aligned.  Every thread requests its (at most four) 8-element chunks of both
// operands before using any.  Ends with a barrier: xn is readable by the whole block on return.
constexpr int kMaxFusedNormD = 8192;
__device__ __forceinline__ void block_rmsnorm_to_lds(const half_t *x, const uint16_t *w_bf16, float eps, int k, half_t *xn,
                                                     float *partial) {
    const int nchunks = k >> 3;
    u32x4 xr[4], wr[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int c = threadIdx.x + 256 * p;
        xr[p] = wr[p] = u32x4{0u, 0u, 0u, 0u};
        if (c < nchunks) {
            xr[p] = load16(x + c * 8);
            wr[p] = load16(w_bf16 + c * 8);
        }
    }
    float acc = 0.0f;
#pragma unroll
    for (int p = 0; p < 4; ++p)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t h = as_half2(xr[p][j]);
            acc = fmaf((float)h[0], (float)h[0], acc);
            acc = fmaf((float)h[1], (float)h[1], acc);
        }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float inv = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)k + eps);
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const int c = threadIdx.x + 256 * p;
        if (c < nchunks) {
            u32x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half2_t h = as_half2(xr[p][j]);
                half2_t n;
                n[0] = (half_t)((float)h[0] * inv * __uint_as_float(wr[p][j] << 16));
                n[1] = (half_t)((float)h[1] * inv * __uint_as_float(wr[p][j] & 0xFFFF0000u));
                o[j] = as_u32(n);
            }
            *reinterpret_cast<u32x4 *>(xn + c * 8) = o;
        }
    }
    __syncthreads();
}

int32_t launch_gemv4(tf_ctx *ctx, hipStream_t st, const uint8_t *w, const uint8_t *s, const uint8_t *b, const void *x,
                     void *y, uint32_t m, uint32_t n, tf_dtype sd, tf_dtype od, const void *norm_w = nullptr, float eps = 0.0f);
bool gemv4_can_fuse_norm(const uint8_t *w, const void *x, const void *norm_w, uint32_t n);
int32_t launch_rmsnorm_bf16w(tf_ctx *ctx, hipStream_t st, const void *x, const void *w, void *out, uint32_t d, float eps);
int32_t launch_gelu_mul(tf_ctx *ctx, hipStream_t st, const void *gate, const void *up, void *out, uint32_t count);
int32_t validate_gemv(tf_ctx *ctx, const char *who, const void *weights, uint64_t wo, const void *scales, uint64_t so,
                      const void *biases, uint64_t bo, const void *x, uint64_t xo, const void *y, uint64_t yo,
                      uint32_t m, uint32_t n, tf_dtype sd, tf_dtype od, unsigned weights_align);

}  // namespace tfk

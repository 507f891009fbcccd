// Row-wide element-wise / normalisation arithmetic of the stages either side of the MoE block: one 256-thread block holds a
// row (at most 4096 values) in registers between its reductions.  Shared by the glue kernels and by the kernels that repeat
// a glue stage in their own prologue instead of waiting for a launch of it.
#pragma once

#include "tf_rowdot.hpp"

namespace tfk {

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

// The post-attention setup on the elements one thread owns:
//   h   = half(hidden + half(attn * inv_rms(attn) * w_post_attn))      (the new residual stream, fp16 values)
//   inv = inv_rms(h)
// partial: 8 floats of LDS.  Every thread of the block must call it (two block barriers inside).
template <bool VEC>
struct PostAttnRow {
    float h[kPerThread];
    float inv;

    __device__ __forceinline__ void compute(const RowSlice<VEC> &rs, const half_t *attn_row, const half_t *hidden_row, const uint16_t *w_post_attn,
                                            float eps, float *partial) {
        float at[kPerThread], w[kPerThread];
        rs.load_f16(attn_row, at);
        rs.load_bf16(w_post_attn, w);
        rs.load_f16(hidden_row, h);
        finish(rs, at, w, eps, partial);
    }
    // the same with the three rows already in registers (h holds the hidden row)
    __device__ __forceinline__ void finish(const RowSlice<VEC> &rs, const float *at, const float *w, float eps, float *partial) {
        const float attn_inv = block_inv_rms(at, rs.d, eps, partial);
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) h[j] = round_half(h[j] + round_half(at[j] * attn_inv * w[j]));
        inv = block_inv_rms(h, rs.d, eps, partial + 4);
    }
};

// The layer tail on the elements one thread owns (x: the routed experts' sum h2 on entry; hid: the residual stream on entry, the
// layer's output on return):
//   NORM_H1: h1 <- half(h1 * inv_rms(h1) * w1) first (rmsnorm_bf16w of the shared expert's raw output)
//   h12 = half(h1 + half(h2 * inv_rms(h2) * w2));
//   hid <- half(half(hid + half(h12 * inv_rms(h12) * wp)) * half(layer_scalar)).
// partial: 12 floats of LDS.  Every thread of the block must call it (block barriers inside).
template <bool NORM_H1>
__device__ __forceinline__ void layer_tail_row(uint32_t d, float *x, const float *w2, float *h1, const float *wp, float *hid, const float *w1, float eps,
                                               float layer_scalar, float *partial) {
    float inv_h2;
    if constexpr (NORM_H1) {
        // the sums of squares of h1 and h2 do not depend on each other: one barrier for both
        float acc1 = 0.0f, acc2 = 0.0f;
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) acc1 = fmaf(h1[j], h1[j], acc1);
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) acc2 = fmaf(x[j], x[j], acc2);
        acc1 = wave_sum(acc1);
        acc2 = wave_sum(acc2);
        if ((threadIdx.x & 63) == 0) {
            partial[8 + (threadIdx.x >> 6)] = acc1;
            partial[threadIdx.x >> 6] = acc2;
        }
        __syncthreads();
        const float inv_h1 = 1.0f / sqrtf((partial[8] + partial[9] + partial[10] + partial[11]) / (float)d + eps);
        inv_h2 = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)d + eps);
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) h1[j] = round_half(h1[j] * inv_h1 * w1[j]);
    } else {
        inv_h2 = block_inv_rms(x, d, eps, partial);
    }
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) x[j] = round_half(h1[j] + round_half(x[j] * inv_h2 * w2[j]));
    const float inv_h12 = block_inv_rms(x, d, eps, partial + 4);
    const float scale = round_half(layer_scalar);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) hid[j] = round_half(round_half(hid[j] + round_half(x[j] * inv_h12 * wp[j])) * scale);
}

// 8 fp16 values (held as floats) -> one 16-byte piece
__device__ __forceinline__ u32x4 pack_half8(const float *v) {
    u32x4 r;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const half2_t h = {(half_t)v[2 * j], (half_t)v[2 * j + 1]};
        r[j] = as_u32(h);
    }
    return r;
}

}  // namespace tfk

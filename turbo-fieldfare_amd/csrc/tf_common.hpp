// Device-side building blocks shared by the gfx950 kernels: type aliases, affine scale decoding,
// nibble -> fp16 expansion, wave64 reductions.  Written for CDNA4 only (64-wide waves, GFX9 DPP).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tf_kernels.h"

namespace tfk {

typedef _Float16 half_t;
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;
constexpr int kGroup = 64;  // elements per (scale, bias) pair

__device__ __forceinline__ float bf16_to_f32(uint16_t b) { return __uint_as_float((uint32_t)b << 16); }
__device__ __forceinline__ float f16_to_f32(uint16_t b) { return (float)__builtin_bit_cast(half_t, b); }

// SD: 0 = BF16 (reference-exact), 1 = FP16
template <int SD>
__device__ __forceinline__ float sb_to_f32(uint16_t v) {
    if constexpr (SD == 0) return bf16_to_f32(v);
    else return f16_to_f32(v);
}

__device__ __forceinline__ half2_t as_half2(uint32_t v) { return __builtin_bit_cast(half2_t, v); }
__device__ __forceinline__ uint32_t as_u32(half2_t v) { return __builtin_bit_cast(uint32_t, v); }

// --- DPP helpers --------------------------------------------------------------------------------
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f32(float v) {
    // lanes whose row is masked off, or whose source lane is invalid, read 0
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, 0xF, false));
}

// After this every lane of a 16-lane DPP row holds that row's sum.
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]
    v += dpp_f32<0x141>(v);  // row_half_mirror
    v += dpp_f32<0x140>(v);  // row_mirror
    return v;
}

// Sum over the 64 lanes; the result is wave-uniform (returned through an SGPR).
__device__ __forceinline__ float wave_sum(float v) {
    v = row16_sum(v);
    v += dpp_f32<0x142, 0xA>(v);  // row_bcast15 into rows 1 and 3
    v += dpp_f32<0x143, 0xC>(v);  // row_bcast31 into rows 2 and 3
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Sums of lanes 0..31 and 32..63; lo/hi are wave-uniform.
__device__ __forceinline__ void half_wave_sums(float v, float &lo, float &hi) {
    v = row16_sum(v);
    v += dpp_f32<0x142, 0xA>(v);
    lo = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 31));
    hi = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

// Maximum over the 64 lanes (DPP, no LDS traffic); wave-uniform result.  NaNs must be filtered by the caller.
template <int CTRL, int ROW_MASK = 0xF>
__device__ __forceinline__ float dpp_f32_neg_inf(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp((int)0xFF800000u, __builtin_bit_cast(int, v), CTRL,
                                                                 ROW_MASK, 0xF, false));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_f32_neg_inf<0xB1>(v));
    v = fmaxf(v, dpp_f32_neg_inf<0x4E>(v));
    v = fmaxf(v, dpp_f32_neg_inf<0x141>(v));
    v = fmaxf(v, dpp_f32_neg_inf<0x140>(v));
    v = fmaxf(v, dpp_f32_neg_inf<0x142, 0xA>(v));
    v = fmaxf(v, dpp_f32_neg_inf<0x143, 0xC>(v));
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
__device__ __forceinline__ float read_lane(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// (value descending, index ascending) maximum across the wave; every lane ends with the winner.
// Candidates that must never win carry value -inf and index 0xFFFFFFFF.
__device__ __forceinline__ void wave_best_pair(float &v, uint32_t &idx) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float ov = __shfl_xor(v, off, kWave);
        const uint32_t oi = (uint32_t)__shfl_xor((int)idx, off, kWave);
        const bool take = (ov > v) || (ov == v && oi < idx);
        v = take ? ov : v;
        idx = take ? oi : idx;
    }
}

// --- int4 chunk arithmetic -------------------------------------------------------------------------
// A "chunk" is 16 consecutive bytes of a packed row: 32 nibbles = half a quantization group.
// Word d of the chunk holds elements 8d..8d+7, nibble i of the word = element 8d+i.
//
// Unpacking costs one AND per element pair and no conversion: masking a word with 0x000F000F leaves nibbles (i, i+4)
// in the low mantissa bits of two fp16 values, which read as fp16 subnormals are exactly q * 2^-24; the 0x00F000F0 mask
// leaves nibbles (i+1, i+5) as 16 q * 2^-24, and their activations are stored pre-multiplied by 1/16 (exact for
// |x| >= 2^-10, otherwise off by at most 2^-25).  fp16 denormals are not flushed by the matrix pipe.
//
// The multiply-accumulate runs on the matrix pipe, which is otherwise idle in these kernels: v_mfma_f32_4x4x4_16b_f16
// computes, for each group of four lanes, the 4x4 products of the lanes' A rows with the lanes' B columns over K = 4.
// With A = this lane's four weights and B = this lane's four activations, the diagonal element of the group's 4x4
// result, which lands in result register (lane & 3) of this lane, is the lane's own 4-element dot product; the
// off-diagonal elements are discarded.  Eight such instructions cover the chunk and accumulate in fp32; every product
// q*x (4 bits x 11 bits) is exact.  The instruction ignores the execution mask, so chunk_dot() must be called from
// wave-uniform control flow.
//
// xq[16] holds the chunk's 32 activations arranged to match: xq[4d+0] = (x[8d], x[8d+4]), xq[4d+1] = (x[8d+1], x[8d+5]) / 16,
// xq[4d+2] = (x[8d+2], x[8d+6]), xq[4d+3] = (x[8d+3], x[8d+7]) / 16.
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int lane_index() { return (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u)); }

__device__ __forceinline__ float chunk_dot(const u32x4 w, const half2_t *xq) {
    const int sel = lane_index() & 3;
    f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t v = w[d];
        const uint32_t v8 = v >> 8;
        const u32x2 a0 = {v & 0x000F000Fu, v & 0x00F000F0u};     // (e0, e4), 16 (e1, e5)
        const u32x2 a1 = {v8 & 0x000F000Fu, v8 & 0x00F000F0u};   // (e2, e6), 16 (e3, e7)
        const half4_t b0 = __builtin_shufflevector(xq[4 * d + 0], xq[4 * d + 1], 0, 1, 2, 3);
        const half4_t b1 = __builtin_shufflevector(xq[4 * d + 2], xq[4 * d + 3], 0, 1, 2, 3);
        c = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a0), b0, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, a1), b1, c, 0, 0, 0);
    }
    const float c01 = (sel & 1) ? c[1] : c[0];
    const float c23 = (sel & 1) ? c[3] : c[2];
    return ((sel & 2) ? c23 : c01) * 16777216.0f;   // subnormal units -> integers
}

// The same in two steps, for a chunk of weights that meets many activation vectors: chunk_operands() isolates the nibble pairs
// once (20 instructions), chunk_dot_pre() multiplies them with one vector's activations (8 matrix instructions and the pick
// of the diagonal element).  chunk_dot(w, xq) == chunk_dot_pre(chunk_operands(w), xq) bit for bit.
struct ChunkOperands {
    u32x2 a[8];
};
__device__ __forceinline__ ChunkOperands chunk_operands(const u32x4 w) {
    ChunkOperands o;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t v = w[d];
        const uint32_t v8 = v >> 8;
        o.a[2 * d] = u32x2{v & 0x000F000Fu, v & 0x00F000F0u};
        o.a[2 * d + 1] = u32x2{v8 & 0x000F000Fu, v8 & 0x00F000F0u};
    }
    return o;
}
__device__ __forceinline__ float chunk_dot_pre(const ChunkOperands &o, const half2_t *xq) {
    const int sel = lane_index() & 3;
    f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const half4_t b0 = __builtin_shufflevector(xq[4 * d + 0], xq[4 * d + 1], 0, 1, 2, 3);
        const half4_t b1 = __builtin_shufflevector(xq[4 * d + 2], xq[4 * d + 3], 0, 1, 2, 3);
        c = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, o.a[2 * d]), b0, c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4_t, o.a[2 * d + 1]), b1, c, 0, 0, 0);
    }
    const float c01 = (sel & 1) ? c[1] : c[0];
    const float c23 = (sel & 1) ? c[3] : c[2];
    return ((sel & 2) ? c23 : c01) * 16777216.0f;
}

// Arrange 32 consecutive activations (four 16-byte loads, xr[d] = elements 8d..8d+7 as 4 packed pairs)
// into the order chunk_dot() consumes, and return their fp32 sum.
__device__ __forceinline__ float arrange_x(const u32x4 *xr, half2_t *xq) {
    float sum = 0.0f;
    const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t p01 = xr[d][0], p23 = xr[d][1], p45 = xr[d][2], p67 = xr[d][3];
        xq[4 * d + 0] = as_half2((p01 & 0xFFFFu) | (p45 << 16));                     // (e0, e4)
        xq[4 * d + 1] = as_half2((p01 >> 16) | (p45 & 0xFFFF0000u)) * sixteenth;     // (e1, e5) / 16
        xq[4 * d + 2] = as_half2((p23 & 0xFFFFu) | (p67 << 16));                     // (e2, e6)
        xq[4 * d + 3] = as_half2((p23 >> 16) | (p67 & 0xFFFF0000u)) * sixteenth;     // (e3, e7) / 16
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t h = as_half2(xr[d][j]);
            sum += (float)h[0];
            sum += (float)h[1];
        }
    }
    return sum;
}

// Block barrier that orders LDS traffic only: unlike __syncthreads() it does not wait for global loads that are still in
// flight, so requests issued ahead of their use stay ahead across the barrier.
__device__ __forceinline__ void lds_barrier() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_s_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
}

__device__ __forceinline__ u32x4 load16(const void *p) { return *reinterpret_cast<const u32x4 *>(p); }

// GELU, tanh approximation, as the reference kernels compute it (Metal/MoE/moe.metal:53-60):
// 0.5 x (1 + tanh(clamp(sqrt(2/pi) (x + 0.044715 x^3), -20, 20))).
__device__ __forceinline__ float gelu_tanh(float x) {
    const float x3 = x * x * x;
    float inner = 0.7978845608028654f * (x + 0.044715f * x3);
    inner = fminf(fmaxf(inner, -20.0f), 20.0f);
    return 0.5f * x * (1.0f + tanhf(inner));
}

// The same function through the identity 0.5 (1 + tanh u) = 1 / (1 + exp(-2u)): one hardware exponential and one
// hardware reciprocal (about a dozen instructions against about forty), a few fp32 ulps from gelu_tanh() and without
// its cancellation for very negative u.  For epilogues that apply it to whole accumulator tiles.
__device__ __forceinline__ float gelu_tanh_fast(float x) {
    const float x3 = x * x * x;
    float inner = 0.7978845608028654f * (x + 0.044715f * x3);
    inner = fminf(fmaxf(inner, -20.0f), 20.0f);
    const float e = __builtin_amdgcn_exp2f(inner * -2.885390081777927f);   // exp(-2 u) = 2^(-2 u log2 e)
    return x * __builtin_amdgcn_rcpf(1.0f + e);
}

__device__ __forceinline__ uint16_t f32_to_f16_bits(float v) { return __builtin_bit_cast(uint16_t, (half_t)v); }

}  // namespace tfk

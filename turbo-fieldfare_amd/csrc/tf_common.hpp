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
// Masking a word with 0x000F000F leaves nibbles (i, i+4) in the low mantissa bits of two fp16 values: read as
// fp16 subnormals they are exactly q * 2^-24, which v_dot2_f32_f16 multiplies without flushing (fp16 denormals are
// enabled in the kernels' float mode).  The 0x00F000F0 mask leaves nibbles (i+1, i+5) as 16 q * 2^-24; those products
// go to a second accumulator.  Both accumulators are rescaled once per chunk.  Every product q*x (4 bits x 11 bits)
// is exact in fp32, so unpacking costs one AND per pair and no conversion instruction.
//
// xq[16] holds the chunk's 32 activations arranged to match: xq[4d+j] = (x[8d+j], x[8d+j+4]).
__device__ __forceinline__ float chunk_dot(const u32x4 w, const half2_t *xq) {
    float lo = 0.0f, hi = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t v = w[d];
        const uint32_t v8 = v >> 8;
        lo = __builtin_amdgcn_fdot2(as_half2(v & 0x000F000Fu), xq[4 * d + 0], lo, false);   // (e0, e4)
        hi = __builtin_amdgcn_fdot2(as_half2(v & 0x00F000F0u), xq[4 * d + 1], hi, false);   // 16 (e1, e5)
        lo = __builtin_amdgcn_fdot2(as_half2(v8 & 0x000F000Fu), xq[4 * d + 2], lo, false);  // (e2, e6)
        hi = __builtin_amdgcn_fdot2(as_half2(v8 & 0x00F000F0u), xq[4 * d + 3], hi, false);  // 16 (e3, e7)
    }
    return fmaf(hi, 1048576.0f, lo * 16777216.0f);   // hi * 2^20 + lo * 2^24
}

// Arrange 32 consecutive activations (four 16-byte loads, xr[d] = elements 8d..8d+7 as 4 packed pairs)
// into the order chunk_dot() consumes, and return their fp32 sum.
__device__ __forceinline__ float arrange_x(const u32x4 *xr, half2_t *xq) {
    float sum = 0.0f;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const uint32_t p01 = xr[d][0], p23 = xr[d][1], p45 = xr[d][2], p67 = xr[d][3];
        // (e0,e4) (e1,e5) (e2,e6) (e3,e7)
        xq[4 * d + 0] = as_half2((p01 & 0xFFFFu) | (p45 << 16));
        xq[4 * d + 1] = as_half2((p01 >> 16) | (p45 & 0xFFFF0000u));
        xq[4 * d + 2] = as_half2((p23 & 0xFFFFu) | (p67 << 16));
        xq[4 * d + 3] = as_half2((p23 >> 16) | (p67 & 0xFFFF0000u));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t h = as_half2(xr[d][j]);
            sum += (float)h[0];
            sum += (float)h[1];
        }
    }
    return sum;
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

__device__ __forceinline__ uint16_t f32_to_f16_bits(float v) { return __builtin_bit_cast(uint16_t, (half_t)v); }

}  // namespace tfk

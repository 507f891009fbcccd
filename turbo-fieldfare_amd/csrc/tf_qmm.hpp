// int4 x fp16 matrix multiply on the CDNA4 matrix cores: Y[M,N] = X[M,K] . W[N,K]^T with W in the affine group-64
// int4 layout.  One 256-thread block owns a BM x BN output tile and walks K one quantization group (64) at a time:
//
//   global -> registers   X rows (16-byte loads) and the packed W rows of the group (+ their scale/bias), requested for
//                         step t+1 while step t is being multiplied;
//   registers -> LDS      W is expanded to fp16  half(q * s + b)  exactly once per block and K step (the rounding point
//                         of the reference's staged-affine path, tensorops.metal:57-94); X is copied;
//   LDS -> MFMA           v_mfma_f32_32x32x16_f16, fp32 accumulators, each wave a 64 x 32 slice of the tile.
//
// Elements inside every 8-wide k fragment are stored in the order (0,4,1,5,2,6,3,7) for both operands — the order the
// nibble masks produce — which leaves every dot product unchanged.
//
// Row indirection makes the same kernel serve the grouped expert GEMMs: A rows can be gathered through a row table
// (tokens routed to one expert) and C rows scattered through another.
#pragma once

#include "tf_common.hpp"

namespace tfk {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kQmmBM = 64;    // rows per block tile
constexpr int kQmmBN = 128;   // columns per block tile (4 waves x 32)
constexpr int kQmmLDK = 72;   // LDS row pitch in halves: 64 + 8 padding (keeps 16-byte alignment, spreads banks)

struct QmmSmem {
    half_t a[2][kQmmBM * kQmmLDK];
    half_t b[2][kQmmBN * kQmmLDK];
};
struct QmmSmemDual {
    half_t a[2][kQmmBM * kQmmLDK];
    half_t b[2][2][kQmmBN * kQmmLDK];   // [buffer][gate/up]
};

// (0,1)(2,3)(4,5)(6,7) -> (0,4)(1,5)(2,6)(3,7)
__device__ __forceinline__ u32x4 permute_k8(const u32x4 v) {
    u32x4 o;
    o[0] = (v[0] & 0xFFFFu) | (v[2] << 16);
    o[1] = (v[0] >> 16) | (v[2] & 0xFFFF0000u);
    o[2] = (v[1] & 0xFFFFu) | (v[3] << 16);
    o[3] = (v[1] >> 16) | (v[3] & 0xFFFF0000u);
    return o;
}

// 8 nibbles of one word -> 8 fp16 weights half(q * s + b) in the order (0,4)(1,5)(2,6)(3,7).
// q is formed exactly as fp16 (1024 + q, minus 1024); q * s + b is one fp16 fused multiply-add on fp16 copies of the
// scale and bias.
__device__ __forceinline__ u32x4 dequant_word(uint32_t v, half2_t s2, half2_t b2) {
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    const uint32_t v4 = v >> 4, v8 = v >> 8, v12 = v >> 12;
    u32x4 o;
    const half2_t q0 = as_half2((v & 0x000F000Fu) | 0x64006400u) - k1024;
    const half2_t q1 = as_half2((v4 & 0x000F000Fu) | 0x64006400u) - k1024;
    const half2_t q2 = as_half2((v8 & 0x000F000Fu) | 0x64006400u) - k1024;
    const half2_t q3 = as_half2((v12 & 0x000F000Fu) | 0x64006400u) - k1024;
    o[0] = as_u32(__builtin_elementwise_fma(q0, s2, b2));
    o[1] = as_u32(__builtin_elementwise_fma(q1, s2, b2));
    o[2] = as_u32(__builtin_elementwise_fma(q2, s2, b2));
    o[3] = as_u32(__builtin_elementwise_fma(q3, s2, b2));
    return o;
}

template <int SD>
__device__ __forceinline__ half2_t sb_to_half2(uint16_t v) {
    const half_t h = (half_t)sb_to_f32<SD>(v);
    return half2_t{h, h};
}

// Per-thread staging registers for one K step of one W matrix: 16 packed bytes (32 nibbles = half a group) of row
// (tid / 2), plus that row's scale/bias for the group.
struct WStage {
    u32x4 w;
    uint16_t s, b;
};

// w_rows: first row of the tile; rows_left: valid rows from there; row_bytes = K/2; groups = K/64
__device__ __forceinline__ void w_stage_load(WStage &st, const uint8_t *w_rows, const uint8_t *s_rows, const uint8_t *b_rows,
                                             int rows_left, int row_bytes, int groups, int kt) {
    const int r = threadIdx.x >> 1, hc = threadIdx.x & 1;
    st.w = u32x4{0u, 0u, 0u, 0u};
    st.s = 0;
    st.b = 0;
    if (r < rows_left) {
        st.w = load16(w_rows + (size_t)r * row_bytes + kt * 32 + hc * 16);
        st.s = *reinterpret_cast<const uint16_t *>(s_rows + ((size_t)r * groups + kt) * 2);
        st.b = *reinterpret_cast<const uint16_t *>(b_rows + ((size_t)r * groups + kt) * 2);
    }
}

template <int SD>
__device__ __forceinline__ void w_stage_store(const WStage &st, half_t *bs) {
    const int r = threadIdx.x >> 1, hc = threadIdx.x & 1;
    const half2_t s2 = sb_to_half2<SD>(st.s), b2 = sb_to_half2<SD>(st.b);
#pragma unroll
    for (int d = 0; d < 4; ++d)
        *reinterpret_cast<u32x4 *>(bs + r * kQmmLDK + hc * 32 + d * 8) = dequant_word(st.w[d], s2, b2);
}

// A tile: 64 rows x 64 halves = 512 16-byte chunks, two per thread.
struct AStage {
    u32x4 v[2];
};

// row_ptr[i]: start of the row this thread's chunk i belongs to (nullptr: row beyond the tile -> zeros)
__device__ __forceinline__ void a_stage_load(AStage &st, const half_t *const row_ptr[2], int kt) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int kc = (threadIdx.x + 256 * i) & 7;
        st.v[i] = u32x4{0u, 0u, 0u, 0u};
        if (row_ptr[i]) st.v[i] = load16(row_ptr[i] + kt * 64 + kc * 8);
    }
}

__device__ __forceinline__ void a_stage_store(const AStage &st, half_t *as) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int c = threadIdx.x + 256 * i;
        *reinterpret_cast<u32x4 *>(as + (c >> 3) * kQmmLDK + (c & 7) * 8) = permute_k8(st.v[i]);
    }
}

// One K group (64) of MFMAs for this wave's 64 x 32 slice: acc[mb] += A[mb*32.., :] . B[wave*32.., :]^T
__device__ __forceinline__ void mfma_group(const half_t *as, const half_t *bs, int wave, int lane, float16_t acc[2]) {
    const int i = lane & 31, kb = lane >> 5;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        const half8_t bf = *reinterpret_cast<const half8_t *>(bs + (wave * 32 + i) * kQmmLDK + ks * 16 + kb * 8);
#pragma unroll
        for (int mb = 0; mb < 2; ++mb) {
            const half8_t af = *reinterpret_cast<const half8_t *>(as + (mb * 32 + i) * kQmmLDK + ks * 16 + kb * 8);
            acc[mb] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf, acc[mb], 0, 0, 0);
        }
    }
}

// Accumulator element r of lane `lane` in a 32 x 32 block sits at (row, col):
__device__ __forceinline__ int acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }
__device__ __forceinline__ int acc_col(int lane) { return lane & 31; }

}  // namespace tfk

// int4 x fp16 matrix multiply on the CDNA4 matrix cores: Y[M,N] = X[M,K] . W[N,K]^T with W in the affine group-64
// int4 layout.  A 256-thread block owns a 128 x 256 output tile (four waves, each 128 rows x 64 columns) and walks K one
// quantization group (64) at a time:
//
//   W   never touches LDS.  In v_mfma_f32_32x32x16_f16 lane (i, kb) supplies, for output column i, the 8 weights of
//       k-slots 8 kb .. 8 kb + 7.  The lane loads 16 packed bytes of "its" row (32 nibbles: the kb-th half of the group)
//       and expands one 32-bit word (8 nibbles) per MFMA straight into the operand registers as half(q * s + b), the
//       rounding point of the reference's staged-affine path (tensorops.metal:57-94).  MFMA number d of the group then
//       covers k = {8d .. 8d+7} u {32+8d .. 32+8d+7}.
//   X   goes through LDS once per block and K step, shared by the four waves: 16-byte chunks, the 8 elements of a chunk
//       stored in the order (0,4,1,5,2,6,3,7) that the nibble masks produce for W, chunk positions XOR-swizzled so that
//       both the row-major stores and the fragment reads are free of bank conflicts.
//   global loads are requested kQmmDepth K steps ahead of their use (a ring of staging registers): one K step of MFMAs
//       is far shorter than a trip to L2 or HBM.
//
// Row indirection makes the same loop serve the grouped expert GEMMs: X rows can be gathered through a row table
// (tokens routed to one expert) and Y rows scattered through another; row tiles beyond the rows present are skipped.
#pragma once

#include "tf_common.hpp"

namespace tfk {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kQmmBM = 128;      // rows per block tile (4 MFMA row tiles)
constexpr int kQmmWaveN = 64;    // columns per wave (2 MFMA column tiles)
constexpr int kQmmBN = 256;      // columns per block tile (4 waves)
constexpr int kQmmDepth = 2;     // K steps between a global request and its use
constexpr int kQmmAChunks = kQmmBM * 8 / 256;   // 16-byte X chunks staged per thread and K step

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
// q is formed exactly in fp16: the low nibble of each half as 1024 + q (0x6400 | q), the next one in place as 64 + q
// (0x5400 | q << 4), each minus its offset; q * s + b is then one fp16 fused multiply-add on fp16 copies of s and b.
__device__ __forceinline__ half8_t dequant_word(uint32_t v, half2_t s2, half2_t b2) {
    const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
    const half2_t k64 = {(half_t)64.0f, (half_t)64.0f};
    const uint32_t v8 = v >> 8;
    const half2_t q0 = as_half2((v & 0x000F000Fu) | 0x64006400u) - k1024;    // (e0, e4)
    const half2_t q1 = as_half2((v & 0x00F000F0u) | 0x54005400u) - k64;      // (e1, e5)
    const half2_t q2 = as_half2((v8 & 0x000F000Fu) | 0x64006400u) - k1024;   // (e2, e6)
    const half2_t q3 = as_half2((v8 & 0x00F000F0u) | 0x54005400u) - k64;     // (e3, e7)
    const half2_t w0 = __builtin_elementwise_fma(q0, s2, b2), w1 = __builtin_elementwise_fma(q1, s2, b2);
    const half2_t w2 = __builtin_elementwise_fma(q2, s2, b2), w3 = __builtin_elementwise_fma(q3, s2, b2);
    return half8_t{w0[0], w0[1], w1[0], w1[1], w2[0], w2[1], w3[0], w3[1]};
}

template <int SD>
__device__ __forceinline__ half2_t sb_to_half2(uint16_t v) {
    const half_t h = (half_t)sb_to_f32<SD>(v);
    return half2_t{h, h};
}

// 16-byte slot of X chunk (row r, chunk c of 8) inside one LDS stage of kQmmBM x 64 halves
__device__ __forceinline__ int a_slot(int r, int c) { return r * 8 + (c ^ ((r >> 1) & 7)); }

// Staging registers of one K step: this thread's X chunks, and for each of the wave's two column tiles the lane's 16
// packed bytes and the row's scale / bias for the group.
struct QmmStage {
    u32x4 a[kQmmAChunks];
    u32x4 w[2];
    uint16_t s[2], b[2];
};

// What a lane needs to know about its two weight rows (one per column tile).  Columns beyond the matrix and rows
// beyond the tile are served by a clamped, valid row: every load is unconditional, and what such lanes compute is
// never stored.
struct QmmBRows {
    const uint8_t *w[2];   // row start + kb * 16
    const uint8_t *s[2];   // scales of the row
    const uint8_t *b[2];
};

__device__ __forceinline__ void qmm_stage_load(QmmStage &st, const half_t *const a_row[kQmmAChunks], const QmmBRows &rows, int kt) {
#pragma unroll
    for (int q = 0; q < kQmmAChunks; ++q) {
        const int kc = (threadIdx.x + 256 * q) & 7;
        st.a[q] = load16(a_row[q] + kt * 64 + kc * 8);
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        st.w[j] = load16(rows.w[j] + kt * 32);
        st.s[j] = *reinterpret_cast<const uint16_t *>(rows.s[j] + kt * 2);
        st.b[j] = *reinterpret_cast<const uint16_t *>(rows.b[j] + kt * 2);
    }
}

__device__ __forceinline__ void qmm_stage_store_a(const QmmStage &st, u32x4 *as) {
#pragma unroll
    for (int q = 0; q < kQmmAChunks; ++q) {
        const int c = threadIdx.x + 256 * q;
        as[a_slot(c >> 3, c & 7)] = permute_k8(st.a[q]);
    }
}

// One K group for this wave: acc[mt][j] += X[mt*32.., group] . W_j[.., group]^T for the row tiles mt < RT.
template <int SD, int RT>
__device__ __forceinline__ void qmm_group(const QmmStage &st, const u32x4 *as, int lane, float16_t acc[4][2]) {
    const int i = lane & 31, kb = lane >> 5;
    half2_t s2[2], b2[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        s2[j] = sb_to_half2<SD>(st.s[j]);
        b2[j] = sb_to_half2<SD>(st.b[j]);
    }
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const half8_t bf0 = dequant_word(st.w[0][d], s2[0], b2[0]);
        const half8_t bf1 = dequant_word(st.w[1][d], s2[1], b2[1]);
#pragma unroll
        for (int mt = 0; mt < RT; ++mt) {
            const half8_t af = __builtin_bit_cast(half8_t, as[a_slot(mt * 32 + i, kb * 4 + d)]);
            acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf0, acc[mt][0], 0, 0, 0);
            acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, bf1, acc[mt][1], 0, 0, 0);
        }
    }
}

// The K loop.  Step kt lives in staging slot kt % kQmmDepth; its X tile is in LDS stage kt & 1 when it is multiplied.
// While step kt is multiplied, the X tile of step kt + 1 goes to the other LDS stage and the slot of step kt is
// refilled with step kt + kQmmDepth.  Requests and stores are unconditional (past the end they repeat the last step,
// which nobody reads): a load under a branch would make every later wait for memory a wait for all of it.
template <int SD, int RT>
__device__ __forceinline__ void qmm_k_loop_rt(int kt_count, const half_t *const a_row[kQmmAChunks], const QmmBRows &rows,
                                              u32x4 *lds /* 2 stages of kQmmBM * 8 */, int lane, float16_t acc[4][2]) {
    QmmStage st[kQmmDepth];
    const int last = kt_count - 1;
#pragma unroll
    for (int u = 0; u < kQmmDepth; ++u) qmm_stage_load(st[u], a_row, rows, min(u, last));
    qmm_stage_store_a(st[0], lds);
    __syncthreads();
    int kt0 = 0;
    for (; kt0 + kQmmDepth <= kt_count; kt0 += kQmmDepth) {
#pragma unroll
        for (int u = 0; u < kQmmDepth; ++u) {
            const int kt = kt0 + u;
            qmm_group<SD, RT>(st[u], lds + (kt & 1) * (kQmmBM * 8), lane, acc);
            qmm_stage_store_a(st[(u + 1) % kQmmDepth], lds + ((kt + 1) & 1) * (kQmmBM * 8));
            qmm_stage_load(st[u], a_row, rows, min(kt + kQmmDepth, last));
            __syncthreads();
        }
    }
#pragma unroll
    for (int u = 0; u < kQmmDepth - 1; ++u) {   // the kt_count % kQmmDepth steps left
        const int kt = kt0 + u;
        if (kt < kt_count) {
            qmm_group<SD, RT>(st[u], lds + (kt & 1) * (kQmmBM * 8), lane, acc);
            qmm_stage_store_a(st[(u + 1) % kQmmDepth], lds + ((kt + 1) & 1) * (kQmmBM * 8));
            __syncthreads();
        }
    }
}

// row_tiles (1..4, block-uniform): 32-row tiles that hold rows; the others are not multiplied.
template <int SD>
__device__ __forceinline__ void qmm_k_loop(int kt_count, const half_t *const a_row[kQmmAChunks], const QmmBRows &rows, u32x4 *lds,
                                           int lane, int row_tiles, float16_t acc[4][2]) {
    switch (row_tiles) {
        case 1: qmm_k_loop_rt<SD, 1>(kt_count, a_row, rows, lds, lane, acc); break;
        case 2: qmm_k_loop_rt<SD, 2>(kt_count, a_row, rows, lds, lane, acc); break;
        case 3: qmm_k_loop_rt<SD, 3>(kt_count, a_row, rows, lds, lane, acc); break;
        default: qmm_k_loop_rt<SD, 4>(kt_count, a_row, rows, lds, lane, acc); break;
    }
}

// Accumulator element r of lane `lane` in a 32 x 32 block sits at (row, col):
__device__ __forceinline__ int acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }
__device__ __forceinline__ int acc_col(int lane) { return lane & 31; }

}  // namespace tfk

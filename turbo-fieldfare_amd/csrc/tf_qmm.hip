// Matrix-core (MFMA) kernels: dense int4 QMM, and the grouped expert GEMMs of batched prefill
// (gate/up + GeGLU, then down) driven by a work list of (expert, pair range) chunks.
#include "tf_prefill_kernels.hpp"

using namespace tfk;

namespace {

// ------------------------------------------------------------------------------------------------ dense
template <int SD>
__global__ __launch_bounds__(256) void qmm_dense_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B, const half_t *X,
                                                        long ldx, half_t *Y, long ldy, int M, int N, int K) {
    __shared__ __align__(16) QmmSmem sm;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * kQmmBN, m0 = blockIdx.y * kQmmBM;
    const int groups = K >> 6, row_bytes = K >> 1, kt_count = K >> 6;
    const half_t *arow[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int r = (threadIdx.x + 256 * i) >> 3;
        arow[i] = (m0 + r < M) ? X + (size_t)(m0 + r) * ldx : nullptr;
    }
    const int n_left = min(kQmmBN, N - n0);
    const uint8_t *w_rows = W + (size_t)n0 * row_bytes;
    const uint8_t *s_rows = S + (size_t)n0 * groups * 2;
    const uint8_t *b_rows = B + (size_t)n0 * groups * 2;

    AStage ast;
    WStage wst;
    a_stage_load(ast, arow, 0);
    w_stage_load(wst, w_rows, s_rows, b_rows, n_left, row_bytes, groups, 0);
    a_stage_store(ast, sm.a[0]);
    w_stage_store<SD>(wst, sm.b[0]);
    __syncthreads();
    float16_t acc[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][r] = 0.0f;
    for (int kt = 0; kt < kt_count; ++kt) {
        const bool more = kt + 1 < kt_count;
        if (more) {
            a_stage_load(ast, arow, kt + 1);
            w_stage_load(wst, w_rows, s_rows, b_rows, n_left, row_bytes, groups, kt + 1);
        }
        mfma_group(sm.a[kt & 1], sm.b[kt & 1], wave, lane, acc);
        if (more) {
            a_stage_store(ast, sm.a[(kt + 1) & 1]);
            w_stage_store<SD>(wst, sm.b[(kt + 1) & 1]);
        }
        __syncthreads();
    }
    const int n = n0 + wave * 32 + acc_col(lane);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + mb * 32 + acc_row(r, lane);
            if (m < M && n < N) Y[(size_t)m * ldy + n] = (half_t)acc[mb][r];
        }
}

// ------------------------------------------------------------------------------------------------ grouped phase 1
// Block = one chunk (<= 64 sorted pairs of one expert) x 64 intermediate columns.  Wave w owns rows (w/2)*32.. and columns
// (w%2)*32.. for BOTH the gate and the up matrix, so GeGLU is applied to the fp32 accumulators in registers.
constexpr int kP1BN = 64;

template <int SD>
__global__ __launch_bounds__(256) void grouped_phase1_mfma_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl,
                                                                  const tf_prefill_pair *pairs, const half_t *hidden,
                                                                  long hidden_stride, half_t *acts, uint32_t acts_pair_base,
                                                                  int D, int F) {
    __shared__ __align__(16) half_t sa[2][kQmmBM * kQmmLDK];
    __shared__ __align__(16) half_t sb[2][2][kP1BN * kQmmLDK];
    tf_prefill_group ch;
    if (!get_chunk(cl, blockIdx.y, ch)) return;
    const uint8_t *base = expert_base(tab, ch.expert);
    if (!base) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * kP1BN;
    const int groups = D >> 6, row_bytes = D >> 1, kt_count = D >> 6;
    const half_t *arow[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t r = (threadIdx.x + 256 * i) >> 3;
        arow[i] = r < ch.pair_count ? hidden + (size_t)pairs[ch.pair_start + r].token * hidden_stride : nullptr;
    }
    // 64 rows x 32 bytes per matrix and K step = 128 16-byte chunks: threads 0..127 stage gate, 128..255 stage up
    const int which = threadIdx.x >> 7, tt = threadIdx.x & 127;
    const int wr = tt >> 1, hc = tt & 1;
    const int n_left = min(kP1BN, F - n0);
    const uint32_t w_off = which ? off.up_W_off : off.gate_W_off;
    const uint32_t s_off = which ? off.up_s_off : off.gate_s_off;
    const uint32_t b_off = which ? off.up_b_off : off.gate_b_off;
    const uint8_t *w_row = base + w_off + (size_t)(n0 + wr) * row_bytes + hc * 16;
    const uint8_t *s_row = base + s_off + (size_t)(n0 + wr) * groups * 2;
    const uint8_t *b_row = base + b_off + (size_t)(n0 + wr) * groups * 2;
    const bool w_valid = wr < n_left;

    AStage ast;
    WStage wst;
    auto load_w = [&](int kt) {
        wst.w = u32x4{0u, 0u, 0u, 0u};
        wst.s = 0;
        wst.b = 0;
        if (w_valid) {
            wst.w = load16(w_row + kt * 32);
            wst.s = *reinterpret_cast<const uint16_t *>(s_row + kt * 2);
            wst.b = *reinterpret_cast<const uint16_t *>(b_row + kt * 2);
        }
    };
    auto store_w = [&](int buf) {
        const half2_t s2 = sb_to_half2<SD>(wst.s), b2 = sb_to_half2<SD>(wst.b);
        half_t *dst = sb[buf][which] + wr * kQmmLDK + hc * 32;
#pragma unroll
        for (int d = 0; d < 4; ++d) *reinterpret_cast<u32x4 *>(dst + d * 8) = dequant_word(wst.w[d], s2, b2);
    };
    a_stage_load(ast, arow, 0);
    load_w(0);
    a_stage_store(ast, sa[0]);
    store_w(0);
    __syncthreads();
    float16_t ag, au;
#pragma unroll
    for (int r = 0; r < 16; ++r) { ag[r] = 0.0f; au[r] = 0.0f; }
    const int mb = wave >> 1, nb = wave & 1;
    const int i = lane & 31, kb = lane >> 5;
    for (int kt = 0; kt < kt_count; ++kt) {
        const bool more = kt + 1 < kt_count;
        if (more) {
            a_stage_load(ast, arow, kt + 1);
            load_w(kt + 1);
        }
        const half_t *as = sa[kt & 1] + (mb * 32 + i) * kQmmLDK + kb * 8;
        const half_t *gs = sb[kt & 1][0] + (nb * 32 + i) * kQmmLDK + kb * 8;
        const half_t *us = sb[kt & 1][1] + (nb * 32 + i) * kQmmLDK + kb * 8;
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const half8_t af = *reinterpret_cast<const half8_t *>(as + ks * 16);
            const half8_t gf = *reinterpret_cast<const half8_t *>(gs + ks * 16);
            const half8_t uf = *reinterpret_cast<const half8_t *>(us + ks * 16);
            ag = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, gf, ag, 0, 0, 0);
            au = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, uf, au, 0, 0, 0);
        }
        if (more) {
            a_stage_store(ast, sa[(kt + 1) & 1]);
            store_w((kt + 1) & 1);
        }
        __syncthreads();
    }
    const int n = n0 + nb * 32 + acc_col(lane);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const uint32_t m = mb * 32 + acc_row(r, lane);
        if (m < ch.pair_count && n < F)
            acts[(size_t)(ch.pair_start + m - acts_pair_base) * F + n] = (half_t)(gelu_tanh(ag[r]) * au[r]);
    }
}

// ------------------------------------------------------------------------------------------------ grouped down
// Block = one chunk x 128 output columns: A rows are the chunk's activation rows, C rows scatter to
// route_partials[(token * top_k + rank) * D + c].
template <int SD>
__global__ __launch_bounds__(256) void grouped_down_mfma_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl,
                                                                const tf_prefill_pair *pairs, const half_t *acts,
                                                                uint32_t acts_pair_base, half_t *route_partials, int D, int F,
                                                                int top_k) {
    __shared__ __align__(16) QmmSmem sm;
    tf_prefill_group ch;
    if (!get_chunk(cl, blockIdx.y, ch)) return;
    const uint8_t *base = expert_base(tab, ch.expert);
    if (!base) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = blockIdx.x * kQmmBN;
    const int groups = F >> 6, row_bytes = F >> 1, kt_count = F >> 6;
    const half_t *arow[2];
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const uint32_t r = (threadIdx.x + 256 * i) >> 3;
        arow[i] = r < ch.pair_count ? acts + (size_t)(ch.pair_start + r - acts_pair_base) * F : nullptr;
    }
    const int n_left = min(kQmmBN, D - n0);
    const uint8_t *w_rows = base + off.down_W_off + (size_t)n0 * row_bytes;
    const uint8_t *s_rows = base + off.down_s_off + (size_t)n0 * groups * 2;
    const uint8_t *b_rows = base + off.down_b_off + (size_t)n0 * groups * 2;

    AStage ast;
    WStage wst;
    a_stage_load(ast, arow, 0);
    w_stage_load(wst, w_rows, s_rows, b_rows, n_left, row_bytes, groups, 0);
    a_stage_store(ast, sm.a[0]);
    w_stage_store<SD>(wst, sm.b[0]);
    __syncthreads();
    float16_t acc[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[mb][r] = 0.0f;
    for (int kt = 0; kt < kt_count; ++kt) {
        const bool more = kt + 1 < kt_count;
        if (more) {
            a_stage_load(ast, arow, kt + 1);
            w_stage_load(wst, w_rows, s_rows, b_rows, n_left, row_bytes, groups, kt + 1);
        }
        mfma_group(sm.a[kt & 1], sm.b[kt & 1], wave, lane, acc);
        if (more) {
            a_stage_store(ast, sm.a[(kt + 1) & 1]);
            w_stage_store<SD>(wst, sm.b[(kt + 1) & 1]);
        }
        __syncthreads();
    }
    const int n = n0 + wave * 32 + acc_col(lane);
#pragma unroll
    for (int mb = 0; mb < 2; ++mb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t m = mb * 32 + acc_row(r, lane);
            if (m < ch.pair_count && n < D) {
                const tf_prefill_pair p = pairs[ch.pair_start + m];
                route_partials[((size_t)p.token * top_k + p.rank) * D + n] = (half_t)acc[mb][r];
            }
        }
}

}  // namespace

namespace tfk {

bool qmm_operands_ok(const void *w, const void *x, long ldx_halves, int k) {
    return aligned16(w) && aligned16(x) && (ldx_halves % 8 == 0) && k > 0 && (k % 64 == 0);
}

int32_t launch_grouped_phase1_mfma(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off,
                                   const ChunkList &cl, uint32_t n_chunks_upper, const tf_prefill_pair *pairs,
                                   const half_t *hidden, long hidden_stride, half_t *acts, uint32_t acts_pair_base, int d, int f,
                                   tf_dtype sd) {
    const dim3 grid((f + kP1BN - 1) / kP1BN, n_chunks_upper);
    if (sd == TF_BF16)
        hipLaunchKernelGGL(grouped_phase1_mfma_kernel<0>, grid, dim3(256), 0, st, tab, off, cl, pairs, hidden, hidden_stride, acts, acts_pair_base, d, f);
    else
        hipLaunchKernelGGL(grouped_phase1_mfma_kernel<1>, grid, dim3(256), 0, st, tab, off, cl, pairs, hidden, hidden_stride, acts, acts_pair_base, d, f);
    return check_launch(ctx, "grouped_phase1_mfma");
}

int32_t launch_grouped_down_mfma(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off,
                                 const ChunkList &cl, uint32_t n_chunks_upper, const tf_prefill_pair *pairs, const half_t *acts,
                                 uint32_t acts_pair_base, half_t *route_partials, int d, int f, int top_k, tf_dtype sd) {
    const dim3 grid((d + kQmmBN - 1) / kQmmBN, n_chunks_upper);
    if (sd == TF_BF16)
        hipLaunchKernelGGL(grouped_down_mfma_kernel<0>, grid, dim3(256), 0, st, tab, off, cl, pairs, acts, acts_pair_base, route_partials, d, f, top_k);
    else
        hipLaunchKernelGGL(grouped_down_mfma_kernel<1>, grid, dim3(256), 0, st, tab, off, cl, pairs, acts, acts_pair_base, route_partials, d, f, top_k);
    return check_launch(ctx, "grouped_down_mfma");
}

}  // namespace tfk

extern "C" {

int32_t tf_int4_qmm(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                    uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *x, uint64_t x_offset,
                    void *y, uint64_t y_offset, int32_t m, int32_t n, int32_t k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx && weights && scales && biases && x && y, TF_ERR_INVALID_ARGUMENT, "int4_qmm: null argument");
    // MPPPrefillInt4QMM.encode's guard list (MPPPrefillInt4QMM.swift:40-56): anything it refuses is "unavailable", not an error
    const bool shape_ok = m > 0 && n > 0 && k > 0 && (k % (int32_t)TF_GROUP_SIZE == 0);
    const bool offs_ok = scales_offset % 2 == 0 && biases_offset % 2 == 0 && x_offset % 2 == 0 && y_offset % 2 == 0;
    if (!shape_ok || !offs_ok || !(scale_dtype == TF_BF16 || scale_dtype == TF_FP16)) return fail(ctx, TF_ERR_UNAVAILABLE, "int4_qmm: unsupported shape or offsets");
    const uint8_t *w = at(weights, weights_offset);
    const half_t *xp = reinterpret_cast<const half_t *>(at(x, x_offset));
    if (!qmm_operands_ok(w, xp, k, k) || !aligned(at(y, y_offset), 2)) return fail(ctx, TF_ERR_UNAVAILABLE, "int4_qmm: operands are not 16-byte aligned");
    const dim3 grid((n + kQmmBN - 1) / kQmmBN, (m + kQmmBM - 1) / kQmmBM);
    hipStream_t st = static_cast<hipStream_t>(stream);
    half_t *yp = reinterpret_cast<half_t *>(at(y, y_offset));
    if (scale_dtype == TF_BF16)
        hipLaunchKernelGGL(qmm_dense_kernel<0>, grid, dim3(256), 0, st, w, at(scales, scales_offset), at(biases, biases_offset), xp, (long)k, yp, (long)n, m, n, k);
    else
        hipLaunchKernelGGL(qmm_dense_kernel<1>, grid, dim3(256), 0, st, w, at(scales, scales_offset), at(biases, biases_offset), xp, (long)k, yp, (long)n, m, n, k);
    return check_launch(ctx, "int4_qmm");
}

}  // extern "C"

// Prefill / multi-token path: per-token router, (token, expert) pair grouping on the host and on the device, the grouped
// routed-expert computation (row-streaming for small groups, matrix cores for large ones), token-major weighted reduce.
#include <algorithm>
#include <unordered_set>
#include <vector>

#include "tf_prefill_kernels.hpp"
#include "tf_router.hpp"

using namespace tfk;

namespace tfk {
bool qmm_operands_ok(const void *w, const void *x, long ldx_halves, int k);
int32_t launch_grouped_phase1_mfma(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off,
                                   const ChunkList &cl, uint32_t n_chunks_upper, const tf_prefill_pair *pairs,
                                   const half_t *hidden, long hidden_stride, half_t *acts, uint32_t acts_pair_base, int d, int f,
                                   tf_dtype sd, const DenseRide *ride);
int32_t launch_grouped_down_mfma(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off,
                                 const ChunkList &cl, uint32_t n_chunks_upper, const tf_prefill_pair *pairs, const half_t *acts,
                                 uint32_t acts_pair_base, half_t *route_partials, int d, int f, int top_k, tf_dtype sd, const DenseRide *ride);
bool dense_ride_ok(const DenseRide &ride);
int32_t shared_expert_block_plan(tf_ctx *ctx, const void *x, uint64_t x_offset, void *y, uint64_t y_offset, const tf_projection *gate,
                                 const tf_projection *up, const tf_projection *down, void *scratch_gate, uint64_t scratch_gate_offset,
                                 uint64_t scratch_gate_length, void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                                 void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length, uint32_t query_count,
                                 uint32_t d, uint32_t intermediate, uint32_t x_stride_elements, uint32_t y_stride_elements,
                                 uint32_t weight_bits, tf_dtype scale_dtype, DenseRide *plan);
}  // namespace tfk

namespace {

constexpr uint32_t kFewTokens = 64;   // up to here the router runs one wave per (token, expert)

// ------------------------------------------------------------------------------------------------ router block
// One 256-thread block per token row: the four waves share the experts (wave w takes e = w, w+4, ...), the logits meet in
// LDS, wave 0 selects.
template <int NPASS>
__global__ __launch_bounds__(256) void prefill_router_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                             const half_t *hidden, long hidden_stride, const uint16_t *eff,
                                                             const uint16_t *per_expert_scale, uint32_t *out_indices,
                                                             half_t *out_weights, uint32_t num_experts, int d, uint32_t top_k) {
    __shared__ float logits[256];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t t = blockIdx.x;
    const half_t *row = hidden + (size_t)t * hidden_stride;
    const int groups = d >> 6;
    for (uint32_t e = wave; e < num_experts; e += 4) {
        const float v = router_row<0, NPASS>(W + (size_t)e * d, S + (size_t)e * groups * 2, B + (size_t)e * groups * 2, row, eff, d, lane);
        if (lane == 0) logits[e] = v;
    }
    __syncthreads();
    if (wave != 0) return;
    router_select(logits, per_expert_scale, out_indices + (size_t)t * top_k, out_weights + (size_t)t * top_k, num_experts, top_k, lane);
}

// Few tokens (multi-token verification): one wave per (token, expert) logit, then one wave per token selects, so the
// latency is that of a single row however many experts there are.
template <int NPASS>
__global__ __launch_bounds__(256) void prefill_logits_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                             const half_t *hidden, long hidden_stride, const uint16_t *eff,
                                                             float *logits, uint32_t num_experts, int d) {
    const int lane = threadIdx.x & 63;
    const uint32_t e = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint32_t t = blockIdx.y;
    if (e >= num_experts) return;
    const int groups = d >> 6;
    const float v = router_row<0, NPASS>(W + (size_t)e * d, S + (size_t)e * groups * 2, B + (size_t)e * groups * 2,
                                         hidden + (size_t)t * hidden_stride, eff, d, lane);
    if (lane == 0) logits[(size_t)t * num_experts + e] = v;
}

// The same logits with one 256-thread block per (expert, token) where every operand is 16-byte aligned and d <= 4096: thread c
// takes chunk c of 16 weights, so a row is one memory round trip and a sixteenth of a wave's arithmetic (the decode router's
// row, router_row_block).
__global__ __launch_bounds__(256) void prefill_logits_block_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B, const half_t *hidden,
                                                                   long hidden_stride, const uint16_t *eff, float *logits, uint32_t num_experts, int d) {
    __shared__ float partial[4];
    const uint32_t e = blockIdx.x, t = blockIdx.y;
    const int groups = d >> 6;
    const float v = router_row_block<0>(W + (size_t)e * d, S + (size_t)e * groups * 2, B + (size_t)e * groups * 2,
                                        hidden + (size_t)t * hidden_stride, eff, d, partial);
    if (threadIdx.x == 0) logits[(size_t)t * num_experts + e] = v;
}

// planes > 0: the token's logits are first summed, in plane order, from `planes` partial planes that follow the
// [tokens, experts] logits array (each lane sums the entries it will read back), then selected from.
__global__ __launch_bounds__(64) void prefill_select_kernel(float *logits, const uint16_t *per_expert_scale,
                                                            uint32_t *out_indices, half_t *out_weights, uint32_t num_experts,
                                                            uint32_t top_k, uint32_t planes, size_t plane_stride) {
    const uint32_t t = blockIdx.x;
    float *row = logits + (size_t)t * num_experts;
    if (planes > 0) {
        for (uint32_t e = threadIdx.x; e < num_experts; e += 64) {
            float v = 0.0f;
            for (uint32_t p = 1; p <= planes; ++p) v += row[p * plane_stride + e];
            row[e] = v;
        }
    }
    router_select(row, per_expert_scale, out_indices + (size_t)t * top_k, out_weights + (size_t)t * top_k, num_experts, top_k, threadIdx.x);
}

// Many tokens: the router projection as a matrix product on the matrix cores.  A block takes 32 tokens and up to 128
// experts (wave w: experts 32 w ..), one quantization group of 64 at a time:
//   - the 256 threads form x' = float(hidden) * float(effective_scale) for the block's 32 tokens x 64 columns once,
//     split it into two fp16 parts (x' * 16 = hi + lo, so that nothing of its 24 bits is lost) and put both in LDS,
//     together with the fp32 column sums of x' that the bias term needs;
//   - every wave multiplies its 32 experts' 8-bit weights (exact in fp16) with both parts: the products are exact and
//     accumulate in fp32, per group, and the group's scale is applied to the accumulator, as in the reference's
//     arithmetic (s * sum(q x') + b * sum(x'));
//   - the bias term sum_g b[e,g] * sum(x')[t,g] is one more small product over the groups at the end.
// The selection runs afterwards, one wave per token, on the logits this kernel leaves in scratch.
template <int SD>
__global__ __launch_bounds__(256) void prefill_logits_mfma_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                                  const half_t *hidden, long hidden_stride, const uint16_t *eff,
                                                                  float *logits, uint32_t query_count, uint32_t num_experts, int d,
                                                                  int groups_per_split) {
    __shared__ __align__(16) u32x4 x_hi[2][256], x_lo[2][256];   // [stage][a_slot(token, chunk)]
    __shared__ float xsum[32][65];                                // [token][group], padded
    __shared__ __align__(16) u32x4 g_hi[256], g_lo[256];         // the sums as fp16 parts, a_slot(token, chunk of 8 groups)
    __shared__ __align__(16) half_t bias_h[128][64];              // [expert of the block][group] biases as fp16, 0 beyond
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 31, kb = lane >> 5;
    // blockIdx.y: which run of quantization groups this block sums; its partial logits go to plane blockIdx.y
    const int all_groups = d >> 6;
    const int group0 = (int)blockIdx.y * groups_per_split;
    const int groups = min(groups_per_split, all_groups - group0);
    logits += (size_t)blockIdx.y * query_count * num_experts;
    const uint32_t t0 = blockIdx.x * 32;
    // producer role: token p_tok, 8 columns p_chunk * 8 .. of every group
    const int p_tok = threadIdx.x >> 3, p_chunk = threadIdx.x & 7;
    const half_t *p_row = hidden + (size_t)min(t0 + (uint32_t)p_tok, query_count - 1) * hidden_stride + group0 * 64 + p_chunk * 8;
    const uint16_t *p_eff = eff + group0 * 64 + p_chunk * 8;
    const int p_slot = a_slot(p_tok, p_chunk);
    // consumer role: expert row e_row (clamped), the kb-th 32 columns of every group
    const uint32_t e_lane = (uint32_t)wave * 32u + (uint32_t)i;
    const uint32_t e_row = min(e_lane, num_experts - 1);
    const uint8_t *w_row = W + (size_t)e_row * d + group0 * 64 + kb * 32;
    const uint8_t *s_row = S + ((size_t)e_row * all_groups + group0) * 2;
    const uint8_t *b_row = B + ((size_t)e_row * all_groups + group0) * 2;
    const bool wave_live = (uint32_t)wave * 32u < num_experts;

    auto produce = [&](const u32x4 hraw, const u32x4 eraw, int stage, int g) {
        float xv[8], sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t h2 = as_half2(hraw[j]);
            xv[2 * j] = (float)h2[0] * __uint_as_float(eraw[j] << 16);
            xv[2 * j + 1] = (float)h2[1] * __uint_as_float(eraw[j] & 0xFFFF0000u);
            sum += xv[2 * j];
            sum += xv[2 * j + 1];
        }
        u32x4 hi, lo;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            half2_t a, b;
            a[0] = (half_t)(xv[2 * j] * 16.0f);
            a[1] = (half_t)(xv[2 * j + 1] * 16.0f);
            b[0] = (half_t)(xv[2 * j] * 16.0f - (float)a[0]);
            b[1] = (half_t)(xv[2 * j + 1] * 16.0f - (float)a[1]);
            hi[j] = as_u32(a);
            lo[j] = as_u32(b);
        }
        x_hi[stage][p_slot] = hi;
        x_lo[stage][p_slot] = lo;
        sum += dpp_f32<0xB1>(sum);    // the 8 chunks of a token sit in 8 neighbouring lanes
        sum += dpp_f32<0x4E>(sum);
        sum += dpp_f32<0x141>(sum);
        if (p_chunk == 0) xsum[p_tok][g] = sum;
    };
    // 8 bytes (two words) -> 8 fp16 weights in element order, exact
    auto expand8 = [&](uint32_t w0, uint32_t w1) {
        const half2_t k1024 = {(half_t)1024.0f, (half_t)1024.0f};
        const half2_t q0 = as_half2(__builtin_amdgcn_perm(0u, w0, 0x0c010c00u) | 0x64006400u) - k1024;
        const half2_t q1 = as_half2(__builtin_amdgcn_perm(0u, w0, 0x0c030c02u) | 0x64006400u) - k1024;
        const half2_t q2 = as_half2(__builtin_amdgcn_perm(0u, w1, 0x0c010c00u) | 0x64006400u) - k1024;
        const half2_t q3 = as_half2(__builtin_amdgcn_perm(0u, w1, 0x0c030c02u) | 0x64006400u) - k1024;
        return half8_t{q0[0], q0[1], q1[0], q1[1], q2[0], q2[1], q3[0], q3[1]};
    };

    for (int z = threadIdx.x; z < 128 * 64 / 8; z += 256) reinterpret_cast<u32x4 *>(&bias_h[0][0])[z] = u32x4{0u, 0u, 0u, 0u};
    // requests run two groups ahead of their use: one group of MFMAs is much shorter than a trip to L2
    const int g1 = min(1, groups - 1);
    u32x4 hraw = load16(p_row), eraw = load16(p_eff);
    u32x4 wq0 = load16(w_row), wq1 = load16(w_row + 16);
    uint16_t sg = *reinterpret_cast<const uint16_t *>(s_row), bg = *reinterpret_cast<const uint16_t *>(b_row);
    u32x4 h1 = load16(p_row + g1 * 64), e1 = load16(p_eff + g1 * 64);
    u32x4 w10 = load16(w_row + g1 * 64), w11 = load16(w_row + g1 * 64 + 16);
    uint16_t s1 = *reinterpret_cast<const uint16_t *>(s_row + g1 * 2), b1 = *reinterpret_cast<const uint16_t *>(b_row + g1 * 2);
    produce(hraw, eraw, 0, 0);
    lds_barrier();
    float16_t acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.0f;
    for (int g = 0; g < groups; ++g) {
        const int g2 = min(g + 2, groups - 1);
        const u32x4 h2 = load16(p_row + g2 * 64), e2 = load16(p_eff + g2 * 64);
        const u32x4 w20 = load16(w_row + g2 * 64), w21 = load16(w_row + g2 * 64 + 16);
        const uint16_t s2 = *reinterpret_cast<const uint16_t *>(s_row + g2 * 2), b2 = *reinterpret_cast<const uint16_t *>(b_row + g2 * 2);
        if (kb == 0) bias_h[wave * 32 + i][g] = (half_t)sb_to_f32<SD>(bg);
        if (wave_live) {
            const int stage = g & 1;
            float16_t cg, cl;   // two chains: consecutive MFMAs do not wait for each other
#pragma unroll
            for (int r = 0; r < 16; ++r) { cg[r] = 0.0f; cl[r] = 0.0f; }
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const u32x4 wsrc = dd < 2 ? wq0 : wq1;
                const half8_t bf = expand8(wsrc[(dd & 1) * 2], wsrc[(dd & 1) * 2 + 1]);
                const int slot = a_slot(i, kb * 4 + dd);
                const half8_t ah = __builtin_bit_cast(half8_t, x_hi[stage][slot]);
                const half8_t al = __builtin_bit_cast(half8_t, x_lo[stage][slot]);
                cg = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bf, cg, 0, 0, 0);
                cl = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, bf, cl, 0, 0, 0);
            }
            const float sc = sb_to_f32<SD>(sg) * 0.0625f;
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[r] = fmaf(sc, cg[r] + cl[r], acc[r]);
        }
        if (g + 1 < groups) produce(h1, e1, (g + 1) & 1, g + 1);
        wq0 = w10; wq1 = w11; sg = s1; bg = b1;
        h1 = h2; e1 = e2; w10 = w20; w11 = w21; s1 = s2; b1 = b2;
        lds_barrier();
    }
    // bias term: the sums as two fp16 parts (scaled by 16 like x'), the biases as fp16
    {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const int g = p_chunk * 8 + j;
            v[j] = g < groups ? xsum[p_tok][g] * 16.0f : 0.0f;
        }
        u32x4 hi, lo;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            half2_t a, b;
            a[0] = (half_t)v[2 * j];
            a[1] = (half_t)v[2 * j + 1];
            b[0] = (half_t)(v[2 * j] - (float)a[0]);
            b[1] = (half_t)(v[2 * j + 1] - (float)a[1]);
            hi[j] = as_u32(a);
            lo[j] = as_u32(b);
        }
        g_hi[p_slot] = hi;
        g_lo[p_slot] = lo;
    }
    __syncthreads();
    if (!wave_live) return;
    float16_t cb;
#pragma unroll
    for (int r = 0; r < 16; ++r) cb[r] = 0.0f;
    for (int m = 0; m * 16 < groups; ++m) {
        const half8_t bf = *reinterpret_cast<const half8_t *>(&bias_h[wave * 32 + i][m * 16 + kb * 8]);
        const int slot = a_slot(i, m * 2 + kb);
        cb = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, g_hi[slot]), bf, cb, 0, 0, 0);
        cb = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8_t, g_lo[slot]), bf, cb, 0, 0, 0);
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const uint32_t t = t0 + (uint32_t)acc_row(r, lane);
        if (t < query_count && e_lane < num_experts) logits[(size_t)t * num_experts + e_lane] = acc[r] + cb[r] * 0.0625f;
    }
}

// ------------------------------------------------------------------------------------------------ device grouping
// A stable counting sort of the (token, rank) pairs by expert in three short launches.  The tokens are cut into at most
// kGroupSegments segments.  (1) one wave per segment counts its pairs per expert; (2) one block turns the
// [segment, expert] counts into start positions (expert-major, segments in order), per-expert offsets / counts and the
// work list of <= 128-pair chunks; (3) one wave per segment places its pairs, 64 at a time in (token, rank) order, each
// lane ranking itself among the lanes of the same expert with ballots.  Deterministic: no order depends on timing.
__device__ __forceinline__ uint32_t clamp_expert(uint32_t e, uint32_t num_experts) { return e < num_experts ? e : num_experts - 1; }

__device__ __forceinline__ uint32_t wave_inclusive_scan_u32(uint32_t v) {
    auto shifted = [](uint32_t x, auto ctrl, auto rows) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, decltype(ctrl)::value, decltype(rows)::value, 0xF, false);
    };
    v += shifted(v, std::integral_constant<int, 0x111>{}, std::integral_constant<int, 0xF>{});      // row_shr:1 (no source inside the row of 16: adds 0)
    v += shifted(v, std::integral_constant<int, 0x112>{}, std::integral_constant<int, 0xF>{});      // row_shr:2
    v += shifted(v, std::integral_constant<int, 0x114>{}, std::integral_constant<int, 0xF>{});      // row_shr:4
    v += shifted(v, std::integral_constant<int, 0x118>{}, std::integral_constant<int, 0xF>{});      // row_shr:8
    v += shifted(v, std::integral_constant<int, 0x142>{}, std::integral_constant<int, 0xA>{});      // row_bcast15 into rows 1 and 3
    v += shifted(v, std::integral_constant<int, 0x143>{}, std::integral_constant<int, 0xC>{});      // row_bcast31 into rows 2 and 3
    return v;
}

__global__ __launch_bounds__(64) void group_count_kernel(const uint32_t *indices, uint32_t n_pairs, uint32_t seg_pairs,
                                                         uint32_t num_experts, uint32_t *seg_counts) {
    __shared__ uint32_t cnt[256];
    const uint32_t lane = threadIdx.x;
    for (uint32_t e = lane; e < 256; e += 64) cnt[e] = 0;
    __syncthreads();
    const uint32_t first = blockIdx.x * seg_pairs, last = min(first + seg_pairs, n_pairs);
    for (uint32_t i = first + lane; i < last; i += 64) atomicAdd(&cnt[clamp_expert(indices[i], num_experts)], 1u);
    __syncthreads();
    for (uint32_t e = lane; e < 256; e += 64) seg_counts[blockIdx.x * 256 + e] = cnt[e];
}

// 256 threads, thread e owns expert e.  seg_counts[s][e] becomes the position of segment s's first pair of expert e.
__global__ __launch_bounds__(256) void group_scan_kernel(uint32_t *seg_counts, uint32_t n_segments, uint32_t num_experts,
                                                         uint32_t *per_expert_offsets, uint32_t *per_expert_counts,
                                                         tf_prefill_group *chunks, uint32_t *chunk_count) {
    __shared__ uint32_t scan_pairs[4], scan_chunks[4];      // the four waves' totals
    const uint32_t e = threadIdx.x;
    // all of this expert's segment counts are requested at once (one memory round trip), then summed in registers
    uint32_t v[kGroupSegments];
#pragma unroll
    for (uint32_t s = 0; s < kGroupSegments; ++s) v[s] = s < n_segments ? seg_counts[s * 256 + e] : 0u;
    uint32_t total = 0;
#pragma unroll
    for (uint32_t s = 0; s < kGroupSegments; ++s) {
        const uint32_t c = v[s];
        v[s] = total;   // exclusive prefix inside expert e
        total += c;
    }
    const uint32_t nch = (total + kChunkPairs - 1) / kChunkPairs;
    // inclusive scans over the experts: across the lanes of each wave, then the waves before added on
    uint32_t sum_pairs = wave_inclusive_scan_u32(total), sum_chunks = wave_inclusive_scan_u32(nch);
    const uint32_t wave = e >> 6;
    if ((e & 63) == 63) {
        scan_pairs[wave] = sum_pairs;
        scan_chunks[wave] = sum_chunks;
    }
    __syncthreads();
    for (uint32_t w = 0; w < wave; ++w) {
        sum_pairs += scan_pairs[w];
        sum_chunks += scan_chunks[w];
    }
    const uint32_t start = sum_pairs - total, chunk_start = sum_chunks - nch;
    if (e == 255) chunk_count[0] = sum_chunks;
    if (e < num_experts) {
        per_expert_offsets[e] = total ? start : 0xFFFFFFFFu;
        per_expert_counts[e] = total;
    }
#pragma unroll
    for (uint32_t s = 0; s < kGroupSegments; ++s)
        if (s < n_segments) seg_counts[s * 256 + e] = v[s] + start;
    for (uint32_t c = 0; c < nch; ++c) {
        tf_prefill_group g;
        g.expert = e;
        g.pair_start = start + c * kChunkPairs;
        g.pair_count = min(kChunkPairs, total - c * kChunkPairs);
        chunks[chunk_start + c] = g;
    }
}

// Ranks 64 pairs at a time: every lane ORs its bit into its expert's 64-bit mask in LDS, then reads the mask back: the
// set bits below its own are the earlier pairs of the same expert (order = (token, rank) order, whatever the timing).
__device__ __forceinline__ uint32_t place_batch(uint32_t e, bool valid, uint32_t lane, unsigned long long *mask, uint32_t *next) {
    const unsigned long long bit = 1ull << lane;
    if (valid) atomicOr(&mask[e], bit);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    uint32_t pos = 0;
    unsigned long long same = 0ull;
    if (valid) {
        same = mask[e];
        pos = next[e] + (uint32_t)__builtin_popcountll(same & (bit - 1ull));
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    if (valid && (same & (bit - 1ull)) == 0ull) {   // the first pair of its expert in this batch moves the expert on
        next[e] += (uint32_t)__builtin_popcountll(same);
        mask[e] = 0ull;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup", "local");
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup", "local");
    return pos;
}

__global__ __launch_bounds__(64) void group_place_kernel(const uint32_t *indices, const uint16_t *weights, uint32_t n_pairs,
                                                         uint32_t seg_pairs, uint32_t top_k, uint32_t num_experts,
                                                         const uint32_t *seg_starts, tf_prefill_pair *sorted_pairs) {
    __shared__ uint32_t next[256];
    __shared__ unsigned long long mask[256];
    const uint32_t lane = threadIdx.x;
    for (uint32_t e = lane; e < 256; e += 64) {
        next[e] = seg_starts[blockIdx.x * 256 + e];
        mask[e] = 0ull;
    }
    __syncthreads();
    const uint32_t first = blockIdx.x * seg_pairs, last = min(first + seg_pairs, n_pairs);
    for (uint32_t i0 = first; i0 < last; i0 += 64) {
        const uint32_t i = i0 + lane;
        const bool valid = i < last;
        const uint32_t e = valid ? clamp_expert(indices[i], num_experts) : 0u;
        const uint16_t wbits = valid ? weights[i] : (uint16_t)0;
        const uint32_t pos = place_batch(e, valid, lane, mask, next);
        if (valid) {
            tf_prefill_pair p;
            p.token = i / top_k;
            p.expert = e;
            p.rank = i - p.token * top_k;
            p.weight_bits_and_reserved = (uint32_t)wbits;
            sorted_pairs[pos] = p;
        }
    }
}

// Up to kGroupBlockPairs pairs (256 tokens at top-8) in ONE block: the three steps above with the segments (64 pairs each, one
// wave's worth) kept in LDS.  A wave counts its segments' pairs per expert; thread e runs over expert e's segment counts and the
// experts are scanned across lanes; then every wave places its segments' pairs, each lane ranking itself among the lanes of the
// same expert (the lanes whose expert number agrees in every bit: eight ballots).  Every thread of the block must call (block-wide
// barriers); the block has at least 256 threads.  indices / weights may live in LDS.
constexpr uint32_t kGroupBlockPairs = 2048, kGroupBlockSegments = kGroupBlockPairs / 64;
struct GroupBlockLds {
    uint32_t seg[kGroupBlockSegments][256];      // [segment][expert]: pair counts, then the position of the segment's first pair of the expert
    uint32_t wave_pairs[4], wave_chunks[4];      // totals of the four waves that own the experts
};
__device__ __forceinline__ void group_block_body(GroupBlockLds &l, const uint32_t *indices, const uint16_t *weights, uint32_t n_pairs, uint32_t top_k,
                                                 uint32_t num_experts, tf_prefill_pair *sorted_pairs, uint32_t *per_expert_offsets,
                                                 uint32_t *per_expert_counts, tf_prefill_group *chunks, uint32_t *chunk_count) {
    const uint32_t e = threadIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
    const bool owner = e < 256;        // thread e owns expert e
    const uint32_t n_seg = (n_pairs + 63) / 64;
    for (uint32_t i = threadIdx.x; i < n_seg * 256; i += blockDim.x) (&l.seg[0][0])[i] = 0u;
    __syncthreads();
    for (uint32_t s = wave; s < n_seg; s += waves) {
        const uint32_t i = s * 64 + lane;
        if (i < n_pairs) atomicAdd(&l.seg[s][clamp_expert(indices[i], num_experts)], 1u);
    }
    __syncthreads();
    uint32_t total = 0;
    if (owner)
        for (uint32_t s = 0; s < n_seg; ++s) {
            const uint32_t c = l.seg[s][e];
            l.seg[s][e] = total;      // exclusive prefix inside expert e
            total += c;
        }
    const uint32_t nch = (total + kChunkPairs - 1) / kChunkPairs;
    // running sums over the experts: inside each of the four owner waves across lanes, then the waves before added on
    uint32_t sum_pairs = wave_inclusive_scan_u32(total), sum_chunks = wave_inclusive_scan_u32(nch);
    if (owner && lane == 63) {
        l.wave_pairs[wave] = sum_pairs;
        l.wave_chunks[wave] = sum_chunks;
    }
    __syncthreads();
    if (owner) {
        for (uint32_t w = 0; w < wave; ++w) {
            sum_pairs += l.wave_pairs[w];
            sum_chunks += l.wave_chunks[w];
        }
        const uint32_t start = sum_pairs - total, chunk_start = sum_chunks - nch;
        if (e == 255) chunk_count[0] = sum_chunks;
        if (e < num_experts) {
            per_expert_offsets[e] = total ? start : 0xFFFFFFFFu;
            per_expert_counts[e] = total;
        }
        for (uint32_t c = 0; c < nch; ++c) {
            tf_prefill_group g;
            g.expert = e;
            g.pair_start = start + c * kChunkPairs;
            g.pair_count = min(kChunkPairs, total - c * kChunkPairs);
            chunks[chunk_start + c] = g;
        }
        for (uint32_t s = 0; s < n_seg; ++s) l.seg[s][e] += start;
    }
    __syncthreads();
    for (uint32_t s = wave; s < n_seg; s += waves) {
        const uint32_t i = s * 64 + lane;
        const bool valid = i < n_pairs;
        const uint32_t x = valid ? clamp_expert(indices[i], num_experts) : 0x100u;      // bit 8: no pair
        const uint16_t wbits = valid ? weights[i] : (uint16_t)0;
        unsigned long long same = ~0ull;      // the lanes whose expert number equals this lane's
#pragma unroll
        for (uint32_t bit = 0; bit < 9; ++bit) {
            const unsigned long long set = __ballot((x >> bit) & 1u);
            same &= ((x >> bit) & 1u) ? set : ~set;
        }
        if (valid) {
            tf_prefill_pair p;
            p.token = i / top_k;
            p.expert = x;
            p.rank = i - p.token * top_k;
            p.weight_bits_and_reserved = (uint32_t)wbits;
            sorted_pairs[l.seg[s][x] + (uint32_t)__builtin_popcountll(same & ((1ull << lane) - 1ull))] = p;
        }
    }
}
__global__ __launch_bounds__(1024) void group_block_kernel(const uint32_t *indices, const uint16_t *weights, uint32_t n_pairs,
                                                           uint32_t top_k, uint32_t num_experts, tf_prefill_pair *sorted_pairs,
                                                           uint32_t *per_expert_offsets, uint32_t *per_expert_counts,
                                                           tf_prefill_group *chunks, uint32_t *chunk_count) {
    __shared__ GroupBlockLds l;
    group_block_body(l, indices, weights, n_pairs, top_k, num_experts, sorted_pairs, per_expert_offsets, per_expert_counts, chunks, chunk_count);
}

// The selection of up to kSelectGroupTokens token rows and the grouping of their pairs in ONE block of sixteen waves: wave w
// selects for tokens w and w + 16 from the logits the launch before left in scratch (the arithmetic of prefill_select_kernel),
// writes the router's outputs and keeps them in LDS, where the grouping above takes them from.  One launch where the
// router block's selection and the device grouping were two.
constexpr uint32_t kSelectGroupTokens = 32, kSelectGroupTopK = 8;
__global__ __launch_bounds__(1024) void select_group_small_kernel(const float *logits, const uint16_t *per_expert_scale, uint32_t *out_indices,
                                                                  half_t *out_weights, uint32_t tokens, uint32_t num_experts, uint32_t top_k,
                                                                  tf_prefill_pair *sorted_pairs, uint32_t *per_expert_offsets,
                                                                  uint32_t *per_expert_counts, tf_prefill_group *chunks, uint32_t *chunk_count) {
    __shared__ GroupBlockLds l;
    __shared__ uint32_t s_idx[kSelectGroupTokens * kSelectGroupTopK];
    __shared__ uint16_t s_w[kSelectGroupTokens * kSelectGroupTopK];
    const int lane = threadIdx.x & 63;
    for (uint32_t tkn = threadIdx.x >> 6; tkn < tokens; tkn += 16) {
        uint32_t idx;
        half_t weight;
        router_select_lanes(logits + (size_t)tkn * num_experts, per_expert_scale, num_experts, top_k, lane, idx, weight);
        if ((uint32_t)lane < top_k) {
            out_indices[(size_t)tkn * top_k + lane] = idx;
            out_weights[(size_t)tkn * top_k + lane] = weight;
            s_idx[tkn * top_k + lane] = idx;
            s_w[tkn * top_k + lane] = f32_to_f16_bits((float)weight);
        }
    }
    __syncthreads();
    group_block_body(l, s_idx, s_w, tokens * top_k, top_k, num_experts, sorted_pairs, per_expert_offsets, per_expert_counts, chunks, chunk_count);
}

// ------------------------------------------------------------------------------------------------ grouped, row-streaming
// Small groups: a wave loads one tile of gate rows and the same tile of up rows ONCE and applies it to every pair of the
// chunk, so each touched expert is read once however many tokens chose it.
__device__ __forceinline__ void store_act(half_t *acts, size_t index, float gate, float up) {
    acts[index] = (half_t)(gelu_tanh(gate) * up);
}

template <int RT, int NP, int SD>
__global__ __launch_bounds__(256) void grouped_phase1_long_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl,
                                                                  const tf_prefill_pair *pairs, const half_t *hidden,
                                                                  long hidden_stride, half_t *acts, uint32_t acts_pair_base,
                                                                  int d, int f) {
    tf_prefill_group ch;
    if (!get_chunk(cl, blockIdx.y, ch)) return;
    const uint8_t *base = uniform_ptr(expert_base(tab, ch.expert));
    if (!base) return;
    const int lane = threadIdx.x & 63;
    const int tile = uniform_int((int)((blockIdx.x * blockDim.x + threadIdx.x) >> 6));
    const int row0 = tile * RT;
    if (row0 >= f) return;
    const size_t w_byte = (size_t)row0 * (d >> 1), sb_byte = (size_t)row0 * (d >> 6) * 2;
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile tg, tu;
    rs.init_map(d, lane);
    rs.load(tg, base + off.gate_W_off + w_byte, base + off.gate_s_off + sb_byte, base + off.gate_b_off + sb_byte, f - row0);
    rs.load(tu, base + off.up_W_off + w_byte, base + off.up_s_off + sb_byte, base + off.up_b_off + sb_byte, f - row0);
    for (uint32_t j = 0; j < ch.pair_count; ++j) {
        const uint32_t pi = ch.pair_start + j;
        rs.init_x(hidden + (size_t)pairs[pi].token * hidden_stride);
        float gate[RT], up[RT];
        rs.template reduce<SD>(tg, gate);
        rs.template reduce<SD>(tu, up);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
                if (row0 + r < f) store_act(acts, (size_t)(pi - acts_pair_base) * f + row0 + r, gate[r], up[r]);
        }
    }
}

// Few tokens (verification / small batches): the experts' weights dominate and every touched expert must stream through
// once at full rate.  Persistent blocks of 8 waves, one per CU: the activations of ALL tokens (at most kStreamTokens rows)
// are staged once per block in LDS in dot-product order, the chunk list and the pairs' token numbers too, so the tile
// loop touches global memory only for weights (two tile buffers, refilled as soon as reduced) and for the results.
constexpr int kStreamTokens = 16;
constexpr int kStreamMaxD = 4096;
constexpr int kStreamMaxPairs = 256;   // pairs and chunks the LDS copies hold

template <int RT, int NP, int SD>
__global__ __launch_bounds__(512) void grouped_phase1_stream_kernel(ExpertTable tab, tf_expert_offsets off, const tf_prefill_group *chunks,
                                                                    const uint32_t *chunk_count, const tf_prefill_pair *pairs,
                                                                    uint32_t n_pairs, const half_t *hidden, long hidden_stride,
                                                                    uint32_t tokens, half_t *acts, uint32_t acts_pair_base, int d, int f) {
    __shared__ __align__(16) u32x4 xa[kStreamTokens * kStreamMaxD / 8];
    __shared__ float xsum[kStreamTokens * kStreamMaxD / 32];
    __shared__ uint32_t pair_token[kStreamMaxPairs];
    __shared__ uint32_t ch_expert[kStreamMaxPairs], ch_start[kStreamMaxPairs], ch_count[kStreamMaxPairs];
    const int lane = threadIdx.x & 63;
    const int nch = d >> 5, pieces = d >> 3;
    // everything the prologue needs is requested before anything is used
    u32x4 raw[kStreamTokens];
#pragma unroll
    for (int t = 0; t < kStreamTokens; ++t) {
        raw[t] = u32x4{0u, 0u, 0u, 0u};
        if ((uint32_t)t < tokens && (int)threadIdx.x < pieces) raw[t] = load16(hidden + (size_t)t * hidden_stride + threadIdx.x * 8);
    }
    uint32_t n_chunks = *chunk_count;
    n_chunks = n_chunks < (uint32_t)kStreamMaxPairs ? n_chunks : (uint32_t)kStreamMaxPairs;
    if (threadIdx.x < n_chunks) {
        const tf_prefill_group c = chunks[threadIdx.x];
        ch_expert[threadIdx.x] = c.expert;
        ch_start[threadIdx.x] = c.pair_start;
        ch_count[threadIdx.x] = c.pair_count;
    }
    if (threadIdx.x < n_pairs) {
        const uint32_t t = pairs[threadIdx.x].token;
        pair_token[threadIdx.x] = t < tokens ? t : tokens - 1;
    }
    __syncthreads();
    const uint32_t tpe = (uint32_t)(f + RT - 1) / RT;                 // tiles per expert
    const uint32_t total = n_chunks * tpe;
    const uint32_t wave = uniform_u32((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
    const uint32_t nwaves = (gridDim.x * blockDim.x) >> 6;
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile ga, ua, gb, ub;
    rs.init_map(d, lane);
    auto request = [&](typename RowStream<RT, NP>::Tile &tg, typename RowStream<RT, NP>::Tile &tu, uint32_t at) {
        const uint32_t c = uniform_u32(at / tpe);
        const uint32_t row0 = (at - c * tpe) * RT;
        const uint8_t *base = uniform_ptr(expert_base(tab, ch_expert[c]));
        const size_t w_byte = (size_t)row0 * (d >> 1), sb_byte = (size_t)row0 * (d >> 6) * 2;
        rs.load(tg, base + off.gate_W_off + w_byte, base + off.gate_s_off + sb_byte, base + off.gate_b_off + sb_byte, f - row0);
        rs.load(tu, base + off.up_W_off + w_byte, base + off.up_s_off + sb_byte, base + off.up_b_off + sb_byte, f - row0);
    };
    uint32_t t0 = wave, t1 = wave + nwaves;
    if (t0 < total) request(ga, ua, t0);
    if (t1 < total) request(gb, ub, t1);
    // arrange the activations while the first tiles are in flight
#pragma unroll
    for (int t = 0; t < kStreamTokens; ++t)
        if ((uint32_t)t < tokens) XStage::publish_piece(raw[t], threadIdx.x, pieces, nch, xa + (size_t)t * pieces, xsum + (size_t)t * nch);
    __syncthreads();
    if (t0 >= total) return;
    auto consume = [&](const typename RowStream<RT, NP>::Tile &tg, const typename RowStream<RT, NP>::Tile &tu, uint32_t at) {
        const uint32_t c = uniform_u32(at / tpe);
        const uint32_t row0 = (at - c * tpe) * RT;
        const uint32_t first = uniform_u32(ch_start[c]), count = uniform_u32(ch_count[c]);
        for (uint32_t j = 0; j < count; ++j) {
            const uint32_t pi = first + j;
            const uint32_t token = uniform_u32(pair_token[pi < (uint32_t)kStreamMaxPairs ? pi : 0]);
            rs.init_x_lds(xa + (size_t)token * pieces, xsum + (size_t)token * nch, d);
            float gate[RT], up[RT];
            rs.template reduce<SD>(tg, gate);
            rs.template reduce<SD>(tu, up);
            if (lane == 0) {
#pragma unroll
                for (int r = 0; r < RT; ++r)
                    if (row0 + r < (uint32_t)f) store_act(acts, (size_t)(pi - acts_pair_base) * f + row0 + r, gate[r], up[r]);
            }
        }
    };
    for (;;) {
        consume(ga, ua, t0);
        t0 += 2 * nwaves;
        if (t0 < total) request(ga, ua, t0);
        if (t1 >= total) break;
        consume(gb, ub, t1);
        t1 += 2 * nwaves;
        if (t1 < total) request(gb, ub, t1);
        if (t0 >= total) break;
    }
}


template <int SD>
__global__ __launch_bounds__(256) void grouped_phase1_generic_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl,
                                                                     const tf_prefill_pair *pairs, const half_t *hidden,
                                                                     long hidden_stride, half_t *acts, uint32_t acts_pair_base,
                                                                     int d, int f) {
    tf_prefill_group ch;
    if (!get_chunk(cl, blockIdx.y, ch)) return;
    const uint8_t *base = expert_base(tab, ch.expert);
    if (!base) return;
    const int lane = threadIdx.x & 63;
    const int r = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (r >= f) return;
    const int groups = d >> 6;
    const size_t w_byte = (size_t)r * (d >> 1), sb_byte = (size_t)r * groups * 2;
    for (uint32_t j = 0; j < ch.pair_count; ++j) {
        const uint32_t pi = ch.pair_start + j;
        const half_t *x = hidden + (size_t)pairs[pi].token * hidden_stride;
        const float gate = generic_row_dot<SD>(base + off.gate_W_off + w_byte, base + off.gate_s_off + sb_byte, base + off.gate_b_off + sb_byte, x, d, lane);
        const float up = generic_row_dot<SD>(base + off.up_W_off + w_byte, base + off.up_s_off + sb_byte, base + off.up_b_off + sb_byte, x, d, lane);
        if (lane == 0) store_act(acts, (size_t)(pi - acts_pair_base) * f + r, gate, up);
    }
}

// down rows, F <= 1024: half-wave per row, 2 * NPASS rows per wave, loaded once, applied to every pair of the chunk
template <int NPASS, int SD>
__global__ __launch_bounds__(256) void grouped_down_short_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl,
                                                                 const tf_prefill_pair *pairs, const half_t *acts,
                                                                 uint32_t acts_pair_base, half_t *route_partials, int d, int f,
                                                                 int top_k) {
    tf_prefill_group ch;
    if (!get_chunk(cl, blockIdx.y, ch)) return;
    const uint8_t *base = expert_base(tab, ch.expert);
    if (!base) return;
    const int lane = threadIdx.x & 63;
    const long row0 = (long)((blockIdx.x * blockDim.x + threadIdx.x) >> 6) * 2 * NPASS;
    if (row0 >= d) return;
    ShortRows sr;
    ShortRows::Pair t[NPASS];
    sr.init_map(f, lane);
#pragma unroll
    for (int p = 0; p < NPASS; ++p)
        sr.load(t[p], base + off.down_W_off, base + off.down_s_off, base + off.down_b_off, row0 + 2 * p, d, f);
    // the pair record and the activations of pair j + 1 are requested before pair j is reduced
    const int col = sr.col < 0 ? 0 : sr.col;
    auto fetch = [&](uint32_t j, tf_prefill_pair &pr, u32x4 *xr) {
        pr = pairs[ch.pair_start + j];
        const half_t *a = acts + (size_t)(ch.pair_start + j - acts_pair_base) * f + col * 32;
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) xr[dd] = load16(a + dd * 8);
    };
    tf_prefill_pair pr, pr_next;
    u32x4 xr[4], xr_next[4];
    fetch(0, pr, xr);
    for (uint32_t j = 0; j < ch.pair_count; ++j) {
        if (j + 1 < ch.pair_count) fetch(j + 1, pr_next, xr_next);
        sr.xs = arrange_x(xr, sr.xq);
        half_t *out = route_partials + ((size_t)pr.token * top_k + pr.rank) * d;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            float lo, hi;
            sr.template reduce<SD>(t[p], lo, hi);
            if (lane == 0) {
                if (row0 + 2 * p < d) out[row0 + 2 * p] = (half_t)lo;
                if (row0 + 2 * p + 1 < d) out[row0 + 2 * p + 1] = (half_t)hi;
            }
        }
        pr = pr_next;
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) xr[dd] = xr_next[dd];
    }
}

template <int SD>
__global__ __launch_bounds__(256) void grouped_down_generic_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl,
                                                                   const tf_prefill_pair *pairs, const half_t *acts,
                                                                   uint32_t acts_pair_base, half_t *route_partials, int d, int f,
                                                                   int top_k) {
    tf_prefill_group ch;
    if (!get_chunk(cl, blockIdx.y, ch)) return;
    const uint8_t *base = expert_base(tab, ch.expert);
    if (!base) return;
    const int lane = threadIdx.x & 63;
    const int r = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (r >= d) return;
    const int groups = f >> 6;
    for (uint32_t j = 0; j < ch.pair_count; ++j) {
        const tf_prefill_pair pr = pairs[ch.pair_start + j];
        const float v = generic_row_dot<SD>(base + off.down_W_off + (size_t)r * (f >> 1), base + off.down_s_off + (size_t)r * groups * 2,
                                            base + off.down_b_off + (size_t)r * groups * 2,
                                            acts + (size_t)(ch.pair_start + j - acts_pair_base) * f, f, lane);
        if (lane == 0) route_partials[((size_t)pr.token * top_k + pr.rank) * d + r] = (half_t)v;
    }
}

// ------------------------------------------------------------------------------------------------ reduce
__global__ __launch_bounds__(256) void reduce_token_major_kernel(const half_t *partials, const half_t *weights, half_t *h2,
                                                                 uint32_t T, uint32_t top_k, uint32_t D) {
    const uint32_t c = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t t = blockIdx.y;
    if (c >= D || t >= T) return;
    float acc = 0.0f;
    for (uint32_t r = 0; r < top_k; ++r)
        acc = fmaf((float)weights[t * top_k + r], (float)partials[((size_t)t * top_k + r) * D + c], acc);
    h2[(size_t)t * D + c] = (half_t)acc;
}

// Same sums, eight columns a thread: 16-byte aligned operands and D % 8 == 0. Each column still adds its ranks in rank order.
constexpr uint32_t kReduceRanksInFlight = 8;
__global__ __launch_bounds__(256) void reduce_token_major_vec_kernel(const half_t *partials, const half_t *weights, half_t *h2,
                                                                     uint32_t T, uint32_t top_k, uint32_t D) {
    // threads are numbered through all (token, eight columns) pieces: every block is full whatever D is
    const uint32_t per_token = D / 8, piece = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t t = piece / per_token, c = (piece - t * per_token) * 8;
    if (t >= T) return;
    float acc[8] = {};
    for (uint32_t r0 = 0; r0 < top_k; r0 += kReduceRanksInFlight) {
        u32x4 raw[kReduceRanksInFlight];
        float w[kReduceRanksInFlight];
#pragma unroll
        for (uint32_t j = 0; j < kReduceRanksInFlight; ++j) {
            const uint32_t r = min(r0 + j, top_k - 1);
            raw[j] = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(partials + ((size_t)t * top_k + r) * D + c));   // read once
            w[j] = (float)weights[t * top_k + r];
        }
#pragma unroll
        for (uint32_t j = 0; j < kReduceRanksInFlight; ++j) {
            if (r0 + j >= top_k) break;
            const half_t *v = reinterpret_cast<const half_t *>(&raw[j]);
#pragma unroll
            for (uint32_t e = 0; e < 8; ++e) acc[e] = fmaf(w[j], (float)v[e], acc[e]);
        }
    }
    uint4 packed;
    half_t *o = reinterpret_cast<half_t *>(&packed);
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e) o[e] = (half_t)acc[e];
    *reinterpret_cast<uint4 *>(h2 + (size_t)t * D + c) = packed;
}

// ------------------------------------------------------------------------------------------------ launch helpers

bool table_aligned(const ExpertTable &t) {
    if (t.pool) return aligned16(t.pool) && t.stride % 16 == 0;
    for (uint32_t i = 0; i < t.live; ++i)
        if (!aligned16(t.blob[i])) return false;
    return true;
}

// use_mfma: the chunks are large enough for the matrix cores to pay.  ride: a shared expert's dense tiles to place ahead of the
// grouped tiles when both stages run on the matrix-core tile kernels; *ride_taken says whether that happened.
int32_t run_grouped(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off, const ChunkList &cl,
                    uint32_t n_chunks_upper, const GroupedGeom &g, tf_dtype sd, bool use_mfma, uint32_t stream_tokens = 0,
                    uint32_t stream_pairs = 0, const DenseRide *ride = nullptr, bool *ride_taken = nullptr) {
    if (ride_taken) *ride_taken = false;
    if (n_chunks_upper == 0) return TF_OK;
    const bool blobs16 = table_aligned(tab);
    const bool hidden16 = aligned16(g.hidden) && g.hidden_stride % 8 == 0;
    const bool acts16 = aligned16(g.acts);
    const bool p1_fast = blobs16 && hidden16 && off.gate_W_off % 16 == 0 && off.up_W_off % 16 == 0;
    const bool dn_fast = blobs16 && acts16 && off.down_W_off % 16 == 0;
    int32_t rc;
    // Fewer than five pairs per expert on average: the quad kernels serve the call (chunks longer than their LDS image, if any,
    // in batches).  From there on so few chunks are short that the matrix-core tile kernels are faster (128 experts: 64 tokens
    // 151 us on the quad kernels against 164 us on the tiles; 80 tokens 178 against 173 us; 96 tokens 187 against 173 us; running
    // both families in one call, each on its chunks, was never better than the better of the two).
    const int p1_passes = ((g.d >> 5) + 15) / 16, dn_passes = ((g.f >> 5) + 7) / 8;
    const bool quad_ok = p1_fast && dn_fast && acts16 && g.d <= kQuadMaxD && p1_passes <= 6 && g.f <= kQuadMaxF && dn_passes <= 4 && g.d % 8 == 0 &&
                         g.f % 4 == 0 && aligned(g.route_partials, 8) && aligned(g.acts, 8) && tab.pool != nullptr;
    const bool quad_pays = !use_mfma || (stream_pairs != 0 && (uint64_t)stream_pairs < (uint64_t)tab.num_experts * 5);
    if (quad_ok && quad_pays) return launch_grouped_quad(ctx, st, tab, off, cl, n_chunks_upper, g, sd, stream_pairs);
    const bool p1_tiles = use_mfma && p1_fast && acts16, dn_tiles = use_mfma && dn_fast && aligned16(g.route_partials);
    if (!(p1_tiles && dn_tiles) || (ride && !dense_ride_ok(*ride))) ride = nullptr;
    if (ride && ride_taken) *ride_taken = true;
    // ---- phase 1
    if (p1_tiles) {
        rc = launch_grouped_phase1_mfma(ctx, st, tab, off, cl, n_chunks_upper, g.pairs, g.hidden, g.hidden_stride, g.acts, g.acts_pair_base, g.d, g.f, sd, ride);
    } else {
        const LongPlan plan = plan_long_rows(g.d);
        bool launched = false;
        // all tokens known and few: persistent streaming with the activations staged in LDS
        if (p1_fast && tab.pool && cl.dev && stream_tokens > 0 && stream_tokens <= (uint32_t)kStreamTokens && stream_pairs <= (uint32_t)kStreamMaxPairs &&
            g.d > 1024 && g.d <= kStreamMaxD && g.d <= 512 * 8 && plan.rt > 0) {
            const dim3 grid((uint32_t)ctx->num_cus);
#define TF_GP1S(RT_, NP_)                                                                                                  \
    if (!launched && plan.rt == RT_ && plan.np == NP_) {                                                                   \
        launched = true;                                                                                                   \
        if (sd == TF_BF16)                                                                                                 \
            hipLaunchKernelGGL((grouped_phase1_stream_kernel<RT_, NP_, 0>), grid, dim3(512), 0, st, tab, off, cl.dev, cl.dev_n, g.pairs, \
                               stream_pairs, g.hidden, g.hidden_stride, stream_tokens, g.acts, g.acts_pair_base, g.d, g.f); \
        else                                                                                                               \
            hipLaunchKernelGGL((grouped_phase1_stream_kernel<RT_, NP_, 1>), grid, dim3(512), 0, st, tab, off, cl.dev, cl.dev_n, g.pairs, \
                               stream_pairs, g.hidden, g.hidden_stride, stream_tokens, g.acts, g.acts_pair_base, g.d, g.f); \
    }
            TF_GP1S(1, 1) TF_GP1S(1, 2) TF_GP1S(1, 3) TF_GP1S(1, 4) TF_GP1S(2, 1) TF_GP1S(2, 2) TF_GP1S(2, 3) TF_GP1S(2, 4)
            TF_GP1S(4, 1) TF_GP1S(4, 2) TF_GP1S(4, 3) TF_GP1S(4, 4)
#undef TF_GP1S
        }
        if (!launched && p1_fast && g.d > 1024 && plan.rt > 0) {
            const dim3 grid(((g.f + plan.rt - 1) / plan.rt + 3) / 4, n_chunks_upper);
#define TF_GP1(RT_, NP_)                                                                                                   \
    if (!launched && plan.rt == RT_ && plan.np == NP_) {                                                                   \
        launched = true;                                                                                                   \
        if (sd == TF_BF16)                                                                                                 \
            hipLaunchKernelGGL((grouped_phase1_long_kernel<RT_, NP_, 0>), grid, dim3(256), 0, st, tab, off, cl, g.pairs,   \
                               g.hidden, g.hidden_stride, g.acts, g.acts_pair_base, g.d, g.f);                             \
        else                                                                                                               \
            hipLaunchKernelGGL((grouped_phase1_long_kernel<RT_, NP_, 1>), grid, dim3(256), 0, st, tab, off, cl, g.pairs,   \
                               g.hidden, g.hidden_stride, g.acts, g.acts_pair_base, g.d, g.f);                             \
    }
            TF_GP1(1, 1) TF_GP1(1, 2) TF_GP1(1, 3) TF_GP1(1, 4) TF_GP1(2, 1) TF_GP1(2, 2) TF_GP1(2, 3) TF_GP1(2, 4)
            TF_GP1(4, 1) TF_GP1(4, 2) TF_GP1(4, 3) TF_GP1(4, 4)
#undef TF_GP1
        }
        if (!launched) {
            const dim3 grid((g.f + 3) / 4, n_chunks_upper);
            if (sd == TF_BF16)
                hipLaunchKernelGGL(grouped_phase1_generic_kernel<0>, grid, dim3(256), 0, st, tab, off, cl, g.pairs, g.hidden, g.hidden_stride, g.acts, g.acts_pair_base, g.d, g.f);
            else
                hipLaunchKernelGGL(grouped_phase1_generic_kernel<1>, grid, dim3(256), 0, st, tab, off, cl, g.pairs, g.hidden, g.hidden_stride, g.acts, g.acts_pair_base, g.d, g.f);
        }
        rc = check_launch(ctx, "grouped phase 1");
    }
    if (rc != TF_OK) return rc;
    // ---- down
    if (dn_tiles) {
        return launch_grouped_down_mfma(ctx, st, tab, off, cl, n_chunks_upper, g.pairs, g.acts, g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k, sd, ride);
    }
    if (dn_fast && g.f <= 1024) {
        constexpr int NPASS = 4;
        const dim3 grid(((g.d + 2 * NPASS - 1) / (2 * NPASS) + 3) / 4, n_chunks_upper);
        if (sd == TF_BF16)
            hipLaunchKernelGGL((grouped_down_short_kernel<NPASS, 0>), grid, dim3(256), 0, st, tab, off, cl, g.pairs, g.acts, g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k);
        else
            hipLaunchKernelGGL((grouped_down_short_kernel<NPASS, 1>), grid, dim3(256), 0, st, tab, off, cl, g.pairs, g.acts, g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k);
    } else {
        const dim3 grid((g.d + 3) / 4, n_chunks_upper);
        if (sd == TF_BF16)
            hipLaunchKernelGGL(grouped_down_generic_kernel<0>, grid, dim3(256), 0, st, tab, off, cl, g.pairs, g.acts, g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k);
        else
            hipLaunchKernelGGL(grouped_down_generic_kernel<1>, grid, dim3(256), 0, st, tab, off, cl, g.pairs, g.acts, g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k);
    }
    return check_launch(ctx, "grouped down");
}

}  // namespace

namespace {

// The router logits of up to kFewTokens token rows into `logits` [tokens, experts]: a block per (expert, token) for aligned
// operands (fast), else a wave per (expert, token) with byte loads.
void launch_few_token_logits(hipStream_t st, const uint8_t *w, const uint8_t *s, const uint8_t *b, const half_t *h, uint32_t hidden_stride_elements,
                             const uint16_t *eff, float *logits, uint32_t query_count, uint32_t num_experts, uint32_t d, bool fast) {
    if (fast)
        hipLaunchKernelGGL(prefill_logits_block_kernel, dim3(num_experts, query_count), dim3(256), 0, st, w, s, b, h, (long)hidden_stride_elements, eff,
                           logits, num_experts, (int)d);
    else
        hipLaunchKernelGGL(prefill_logits_kernel<0>, dim3((num_experts + 3) / 4, query_count), dim3(256), 0, st, w, s, b, h,
                           (long)hidden_stride_elements, eff, logits, num_experts, (int)d);
}

}  // namespace

namespace tfk {

// logits [tokens, experts] plus up to four partial planes of the split reduction, never less than the few-token router needs
size_t prefill_logits_floats_for(uint32_t tokens, uint32_t experts) {
    return std::max<size_t>((size_t)kFewTokens * 256, (size_t)tokens * experts * 5);
}

}  // namespace tfk

extern "C" {

int32_t tf_prefill_router_gemma4_block(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset,
                                       const void *scales, uint64_t scales_offset, const void *biases, uint64_t biases_offset,
                                       const void *hidden, uint64_t hidden_offset, const void *effective_scale,
                                       uint64_t effective_scale_offset, const void *per_expert_scale,
                                       uint64_t per_expert_scale_offset, void *out_indices, uint64_t out_indices_offset,
                                       void *out_weights, uint64_t out_weights_offset, uint32_t query_count, uint32_t num_experts,
                                       uint32_t d, uint32_t top_k, uint32_t hidden_stride_elements) {
    TF_REQUIRE(ctx, ctx && weights && scales && biases && hidden && effective_scale && per_expert_scale && out_indices && out_weights,
               TF_ERR_INVALID_ARGUMENT, "prefill_router: null argument");
    TF_REQUIRE(ctx, query_count > 0, TF_ERR_INVALID_ARGUMENT, "prefill_router: queryCount must be positive");
    TF_REQUIRE(ctx, num_experts > 0 && num_experts <= 256, TF_ERR_INVALID_ARGUMENT, "prefill_router: numExperts > 256 is not supported");
    TF_REQUIRE(ctx, top_k > 0 && top_k <= 64, TF_ERR_INVALID_ARGUMENT, "prefill_router: topK must be in 1...64");
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "prefill_router: D must be a multiple of 64");
    TF_REQUIRE(ctx, hidden_stride_elements >= d, TF_ERR_INVALID_ARGUMENT, "prefill_router: hidden stride is too small");
    const uint8_t *w = at(weights, weights_offset);
    const uint8_t *s = at(scales, scales_offset), *b = at(biases, biases_offset);
    const half_t *h = reinterpret_cast<const half_t *>(at(hidden, hidden_offset));
    const uint16_t *eff = reinterpret_cast<const uint16_t *>(at(effective_scale, effective_scale_offset));
    const uint16_t *pes = reinterpret_cast<const uint16_t *>(at(per_expert_scale, per_expert_scale_offset));
    uint32_t *oi = reinterpret_cast<uint32_t *>(at(out_indices, out_indices_offset));
    half_t *ow = reinterpret_cast<half_t *>(at(out_weights, out_weights_offset));
    TF_REQUIRE(ctx, aligned(s, 2) && aligned(b, 2) && aligned(h, 2) && aligned(eff, 2) && aligned(pes, 2) && aligned(oi, 4) && aligned(ow, 2),
               TF_ERR_INVALID_ARGUMENT, "prefill_router: misaligned operand");
    const bool fast = aligned16(w) && aligned16(h) && aligned16(eff) && hidden_stride_elements % 8 == 0 && d <= 4096;
    const int npass = fast ? (int)((d / 16 + 63) / 64) : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool mfma_ok = fast && num_experts <= 128 && d <= 4096 && aligned16(w) && d % 64 == 0;
    if (query_count <= kFewTokens || mfma_ok) {
        // many tokens: enough blocks to fill the chip, by cutting the reduction dimension into up to sixteen runs of groups
        // whose partial logits the selection kernel adds up in a fixed order
        const uint32_t token_blocks = (query_count + 31) / 32;
        const uint32_t groups = d / 64;
        const size_t plane = (size_t)query_count * num_experts;
        uint32_t splits = 1;
        if (query_count > kFewTokens) {
            // a block's time is a fixed part plus its run of groups (12.5 us for 11 groups at 128 tokens): runs of at least three
            // groups, as many as the scratch holds planes for (it is sized for four at the largest call), every run non-empty
            while (splits < 16 && token_blocks * splits < (uint32_t)ctx->num_cus && groups / (splits * 2) >= 3) splits *= 2;
            while (splits > 1 && plane * (1 + splits) > ctx->prefill_logits_count) splits /= 2;
            const uint32_t run = (groups + splits - 1) / splits;
            splits = (groups + run - 1) / run;
        }
        const uint32_t planes = splits > 1 ? splits : 0;   // partial planes behind the logits
        const size_t need = std::max<size_t>((size_t)kFewTokens * 256, plane * (1 + planes));
        if (ctx->prefill_logits_count < need)
            return scratch_too_small(ctx, "prefill_router", need * sizeof(float), ctx->prefill_logits_count * sizeof(float));
        if (query_count > kFewTokens) {
            const int groups_per_split = (int)((groups + splits - 1) / splits);
            hipLaunchKernelGGL(prefill_logits_mfma_kernel<0>, dim3(token_blocks, splits), dim3(256), 0, st, w, s, b, h,
                               (long)hidden_stride_elements, eff, ctx->prefill_logits + (planes ? plane : 0), query_count, num_experts, (int)d,
                               groups_per_split);
        } else {
            launch_few_token_logits(st, w, s, b, h, hidden_stride_elements, eff, ctx->prefill_logits, query_count, num_experts, d, fast);
        }
        const int32_t rc = check_launch(ctx, "prefill_router logits");
        if (rc != TF_OK) return rc;
        hipLaunchKernelGGL(prefill_select_kernel, dim3(query_count), dim3(64), 0, st, ctx->prefill_logits, pes, oi, ow, num_experts, top_k, planes, plane);
        return check_launch(ctx, "prefill_router select");
    }
#define TF_PR(NP_)                                                                                                           \
    hipLaunchKernelGGL(prefill_router_kernel<NP_>, dim3(query_count), dim3(256), 0, st, w, s, b, h, (long)hidden_stride_elements, \
                       eff, pes, oi, ow, num_experts, (int)d, top_k)
    switch (npass) {
        case 1: TF_PR(1); break;
        case 2: TF_PR(2); break;
        case 3: TF_PR(3); break;
        case 4: TF_PR(4); break;
        default: TF_PR(0); break;
    }
#undef TF_PR
    return check_launch(ctx, "prefill_router_gemma4_block");
}

int32_t tf_prefill_make_token_expert_pairs(const uint32_t *indices, const uint16_t *weights_f16, int32_t query_count, int32_t top_k,
                                           tf_prefill_pair *pairs) {
    if (query_count < 0 || top_k < 0) return TF_ERR_INVALID_ARGUMENT;
    if ((int64_t)query_count * top_k > 0 && (!indices || !weights_f16 || !pairs)) return TF_ERR_INVALID_ARGUMENT;
    for (int32_t token = 0; token < query_count; ++token)
        for (int32_t rank = 0; rank < top_k; ++rank) {
            const int64_t i = (int64_t)token * top_k + rank;
            pairs[i].token = (uint32_t)token;
            pairs[i].expert = indices[i];
            pairs[i].rank = (uint32_t)rank;
            pairs[i].weight_bits_and_reserved = (uint32_t)weights_f16[i];
        }
    return TF_OK;
}

int32_t tf_prefill_group_token_expert_pairs(const tf_prefill_pair *pairs, uint64_t pair_count, int32_t query_count, int32_t top_k,
                                            int32_t num_experts, int32_t tile_expert_count, const uint64_t *expert_sort_keys,
                                            uint64_t expert_sort_key_count, tf_prefill_pair *sorted_pairs,
                                            uint32_t *per_expert_offsets, uint32_t *per_expert_counts, tf_prefill_group *groups,
                                            uint32_t *group_count, tf_prefill_tile *tiles, uint32_t *tile_count) {
    if (query_count < 0) return TF_ERR_GROUP_INVALID_QUERY_COUNT;
    if (top_k <= 0) return TF_ERR_GROUP_INVALID_TOP_K;
    if (num_experts <= 0) return TF_ERR_GROUP_INVALID_NUM_EXPERTS;
    if (tile_expert_count < 1 || tile_expert_count > (int32_t)TF_MAX_TILE_EXPERTS) return TF_ERR_GROUP_INVALID_TILE_EXPERT_COUNT;
    if (expert_sort_keys && expert_sort_key_count != (uint64_t)num_experts) return TF_ERR_GROUP_SORT_KEY_COUNT_MISMATCH;
    if (pair_count != (uint64_t)query_count * (uint64_t)top_k) return TF_ERR_GROUP_PAIR_COUNT_MISMATCH;
    if (!per_expert_offsets || !per_expert_counts || !group_count || !tile_count) return TF_ERR_INVALID_ARGUMENT;
    if (pair_count && (!pairs || !sorted_pairs || !groups || !tiles)) return TF_ERR_INVALID_ARGUMENT;

    std::unordered_set<uint64_t> seen;
    seen.reserve((size_t)pair_count);
    for (uint64_t i = 0; i < pair_count; ++i) {
        if (pairs[i].token >= (uint32_t)query_count) return TF_ERR_GROUP_TOKEN_OUT_OF_RANGE;
        if (pairs[i].rank >= (uint32_t)top_k) return TF_ERR_GROUP_RANK_OUT_OF_RANGE;
        if (pairs[i].expert >= (uint32_t)num_experts) return TF_ERR_GROUP_EXPERT_OUT_OF_RANGE;
        if (!seen.insert(((uint64_t)pairs[i].token << 32) | pairs[i].rank).second) return TF_ERR_GROUP_DUPLICATE_TOKEN_RANK;
    }
    std::vector<uint32_t> order((size_t)pair_count);
    for (uint64_t i = 0; i < pair_count; ++i) order[(size_t)i] = (uint32_t)i;
    std::sort(order.begin(), order.end(), [&](uint32_t ia, uint32_t ib) {
        const tf_prefill_pair &a = pairs[ia], &b = pairs[ib];
        if (expert_sort_keys && expert_sort_keys[a.expert] != expert_sort_keys[b.expert])
            return expert_sort_keys[a.expert] < expert_sort_keys[b.expert];
        if (a.expert != b.expert) return a.expert < b.expert;
        if (a.token != b.token) return a.token < b.token;
        return a.rank < b.rank;
    });
    for (int32_t e = 0; e < num_experts; ++e) {
        per_expert_offsets[e] = 0xFFFFFFFFu;
        per_expert_counts[e] = 0;
    }
    uint32_t ng = 0;
    for (uint64_t i = 0; i < pair_count;) {
        const uint32_t expert = pairs[order[(size_t)i]].expert;
        const uint64_t first = i;
        while (i < pair_count && pairs[order[(size_t)i]].expert == expert) {
            sorted_pairs[i] = pairs[order[(size_t)i]];
            ++i;
        }
        per_expert_offsets[expert] = (uint32_t)first;
        per_expert_counts[expert] = (uint32_t)(i - first);
        groups[ng].expert = expert;
        groups[ng].pair_start = (uint32_t)first;
        groups[ng].pair_count = (uint32_t)(i - first);
        ++ng;
    }
    uint32_t nt = 0;
    for (uint32_t gs = 0; gs < ng; gs += (uint32_t)tile_expert_count) {
        const uint32_t ge = std::min(ng, gs + (uint32_t)tile_expert_count);
        tiles[nt].group_start = gs;
        tiles[nt].group_count = ge - gs;
        tiles[nt].pair_start = groups[gs].pair_start;
        tiles[nt].pair_count = groups[ge - 1].pair_start + groups[ge - 1].pair_count - groups[gs].pair_start;
        ++nt;
    }
    *group_count = ng;
    *tile_count = nt;
    return TF_OK;
}

int32_t tf_prefill_group_pairs_device(tf_ctx *ctx, tf_stream stream, const void *indices, const void *weights, uint32_t query_count,
                                      uint32_t top_k, uint32_t num_experts, void *sorted_pairs, void *per_expert_offsets,
                                      void *per_expert_counts, void *chunks, void *chunk_count) {
    TF_REQUIRE(ctx, ctx && indices && weights && sorted_pairs && per_expert_offsets && per_expert_counts && chunks && chunk_count,
               TF_ERR_INVALID_ARGUMENT, "group_pairs_device: null argument");
    TF_REQUIRE(ctx, query_count > 0 && top_k > 0 && num_experts > 0 && num_experts <= 256, TF_ERR_INVALID_ARGUMENT,
               "group_pairs_device: need queryCount > 0, topK > 0, 1 <= numExperts <= 256");
    TF_REQUIRE(ctx, aligned(indices, 4) && aligned(weights, 2) && aligned(sorted_pairs, 4) && aligned(chunks, 4), TF_ERR_INVALID_ARGUMENT,
               "group_pairs_device: misaligned operand");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t n_pairs = query_count * top_k;
    // whole tokens per segment, at least 32 of them, at most kGroupSegments segments
    const uint32_t seg_tokens = std::max<uint32_t>(32u, (query_count + kGroupSegments - 1) / kGroupSegments);
    const uint32_t n_segments = (query_count + seg_tokens - 1) / seg_tokens;
    const uint32_t seg_pairs = seg_tokens * top_k;
    const uint32_t *idx = static_cast<const uint32_t *>(indices);
    if (n_pairs <= kGroupBlockPairs) {
        const uint32_t threads = n_pairs <= 256 ? 256u : n_pairs <= 512 ? 512u : 1024u;      // a wave per 64 pairs, at least the 256 expert owners
        hipLaunchKernelGGL(group_block_kernel, dim3(1), dim3(threads), 0, st, idx, static_cast<const uint16_t *>(weights), n_pairs, top_k,
                           num_experts, static_cast<tf_prefill_pair *>(sorted_pairs), static_cast<uint32_t *>(per_expert_offsets),
                           static_cast<uint32_t *>(per_expert_counts), static_cast<tf_prefill_group *>(chunks),
                           static_cast<uint32_t *>(chunk_count));
        return check_launch(ctx, "group_pairs_device");
    }
    hipLaunchKernelGGL(group_count_kernel, dim3(n_segments), dim3(64), 0, st, idx, n_pairs, seg_pairs, num_experts, ctx->group_scratch);
    hipLaunchKernelGGL(group_scan_kernel, dim3(1), dim3(256), 0, st, ctx->group_scratch, n_segments, num_experts,
                       static_cast<uint32_t *>(per_expert_offsets), static_cast<uint32_t *>(per_expert_counts),
                       static_cast<tf_prefill_group *>(chunks), static_cast<uint32_t *>(chunk_count));
    hipLaunchKernelGGL(group_place_kernel, dim3(n_segments), dim3(64), 0, st, idx, static_cast<const uint16_t *>(weights), n_pairs,
                       seg_pairs, top_k, num_experts, ctx->group_scratch, static_cast<tf_prefill_pair *>(sorted_pairs));
    return check_launch(ctx, "group_pairs_device");
}

int32_t tf_prefill_router_group_block(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                                      uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *hidden,
                                      uint64_t hidden_offset, const void *effective_scale, uint64_t effective_scale_offset,
                                      const void *per_expert_scale, uint64_t per_expert_scale_offset, void *out_indices,
                                      uint64_t out_indices_offset, void *out_weights, uint64_t out_weights_offset, uint32_t query_count,
                                      uint32_t num_experts, uint32_t d, uint32_t top_k, uint32_t hidden_stride_elements, void *sorted_pairs,
                                      void *per_expert_offsets, void *per_expert_counts, void *chunks, void *chunk_count) {
    // both calls' argument checks first, so that a refused call has launched nothing
    TF_REQUIRE(ctx, ctx && weights && scales && biases && hidden && effective_scale && per_expert_scale && out_indices && out_weights &&
                        sorted_pairs && per_expert_offsets && per_expert_counts && chunks && chunk_count,
               TF_ERR_INVALID_ARGUMENT, "prefill_router_group: null argument");
    TF_REQUIRE(ctx, query_count > 0 && num_experts > 0 && num_experts <= 256 && top_k > 0 && top_k <= 64 && d > 0 && d % TF_GROUP_SIZE == 0 &&
                        hidden_stride_elements >= d,
               TF_ERR_INVALID_ARGUMENT, "prefill_router_group: need queryCount > 0, 1 <= numExperts <= 256, 1 <= topK <= 64, D a multiple of 64, hidden stride >= D");
    const uint8_t *w = at(weights, weights_offset);
    const uint8_t *s = at(scales, scales_offset), *b = at(biases, biases_offset);
    const half_t *h = reinterpret_cast<const half_t *>(at(hidden, hidden_offset));
    const uint16_t *eff = reinterpret_cast<const uint16_t *>(at(effective_scale, effective_scale_offset));
    const uint16_t *pes = reinterpret_cast<const uint16_t *>(at(per_expert_scale, per_expert_scale_offset));
    uint32_t *oi = reinterpret_cast<uint32_t *>(at(out_indices, out_indices_offset));
    half_t *ow = reinterpret_cast<half_t *>(at(out_weights, out_weights_offset));
    TF_REQUIRE(ctx, aligned(s, 2) && aligned(b, 2) && aligned(h, 2) && aligned(eff, 2) && aligned(pes, 2) && aligned(oi, 4) && aligned(ow, 2) &&
                        aligned(sorted_pairs, 4) && aligned(chunks, 4) && aligned(per_expert_offsets, 4) && aligned(per_expert_counts, 4) &&
                        aligned(chunk_count, 4),
               TF_ERR_INVALID_ARGUMENT, "prefill_router_group: misaligned operand");
    const size_t need = std::max<size_t>((size_t)kFewTokens * 256, (size_t)query_count * num_experts);
    if (query_count <= kFewTokens && ctx->prefill_logits_count < need)
        return scratch_too_small(ctx, "prefill_router", need * sizeof(float), ctx->prefill_logits_count * sizeof(float));
    if (query_count <= kSelectGroupTokens && top_k <= kSelectGroupTopK) {
        const bool fast = aligned16(w) && aligned16(h) && aligned16(eff) && hidden_stride_elements % 8 == 0 && d <= 4096;
        hipStream_t st = static_cast<hipStream_t>(stream);
        launch_few_token_logits(st, w, s, b, h, hidden_stride_elements, eff, ctx->prefill_logits, query_count, num_experts, d, fast);
        const int32_t rc = check_launch(ctx, "prefill_router logits");
        if (rc != TF_OK) return rc;
        hipLaunchKernelGGL(select_group_small_kernel, dim3(1), dim3(1024), 0, st, ctx->prefill_logits, pes, oi, ow, query_count, num_experts, top_k,
                           static_cast<tf_prefill_pair *>(sorted_pairs), static_cast<uint32_t *>(per_expert_offsets),
                           static_cast<uint32_t *>(per_expert_counts), static_cast<tf_prefill_group *>(chunks), static_cast<uint32_t *>(chunk_count));
        return check_launch(ctx, "prefill_router select + group");
    }
    const int32_t rc = tf_prefill_router_gemma4_block(ctx, stream, weights, weights_offset, scales, scales_offset, biases, biases_offset, hidden,
                                                      hidden_offset, effective_scale, effective_scale_offset, per_expert_scale,
                                                      per_expert_scale_offset, out_indices, out_indices_offset, out_weights, out_weights_offset,
                                                      query_count, num_experts, d, top_k, hidden_stride_elements);
    if (rc != TF_OK) return rc;
    return tf_prefill_group_pairs_device(ctx, stream, oi, ow, query_count, top_k, num_experts, sorted_pairs, per_expert_offsets, per_expert_counts,
                                         chunks, chunk_count);
}

int32_t tf_prefill_grouped_routed_moe_streamed(tf_ctx *ctx, tf_stream stream, const void *hidden, uint64_t hidden_offset,
                                               const void *sorted_pairs, uint64_t sorted_pairs_offset, void *route_partials,
                                               uint64_t route_partials_offset, void *gate_up_act_scratch,
                                               uint64_t gate_up_act_scratch_offset, void *down_scratch, uint64_t down_scratch_offset,
                                               const void *const *blobs, const tf_prefill_streamed_params *params,
                                               const tf_prefill_group *tile_groups, uint32_t tile_group_count,
                                               int32_t pair_microbatch_rows, int32_t *out_microbatches, tf_dtype scale_dtype) {
    if (out_microbatches) *out_microbatches = 0;
    TF_REQUIRE(ctx, ctx && params, TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe: null argument");
    // encodeStreamedBatched's guard (PrefillGroupedRoutedMoE.swift:401-403): nothing to do, zero micro-batches
    if (params->pair_count == 0 || pair_microbatch_rows <= 0) return TF_OK;
    TF_REQUIRE(ctx, hidden && sorted_pairs && route_partials && gate_up_act_scratch && down_scratch && blobs && tile_groups,
               TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe: null argument");
    TF_REQUIRE(ctx, params->live_expert_count >= 1 && params->live_expert_count <= TF_MAX_TILE_EXPERTS, TF_ERR_INVALID_ARGUMENT,
               "invalid streamed tile binding: tile has %u live experts; expected 1...16", params->live_expert_count);
    TF_REQUIRE(ctx, params->d % TF_GROUP_SIZE == 0 && params->routed_intermediate % TF_GROUP_SIZE == 0 && params->d > 0 &&
                   params->routed_intermediate > 0 && params->top_k > 0 && params->hidden_stride_elements >= params->d,
               TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe: bad dimensions");
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe: scale dtype must be bf16 or fp16");
    ExpertTable tab = {};
    tab.live = params->live_expert_count;
    for (uint32_t i = 0; i < tab.live; ++i) {
        TF_REQUIRE(ctx, blobs[i] != nullptr, TF_ERR_INVALID_ARGUMENT, "invalid streamed tile binding: expert %u has no blob", i);
        tab.blob[i] = static_cast<const uint8_t *>(blobs[i]);
        tab.local_id[i] = params->local_expert[i];
    }
    const tf_expert_offsets off = {params->gate_W_off, params->gate_s_off, params->gate_b_off, params->up_W_off, params->up_s_off,
                                   params->up_b_off, params->down_W_off, params->down_s_off, params->down_b_off};
    const tf_prefill_pair *pairs = reinterpret_cast<const tf_prefill_pair *>(at(sorted_pairs, sorted_pairs_offset));
    const uint32_t f = params->routed_intermediate;
    // the activation plane is the third of the reference's [gate | up | act] scratch planes of `rows` pairs each
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t begin = params->pair_start, end = params->pair_start + params->pair_count;
    int32_t microbatches = 0;
    for (uint32_t mb_start = begin; mb_start < end; mb_start += (uint32_t)pair_microbatch_rows) {
        const uint32_t mb_end = std::min(end, mb_start + (uint32_t)pair_microbatch_rows);
        const uint32_t rows = mb_end - mb_start;
        half_t *acts = reinterpret_cast<half_t *>(at(gate_up_act_scratch, gate_up_act_scratch_offset)) + (size_t)2 * rows * f;
        // cut the micro-batch into runs of one expert (<= kChunkPairs pairs) using the host's group table
        std::vector<tf_prefill_group> runs;
        for (uint32_t gi = 0; gi < tile_group_count; ++gi) {
            const uint32_t gs = std::max(tile_groups[gi].pair_start, mb_start);
            const uint32_t ge = std::min(tile_groups[gi].pair_start + tile_groups[gi].pair_count, mb_end);
            for (uint32_t s0 = gs; s0 < ge; s0 += kChunkPairs) runs.push_back(tf_prefill_group{tile_groups[gi].expert, s0, std::min(kChunkPairs, ge - s0)});
        }
        for (size_t r0 = 0; r0 < runs.size(); r0 += kInlineChunks) {
            ChunkList cl = {};
            cl.n = (uint32_t)std::min<size_t>(kInlineChunks, runs.size() - r0);
            for (uint32_t i = 0; i < cl.n; ++i) cl.inline_chunks[i] = runs[r0 + i];
            GroupedGeom g{pairs, reinterpret_cast<const half_t *>(at(hidden, hidden_offset)), (long)params->hidden_stride_elements, acts,
                          mb_start, reinterpret_cast<half_t *>(at(route_partials, route_partials_offset)), (int)params->d, (int)f,
                          (int)params->top_k};
            const int32_t rc = run_grouped(ctx, st, tab, off, cl, cl.n, g, scale_dtype, false);
            if (rc != TF_OK) return rc;
        }
        ++microbatches;
    }
    (void)down_scratch;   // the down outputs go straight to route_partials; the reference's second copy is not needed
    if (out_microbatches) *out_microbatches = microbatches;
    return TF_OK;
}

}  // extern "C"

namespace {

int32_t grouped_resident_impl(tf_ctx *ctx, tf_stream stream, const void *hidden, uint64_t hidden_offset,
                              uint32_t hidden_stride_elements, const void *sorted_pairs, const void *chunks,
                              const void *chunk_count, uint32_t max_chunks, uint32_t pair_count,
                              const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                              const tf_expert_offsets *routed_offsets, void *acts_scratch, void *route_partials,
                              uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype, const DenseRide *ride, bool *ride_taken) {
    if (ride_taken) *ride_taken = false;
    TF_REQUIRE(ctx, ctx && hidden && sorted_pairs && chunks && chunk_count && expert_pool && routed_offsets && acts_scratch && route_partials,
               TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe_resident: null argument");
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0 && f > 0 && f % TF_GROUP_SIZE == 0 && top_k > 0 && num_experts > 0 &&
                   hidden_stride_elements >= d,
               TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe_resident: bad dimensions");
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "grouped_routed_moe_resident: scale dtype must be bf16 or fp16");
    if (pair_count == 0 || max_chunks == 0) return TF_OK;
    ExpertTable tab = {};
    tab.pool = static_cast<const uint8_t *>(expert_pool);
    tab.stride = expert_pool_stride;
    tab.num_experts = num_experts;
    ChunkList cl = {};
    cl.dev = static_cast<const tf_prefill_group *>(chunks);
    cl.dev_n = static_cast<const uint32_t *>(chunk_count);
    GroupedGeom g{static_cast<const tf_prefill_pair *>(sorted_pairs), reinterpret_cast<const half_t *>(at(hidden, hidden_offset)),
                  (long)hidden_stride_elements, static_cast<half_t *>(acts_scratch), 0u, static_cast<half_t *>(route_partials), (int)d,
                  (int)f, (int)top_k};
    // the host only knows the average group size: the matrix cores pay once experts see 2 or more tokens on average (with
    // fewer, up to kStreamTokens tokens, the row-streaming kernels read every touched expert once at a higher rate)
    const bool use_mfma = (uint64_t)pair_count >= (uint64_t)num_experts * 2;
    // the pairs are all (token, rank) combinations of pair_count / top_k token rows
    const uint32_t tokens = pair_count % top_k == 0 ? pair_count / top_k : 0u;
    return run_grouped(ctx, static_cast<hipStream_t>(stream), tab, *routed_offsets, cl, max_chunks, g, scale_dtype, use_mfma, tokens, pair_count,
                       ride, ride_taken);
}

}  // namespace

extern "C" {

int32_t tf_prefill_grouped_routed_moe_resident(tf_ctx *ctx, tf_stream stream, const void *hidden, uint64_t hidden_offset,
                                               uint32_t hidden_stride_elements, const void *sorted_pairs, const void *chunks,
                                               const void *chunk_count, uint32_t max_chunks, uint32_t pair_count,
                                               const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                               const tf_expert_offsets *routed_offsets, void *acts_scratch, void *route_partials,
                                               uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    return grouped_resident_impl(ctx, stream, hidden, hidden_offset, hidden_stride_elements, sorted_pairs, chunks, chunk_count, max_chunks,
                                 pair_count, expert_pool, expert_pool_stride, num_experts, routed_offsets, acts_scratch, route_partials, d, f,
                                 top_k, scale_dtype, nullptr, nullptr);
}

int32_t tf_prefill_grouped_routed_moe_resident_shared(tf_ctx *ctx, tf_stream stream, const void *hidden, uint64_t hidden_offset,
                                                      uint32_t hidden_stride_elements, const void *sorted_pairs, const void *chunks,
                                                      const void *chunk_count, uint32_t max_chunks, uint32_t pair_count,
                                                      const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                                      const tf_expert_offsets *routed_offsets, void *acts_scratch, void *route_partials,
                                                      uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype, const void *shared_x,
                                                      uint64_t shared_x_offset, void *shared_y, uint64_t shared_y_offset,
                                                      const tf_projection *shared_gate, const tf_projection *shared_up,
                                                      const tf_projection *shared_down, void *scratch_gate, uint64_t scratch_gate_offset,
                                                      uint64_t scratch_gate_length, void *scratch_up, uint64_t scratch_up_offset,
                                                      uint64_t scratch_up_length, void *scratch_act, uint64_t scratch_act_offset,
                                                      uint64_t scratch_act_length, uint32_t query_count, uint32_t shared_intermediate,
                                                      uint32_t shared_x_stride_elements, uint32_t shared_y_stride_elements,
                                                      uint32_t shared_weight_bits) {
    // both calls' argument checks first, so that a refused call has launched nothing
    DenseRide ride = {};
    int32_t rc = shared_expert_block_plan(ctx, shared_x, shared_x_offset, shared_y, shared_y_offset, shared_gate, shared_up, shared_down,
                                          scratch_gate, scratch_gate_offset, scratch_gate_length, scratch_up, scratch_up_offset, scratch_up_length,
                                          scratch_act, scratch_act_offset, scratch_act_length, query_count, d, shared_intermediate,
                                          shared_x_stride_elements, shared_y_stride_elements, shared_weight_bits, scale_dtype, &ride);
    if (rc != TF_OK) return rc;
    bool taken = false;
    rc = grouped_resident_impl(ctx, stream, hidden, hidden_offset, hidden_stride_elements, sorted_pairs, chunks, chunk_count, max_chunks,
                               pair_count, expert_pool, expert_pool_stride, num_experts, routed_offsets, acts_scratch, route_partials, d, f,
                               top_k, scale_dtype, ride.rows > 0 ? &ride : nullptr, &taken);
    if (rc != TF_OK || taken) return rc;
    return tf_prefill_shared_expert_int4_block(ctx, stream, shared_x, shared_x_offset, shared_y, shared_y_offset, shared_gate, shared_up,
                                               shared_down, scratch_gate, scratch_gate_offset, scratch_gate_length, scratch_up, scratch_up_offset,
                                               scratch_up_length, scratch_act, scratch_act_offset, scratch_act_length, query_count, d,
                                               shared_intermediate, shared_x_stride_elements, shared_y_stride_elements, shared_weight_bits,
                                               scale_dtype);
}

int32_t tf_prefill_moe_reduce_token_major(tf_ctx *ctx, tf_stream stream, const void *route_partials, uint64_t route_partials_offset,
                                          const void *route_weights, uint64_t route_weights_offset, void *h2, uint64_t h2_offset,
                                          uint32_t query_count, uint32_t top_k, uint32_t d) {
    TF_REQUIRE(ctx, ctx && route_partials && route_weights && h2, TF_ERR_INVALID_ARGUMENT, "moe_reduce_token_major: null argument");
    TF_REQUIRE(ctx, query_count > 0, TF_ERR_INVALID_ARGUMENT, "moe_reduce_token_major: queryCount must be positive");
    TF_REQUIRE(ctx, top_k > 0, TF_ERR_INVALID_ARGUMENT, "moe_reduce_token_major: topK must be positive");
    TF_REQUIRE(ctx, d > 0, TF_ERR_INVALID_ARGUMENT, "moe_reduce_token_major: D must be positive");
    TF_REQUIRE(ctx, route_partials_offset % 2 == 0 && route_weights_offset % 2 == 0 && h2_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT,
               "moe_reduce_token_major: offsets must be 2-byte aligned");
    const half_t *partials_at = reinterpret_cast<const half_t *>(at(route_partials, route_partials_offset));
    const half_t *weights_at = reinterpret_cast<const half_t *>(at(route_weights, route_weights_offset));
    half_t *h2_at = reinterpret_cast<half_t *>(at(h2, h2_offset));
    if (d % 8 == 0 && aligned16(partials_at) && aligned16(h2_at)) {
        const uint64_t pieces = (uint64_t)query_count * (d / 8);
        TF_REQUIRE(ctx, pieces <= 0xFFFFFFFFull - 255, TF_ERR_INVALID_ARGUMENT, "moe_reduce_token_major: queryCount * D / 8 must fit 32 bits");
        const dim3 grid((uint32_t)((pieces + 255) / 256));
        hipLaunchKernelGGL(reduce_token_major_vec_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), partials_at, weights_at,
                           h2_at, query_count, top_k, d);
    } else {
        const dim3 grid((d + 255) / 256, query_count);
        hipLaunchKernelGGL(reduce_token_major_kernel, grid, dim3(256), 0, static_cast<hipStream_t>(stream), partials_at, weights_at,
                           h2_at, query_count, top_k, d);
    }
    return check_launch(ctx, "moe_reduce_token_major");
}

int32_t tf_prefill_int4_qmm(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                            uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *x, uint64_t x_offset,
                            void *y, uint64_t y_offset, int32_t t, int32_t n, int32_t k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "prefill_int4_qmm: null context");
    TF_REQUIRE(ctx, t > 0 && n > 0, TF_ERR_INVALID_ARGUMENT, "prefill_int4_qmm: t and n must be positive");
    TF_REQUIRE(ctx, k > 0 && k % (int32_t)TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "prefill_int4_qmm: K must be a multiple of 64");
    // every token row takes the GEMV path: Y[t, :] = gemv(W, X[t, :]); identical arithmetic, hence QMM == repeated GEMV
    for (int32_t row = 0; row < t; ++row) {
        const int32_t rc = tf_dequant_int4_gemv(ctx, stream, weights, weights_offset, scales, scales_offset, biases, biases_offset, x,
                                                x_offset + (uint64_t)row * k * 2, y, y_offset + (uint64_t)row * n * 2, (uint32_t)n,
                                                (uint32_t)k, scale_dtype, TF_FP16);
        if (rc != TF_OK) return rc;
    }
    return TF_OK;
}

}  // extern "C"

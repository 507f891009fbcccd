// A few token rows (multi-token verification) through the router and the routed experts in THREE launches: router logits;
// gate / up / GeGLU with the selection repeated inside every block; down projection with the token-major reduce inside the
// block.  The grouped path spends five launches on the same work (logits, selection + grouping, gate / up, down, reduce), and at
// two to four tokens the launches' boundaries and their first memory round trips are most of the call: 21.3 / 28.1 / 35.0 us for
// 2 / 3 / 4 tokens of the production shape against 30.8 / 35.2 / 40.1 us.  From six tokens on the grouped path's persistent
// kernels win (every block here pays for its own selection, and the arithmetic per pair is the same), so the entry point at the
// end of this file gives batches of more than five rows to the grouped calls and the kernels here hold at most eight rows.
//
// Experts are still read once however many tokens chose them:
//   * gate / up: the grid has one set of blocks per (token, rank) pair.  Every block ranks its own token's logits (by counting, as
//     the decode step does), looks up the pair's expert e and then asks, for every other token, whether e is among that token's
//     eight: e's place in a token's order is the number of logits that beat it, two compares and two ballots per token.  The pair
//     with the lowest token number owns the expert: its blocks stream e's rows once and apply them to every token that chose
//     it; the other pairs' blocks leave before they request a weight.
//   * down: one block per run of output rows takes those rows of EVERY expert in use (its sixteen waves share the distinct
//     experts out, a round ahead in flight), applies them to the pairs that chose the expert, and — holding all eight partial
//     results of every token for its rows — adds them up in rank order itself.
// Arithmetic is the grouped path's: fp16 activations half(gelu(gate) * up), fp16 partials, h2 = half(sum_r fma(w_r, partial_r)).
#include "tf_gemv_kernels.hpp"
#include "tf_router.hpp"

using namespace tfk;

namespace {

constexpr uint32_t kFewMaxTokens = 8;       // the kernels' capacity: 64 pairs (one lane each of a wave), 4 KiB of logits in LDS
constexpr uint32_t kFewEntryMaxTokens = 32; // what the entry point takes (beyond kFewCrossoverTokens through the grouped calls)
constexpr uint32_t kFewMaxExperts = 128;
constexpr uint32_t kFewTopK = 8;
constexpr uint32_t kNoSlot = 0xFFu;
constexpr uint32_t kFewCrossoverTokens = 5;      // up to here the three launches of this file, beyond the grouped path's five
static_assert(kFewCrossoverTokens <= kFewMaxTokens, "the kernels hold every batch they are given");

// ------------------------------------------------------------------------------------------------ router logits
// One 256-thread block per (expert, token): a row is one memory round trip and a sixteenth of a wave's arithmetic.
template <int SD>
__global__ __launch_bounds__(256) void few_logits_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B, const half_t *hidden,
                                                         uint32_t hidden_stride, const uint16_t *eff, float *logits, uint32_t num_experts, int d) {
    __shared__ float partial[4];
    const uint32_t e = blockIdx.x, t = blockIdx.y;
    const int groups = d >> 6;
    const float v = router_row_block<SD>(W + (size_t)e * d, S + (size_t)e * groups * 2, B + (size_t)e * groups * 2,
                                         hidden + (size_t)t * hidden_stride, eff, d, partial);
    if (threadIdx.x == 0) logits[(size_t)t * num_experts + e] = v;
}

// ------------------------------------------------------------------------------------------------ gate / up / GeGLU
__device__ __forceinline__ void few_store_act(half_t *acts, size_t index, float gate, float up) {
    acts[index] = (half_t)(gelu_tanh(gate) * up);
}

// Grid: (row tiles / 4, tokens * 8).  Dynamic LDS: the token's activations in dot-product order (d / 8 16-byte words), their
// column sums (d / 32 floats, padded to 16 bytes), then every token's logits (tokens * num_experts floats, NaN stored as -inf).
__host__ __device__ constexpr uint32_t few_image_bytes(uint32_t d) { return (d >> 3) * 16u + (((d >> 5) + 3u) & ~3u) * 4u; }

template <int RT, int NP, int SD>
__global__ __launch_bounds__(256, NP <= 3 ? 4 : 3) void few_phase1_kernel(const float *logits, const uint16_t *per_expert_scale, const uint8_t *pool,
                                                                          uint64_t stride, const half_t *hidden, uint32_t hidden_stride, half_t *acts,
                                                                          uint32_t *out_indices, half_t *out_weights, uint32_t tokens,
                                                                          uint32_t num_experts, uint32_t d, uint32_t f, tf_expert_offsets off) {
    extern __shared__ __align__(16) uint8_t few_lds[];
    u32x4 *xa = reinterpret_cast<u32x4 *>(few_lds);
    float *xsum = reinterpret_cast<float *>(few_lds + (size_t)(d >> 3) * 16);
    float *all_logits = reinterpret_cast<float *>(few_lds + few_image_bytes(d));
    __shared__ uint32_t chosen[kFewTopK];
    __shared__ RankSelectLds sel;
    __shared__ uint32_t member[kFewMaxTokens];    // the rank at which token u chose this block's expert, kNoSlot if it did not
    __shared__ uint32_t no_share;

    const int lane = threadIdx.x & 63;
    const uint32_t wave = uniform_u32(threadIdx.x >> 6);
    const uint32_t pair = blockIdx.y, t = pair / kFewTopK, s = pair % kFewTopK;
    const float *my_row = logits + (size_t)t * num_experts;
    // requests first: the token's logits for the ranking, every token's logits, the token's activations
    const float my_logit = rank_select_load(my_row, num_experts);
    const uint32_t n4 = tokens * num_experts / 4;
    f32x4 lg = {-INFINITY, -INFINITY, -INFINITY, -INFINITY};      // at most 8 x 128 logits: one 16-byte piece a thread
    if (threadIdx.x < n4) lg = reinterpret_cast<const f32x4 *>(logits)[threadIdx.x];
    XStage stage;
    stage.request(hidden + (size_t)t * hidden_stride, (int)d);
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile tg, tu;
    rs.init_map((int)d, lane);
    if (threadIdx.x == 0) no_share = 0u;
    const bool ranked = rank_select_block(my_logit, num_experts, sel, chosen);
    const bool publisher = blockIdx.x == 0 && s == 0;      // one block per token writes the router's outputs
    if (!ranked && wave == 0) {
        uint32_t idx;
        half_t weight;
        router_select_lanes(my_row, per_expert_scale, num_experts, kFewTopK, lane, idx, weight);
        if ((uint32_t)lane < kFewTopK) {
            chosen[lane] = idx < num_experts ? idx : num_experts - 1;
            if (publisher) {
                out_indices[t * kFewTopK + lane] = idx;
                out_weights[t * kFewTopK + lane] = weight;
            }
        }
    }
    if (threadIdx.x < n4) {
#pragma unroll
        for (int c = 0; c < 4; ++c) lg[c] = (lg[c] != lg[c]) ? -INFINITY : lg[c];
        reinterpret_cast<f32x4 *>(all_logits)[threadIdx.x] = lg;
    }
    stage.publish((int)d, xa, xsum);            // ends with a block barrier: chosen and all_logits are visible after it
    const uint32_t e = uniform_u32(chosen[s]);
    // Who else chose e, and at which rank: e's place in token u's order (score descending, ties to the lower index) is the number
    // of u's logits that beat it.  A token with fewer than eight finite logits fills its last ranks with expert 0 whatever its
    // score (the selection's rule for unfilled places), which this count does not see: then no block shares anything.
    for (uint32_t u = wave; u < tokens; u += 4) {
        const float *row = all_logits + u * num_experts;
        const float ve = row[e];
        const uint32_t j0 = (uint32_t)lane, j1 = (uint32_t)lane + 64u;
        const float c0 = j0 < num_experts ? row[j0] : -INFINITY;
        const float c1 = j1 < num_experts ? row[j1] : -INFINITY;
        const bool b0 = c0 > ve || (c0 == ve && j0 < e);
        const bool b1 = c1 > ve || (c1 == ve && j1 < e);
        const uint32_t rank = (uint32_t)(__builtin_popcountll(__ballot(b0)) + __builtin_popcountll(__ballot(b1)));
        const uint32_t finite = (uint32_t)(__builtin_popcountll(__ballot(c0 > -INFINITY)) + __builtin_popcountll(__ballot(c1 > -INFINITY)));
        if (lane == 0) {
            member[u] = (ve > -INFINITY && rank < kFewTopK) ? rank : kNoSlot;
            if (finite < kFewTopK) no_share = 1u;
        }
    }
    __syncthreads();
    if (ranked && publisher && wave == 0) {
        uint32_t idx;
        half_t weight;
        rank_select_weights(sel, chosen, per_expert_scale, lane, idx, weight);
        if ((uint32_t)lane < kFewTopK) {
            out_indices[t * kFewTopK + lane] = idx;
            out_weights[t * kFewTopK + lane] = weight;
        }
    }
    const bool share = uniform_u32(no_share) == 0u;
    if (share) {
        for (uint32_t u = 0; u < t; ++u)
            if (uniform_u32(member[u]) != kNoSlot) return;      // an earlier token's pair owns the expert
    }
    const uint32_t tile = blockIdx.x * 4u + wave;
    const uint32_t row0 = tile * RT;
    const bool live = row0 < f;           // a wave of the last block may have no rows: it still helps to stage activations
    if (live) {
        const uint8_t *base = pool + (uint64_t)e * stride;
        const size_t w_byte = (size_t)row0 * (d >> 1), sb_byte = (size_t)row0 * (d >> 6) * 2;
        rs.load(tg, base + off.gate_W_off + w_byte, base + off.gate_s_off + sb_byte, base + off.gate_b_off + sb_byte, f - row0);
        rs.load(tu, base + off.up_W_off + w_byte, base + off.up_s_off + sb_byte, base + off.up_b_off + sb_byte, f - row0);
    }
    uint32_t u = t, slot = s;
    while (true) {
        // the next token that chose the expert
        uint32_t un = u + 1;
        if (share) {
            while (un < tokens && uniform_u32(member[un]) == kNoSlot) ++un;
        } else {
            un = tokens;
        }
        if (live) {
            rs.init_x_lds(xa, xsum, (int)d);
            // the tiles are the same for every token, and the compiler would keep their isolated nibbles (96 registers) across the
            // loop for the rare second token: an empty statement that "rewrites" them keeps that work inside the iteration
#pragma unroll
            for (int p = 0; p < NP; ++p) asm volatile("" : "+v"(tg.w[p]), "+v"(tu.w[p]));
            float gate[RT], up[RT];
            rs.template reduce<SD>(tg, gate);
            rs.template reduce<SD>(tu, up);
            if (lane == 0) {
#pragma unroll
                for (int r = 0; r < RT; ++r)
                    if (row0 + r < f) few_store_act(acts, (size_t)(u * kFewTopK + slot) * f + row0 + r, gate[r], up[r]);
            }
        }
        if (un >= tokens) break;
        stage.request(hidden + (size_t)un * hidden_stride, (int)d);
        u = un;
        slot = uniform_u32(member[u]);
        __syncthreads();                           // every wave has taken the staged activations
        stage.publish((int)d, xa, xsum);           // ends with a block barrier
    }
}

// ------------------------------------------------------------------------------------------------ down + reduce
constexpr int kFewDownWaves = 16;      // 122 registers a lane at four passes: sixteen waves still fit one block on a CU
constexpr uint32_t kFewDownMaxRows = 16;

template <int NP>
struct FewRound {
    u32x4 w[NP];
    uint16_t sv[NP], bv[NP];
};

// Grid: d / rpb blocks of sixteen waves.  A block takes rows [row0, row0 + rpb) of the down matrix of every expert in use: the
// rows of one expert are rpb * f / 2 contiguous bytes, read as one flat stream of 16-byte chunks (pass p, lane l: chunk 64 p + l;
// the chunk lies in row c / nch, column c % nch), the pair's activations staged per wave in LDS in dot-product order, row sums
// taken from a prefix sum across the wave — the decode step's down kernel, once per (expert, pair) instead of once per rank.
// A wave keeps two experts in flight: the next one's rows are requested before this one's are used (loads return in order, so
// what was asked for first can be waited for alone).  The kernel is bound by its arithmetic from about eight tokens on (every
// pair costs the wave some two hundred vector instructions on the block's rows), not by these requests: a third expert in flight
// and the pairs' activations requested a round ahead measured slower at every size.
template <int NP, int SD>
__global__ __launch_bounds__(64 * kFewDownWaves) void few_down_kernel(const uint32_t *indices, const half_t *routing_w, const uint8_t *pool, uint64_t stride,
                                                        const half_t *acts, half_t *route_partials, half_t *h2, uint32_t tokens, uint32_t d,
                                                        uint32_t f, uint32_t rpb, uint32_t inv_nch, uint32_t num_experts, tf_expert_offsets off) {
    __shared__ __align__(16) u32x4 xa[kFewDownWaves][128];
    __shared__ float xsum[kFewDownWaves][32];
    __shared__ float running[kFewDownWaves][NP * 64];
    __shared__ half_t part[kFewMaxTokens * kFewTopK][kFewDownMaxRows];    // the partial results of the block's rows
    __shared__ uint32_t s_idx[kFewMaxTokens * kFewTopK];
    __shared__ half_t s_w[kFewMaxTokens * kFewTopK];
    __shared__ uint32_t first[kFewMaxExperts], uniq[kFewMaxTokens * kFewTopK], n_uniq_lds;

    const int lane = threadIdx.x & 63;
    const uint32_t wave = uniform_u32(threadIdx.x >> 6);
    const uint32_t pairs = tokens * kFewTopK;
    const uint32_t row0 = blockIdx.x * rpb;
    const uint32_t rows_here = min(rpb, d - row0);
    const int nch = (int)(f >> 5), groups = (int)(f >> 6), pieces = (int)(f >> 3);

    // the distinct experts of the call, in order of their first pair
    uint32_t my_e = 0;
    if (threadIdx.x < pairs) {
        const uint32_t e = indices[threadIdx.x];
        my_e = e < num_experts ? e : num_experts - 1;
        s_idx[threadIdx.x] = my_e;
        s_w[threadIdx.x] = routing_w[threadIdx.x];
    }
    if (threadIdx.x < kFewMaxExperts) first[threadIdx.x] = 0xFFFFFFFFu;
    __syncthreads();
    if (threadIdx.x < pairs) atomicMin(&first[my_e], threadIdx.x);
    __syncthreads();
    if (wave == 0) {      // the pairs are the first wave's lanes
        const bool leads = (uint32_t)lane < pairs && first[my_e] == (uint32_t)lane;
        const uint64_t lead_mask = __ballot(leads);
        if (leads) uniq[__builtin_popcountll(lead_mask & ((1ull << lane) - 1ull))] = (uint32_t)lane;
        if (lane == 0) n_uniq_lds = (uint32_t)__builtin_popcountll(lead_mask);
    }
    __syncthreads();
    const uint32_t n_uniq = n_uniq_lds;

    // this lane's chunk positions: the same for every expert
    uint32_t sboff[NP];
    int col[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const uint32_t c = 64u * p + (uint32_t)lane;
        const uint32_t r = (c * inv_nch) >> 16;            // c / nch (the host checked the reciprocal for every c < 64 NP)
        const uint32_t cc = c - r * (uint32_t)nch;
        col[p] = (int)cc;
        sboff[p] = (r * (uint32_t)groups + (cc >> 1)) * 2u;   // past the block's rows: past the descriptor, reads zero
    }
    // the pairs that chose expert e, as a 64-bit mask over the pair numbers
    struct Pairs {
        uint64_t m;
        __device__ __forceinline__ bool any() const { return m != 0ull; }
        __device__ __forceinline__ uint32_t pop() {      // the lowest pair, removed; call only if any()
            const uint32_t q = (uint32_t)__builtin_ctzll(m);
            m &= m - 1ull;
            return q;
        }
    };
    auto pairs_of = [&](uint32_t e) {
        Pairs ps;
        ps.m = __ballot((uint32_t)lane < pairs && s_idx[(uint32_t)lane < pairs ? lane : 0] == e);
        return ps;
    };
    auto request_acts = [&](u32x4 (&xr)[2], uint32_t q) {
        const rsrc_t ra = make_rsrc(acts + (size_t)q * f, f * 2u);
        xr[0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, (uint32_t)lane * 16u, 0, 0));
        xr[1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, (uint32_t)(lane + 64) * 16u, 0, 0));
    };
    auto issue = [&](FewRound<NP> &r, uint32_t k) {
        const uint32_t e = uniform_u32(s_idx[uniform_u32(uniq[k])]);
        const uint8_t *base = pool + (uint64_t)e * stride;
        const rsrc_t rw = make_rsrc(base + off.down_W_off + (size_t)row0 * (f >> 1), rows_here * (f >> 1));
        const rsrc_t rsc = make_rsrc(base + off.down_s_off + (size_t)row0 * groups * 2, rows_here * (uint32_t)groups * 2u);
        const rsrc_t rbi = make_rsrc(base + off.down_b_off + (size_t)row0 * groups * 2, rows_here * (uint32_t)groups * 2u);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            r.w[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, (64u * p + (uint32_t)lane) * 16u, 0, kStreamOnce));
            r.sv[p] = __builtin_amdgcn_raw_buffer_load_b16(rsc, sboff[p], 0, 0);
            r.bv[p] = __builtin_amdgcn_raw_buffer_load_b16(rbi, sboff[p], 0, 0);
        }
    };
    // one pair: its activations into the wave's LDS image, the block's rows of the expert against them, the partial results out
    auto apply = [&](FewRound<NP> &r, const u32x4 (&xr)[2], uint32_t q) {
        // the rows are the same for every pair of the expert, and the compiler would keep their isolated nibbles (two registers for
        // each one of the rows') across the pairs: an empty statement that "rewrites" the rows keeps that work with each pair
#pragma unroll
        for (int p = 0; p < NP; ++p) asm volatile("" : "+v"(r.w[p]));
        XStage::publish_piece(xr[0], lane, pieces, nch, xa[wave], xsum[wave]);
        XStage::publish_piece(xr[1], lane + 64, pieces, nch, xa[wave], xsum[wave]);
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            half2_t xq[16];
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const u32x4 v = xa[wave][dd * nch + col[p]];
#pragma unroll
                for (int j = 0; j < 4; ++j) xq[4 * dd + j] = as_half2(v[j]);
            }
            float v = fmaf(sb_to_f32<SD>(r.sv[p]), chunk_dot(r.w[p], xq), sb_to_f32<SD>(r.bv[p]) * xsum[wave][col[p]]);
            v += dpp_f32<0x111>(v);          // inclusive prefix sum across the wave
            v += dpp_f32<0x112>(v);
            v += dpp_f32<0x114>(v);
            v += dpp_f32<0x118>(v);
            v += dpp_f32<0x142, 0xA>(v);
            v += dpp_f32<0x143, 0xC>(v);
            running[wave][64 * p + lane] = v;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        if ((uint32_t)lane < rows_here) {
            const uint32_t c_first = (uint32_t)lane * (uint32_t)nch, c_last = c_first + (uint32_t)nch - 1u;
            const float *run = running[wave];
            float sum = run[c_last];
            if ((c_first >> 6) != (c_last >> 6)) sum += run[(c_first | 63u)];      // the row started in the pass before
            if (c_first & 63u) sum -= run[c_first - 1u];
            const half_t h = (half_t)sum;
            route_partials[(size_t)q * d + row0 + lane] = h;
            part[q][lane] = h;
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");     // the image and the sums are read before the next pair replaces them
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
    // xr: the activations of the expert's first pair, requested by the caller ahead of the next round's rows
    auto process = [&](FewRound<NP> &r, u32x4 (&xr)[2], uint32_t k) {
        const uint32_t q0 = uniform_u32(uniq[k]);
        Pairs ps = pairs_of(uniform_u32(s_idx[q0]));
        uint32_t q = ps.pop();      // q0: the expert's first pair is its lowest
        while (true) {
            apply(r, xr, q);
            if (!ps.any()) break;
            q = ps.pop();
            request_acts(xr, q);
        }
    };

    FewRound<NP> ra = {}, rb = {};
    u32x4 xr[2];
    uint32_t k = wave;
    if (k < n_uniq) issue(ra, k);
    while (k < n_uniq) {      // the two buffers take turns
        request_acts(xr, uniform_u32(uniq[k]));
        if (k + kFewDownWaves < n_uniq) issue(rb, k + kFewDownWaves);
        process(ra, xr, k);
        k += kFewDownWaves;
        if (k >= n_uniq) break;
        request_acts(xr, uniform_u32(uniq[k]));
        if (k + kFewDownWaves < n_uniq) issue(ra, k + kFewDownWaves);
        process(rb, xr, k);
        k += kFewDownWaves;
    }
    __syncthreads();
    // h2[u, row] = half(sum_r fma(w[u, r], partial[u, r, row])), ranks ascending
    for (uint32_t i = threadIdx.x; i < tokens * rows_here; i += blockDim.x) {
        const uint32_t u = i / rows_here, r = i - u * rows_here;
        float acc = 0.0f;
#pragma unroll
        for (uint32_t j = 0; j < kFewTopK; ++j) acc = fmaf((float)s_w[u * kFewTopK + j], (float)part[u * kFewTopK + j][r], acc);
        asm volatile("" : "+v"(acc));      // the sum is rounded to fp32 and then to fp16, like the reduce kernel's: no fused fp16-result multiply-add
        h2[(size_t)u * d + row0 + r] = (half_t)acc;
    }
}

bool offsets_fit(const tf_expert_offsets &o) {
    return o.gate_W_off % 16 == 0 && o.up_W_off % 16 == 0 && o.down_W_off % 16 == 0 && o.gate_s_off % 2 == 0 && o.gate_b_off % 2 == 0 &&
           o.up_s_off % 2 == 0 && o.up_b_off % 2 == 0 && o.down_s_off % 2 == 0 && o.down_b_off % 2 == 0;
}

}  // namespace

extern "C" int32_t tf_prefill_routed_moe_few_tokens(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset,
                                                    const void *scales, uint64_t scales_offset, const void *biases, uint64_t biases_offset,
                                                    const void *hidden, uint64_t hidden_offset, const void *effective_scale,
                                                    uint64_t effective_scale_offset, const void *per_expert_scale,
                                                    uint64_t per_expert_scale_offset, void *out_indices, uint64_t out_indices_offset,
                                                    void *out_weights, uint64_t out_weights_offset, uint32_t query_count, uint32_t num_experts,
                                                    uint32_t d, uint32_t top_k, uint32_t hidden_stride_elements, const void *routed_hidden,
                                                    uint64_t routed_hidden_offset, uint32_t routed_hidden_stride_elements, const void *expert_pool,
                                                    uint64_t expert_pool_stride, const tf_expert_offsets *routed_offsets, void *acts_scratch,
                                                    void *route_partials, void *h2, uint64_t h2_offset, uint32_t f, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx && weights && scales && biases && hidden && effective_scale && per_expert_scale && out_indices && out_weights &&
                        routed_hidden && expert_pool && routed_offsets && acts_scratch && route_partials && h2,
               TF_ERR_INVALID_ARGUMENT, "prefill_routed_moe_few_tokens: null argument");
    TF_REQUIRE(ctx, query_count > 0 && num_experts > 0 && num_experts <= 256 && top_k > 0 && top_k <= 64 && d > 0 && d % TF_GROUP_SIZE == 0 &&
                        hidden_stride_elements >= d && routed_hidden_stride_elements >= d && f > 0 && f % TF_GROUP_SIZE == 0,
               TF_ERR_INVALID_ARGUMENT,
               "prefill_routed_moe_few_tokens: need queryCount > 0, 1 <= numExperts <= 256, 1 <= topK <= 64, D and F multiples of 64, hidden strides >= D");
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "prefill_routed_moe_few_tokens: scale dtype must be bf16 or fp16");
    const uint8_t *w = at(weights, weights_offset);
    const uint8_t *s = at(scales, scales_offset), *b = at(biases, biases_offset);
    const half_t *h = reinterpret_cast<const half_t *>(at(hidden, hidden_offset));
    const half_t *x = reinterpret_cast<const half_t *>(at(routed_hidden, routed_hidden_offset));
    const uint16_t *eff = reinterpret_cast<const uint16_t *>(at(effective_scale, effective_scale_offset));
    const uint16_t *pes = reinterpret_cast<const uint16_t *>(at(per_expert_scale, per_expert_scale_offset));
    uint32_t *oi = reinterpret_cast<uint32_t *>(at(out_indices, out_indices_offset));
    half_t *ow = reinterpret_cast<half_t *>(at(out_weights, out_weights_offset));
    half_t *out = reinterpret_cast<half_t *>(at(h2, h2_offset));
    const uint8_t *pool = static_cast<const uint8_t *>(expert_pool);
    TF_REQUIRE(ctx, aligned(s, 2) && aligned(b, 2) && aligned(h, 2) && aligned(x, 2) && aligned(eff, 2) && aligned(pes, 2) && aligned(oi, 4) && aligned(ow, 2) &&
                        aligned(out, 2) && aligned(route_partials, 2) && aligned(acts_scratch, 2),
               TF_ERR_INVALID_ARGUMENT, "prefill_routed_moe_few_tokens: misaligned operand");
    // what the three kernels assume; anything else is the grouped path's (four calls)
    const LongPlan plan = plan_long_rows((int)d);
    const uint32_t nch = f / 32;
    const bool plan_ok = (plan.rt == 1 && (plan.np == 1 || plan.np == 2)) || (plan.rt == 2 && plan.np >= 2 && plan.np <= 4) ||
                         (plan.rt == 4 && (plan.np == 3 || plan.np == 4));
    bool ok = plan_ok && query_count <= kFewCrossoverTokens && top_k == kFewTopK && num_experts <= kFewMaxExperts && num_experts % 4 == 0 && d > 1024 && d <= 4096 &&
              plan.rt > 0 && f <= 1024 && aligned16(w) && aligned16(h) && aligned16(eff) && hidden_stride_elements % 8 == 0 && aligned16(x) &&
              routed_hidden_stride_elements % 8 == 0 && aligned16(pool) &&
              expert_pool_stride % 16 == 0 && offsets_fit(*routed_offsets) && aligned16(acts_scratch) &&
              ctx->prefill_logits_count >= (size_t)query_count * num_experts;
    int best_np = 0;
    uint32_t best_rpb = 0, inv_nch = 0;
    if (ok) {
        // rows per block and passes of the down kernel: fewest passes on the busiest CU, then fullest lanes
        double best_cost = 0.0;
        for (int np = 1; np <= 4; ++np) {
            const uint32_t rpb = std::min<uint32_t>((uint32_t)(64 * np) / nch, kFewDownMaxRows);
            if (rpb == 0) continue;
            const uint32_t blocks = (d + rpb - 1) / rpb;
            const uint32_t rounds = (blocks + (uint32_t)ctx->num_cus - 1) / (uint32_t)std::max(ctx->num_cus, 1);
            const double cost = (double)rounds * np + 1e-3 * (1.0 - (double)(rpb * nch) / (64.0 * np));
            if (best_np == 0 || cost < best_cost) {
                best_np = np;
                best_rpb = rpb;
                best_cost = cost;
            }
        }
        inv_nch = (65536u + nch - 1) / nch;
        ok = best_np > 0;
        for (uint32_t c = 0; ok && c < 64u * (uint32_t)best_np; ++c) ok = ((c * inv_nch) >> 16) == c / nch;
    }
    // From six token rows on the grouped path's persistent kernels are faster (every block here pays for its own selection): the
    // call then makes the three calls it stands for itself, with the grouping's outputs in the context's scratch.
    if (!ok) {
        if (query_count > kFewEntryMaxTokens || top_k != kFewTopK || query_count * top_k > kFewScratchPairs ||
            num_experts + query_count * top_k / 64 + 1 > kFewScratchChunks)
            return TF_ERR_UNAVAILABLE;
        uint8_t *scratch = ctx->few_scratch;
        void *sorted_pairs = scratch, *offsets = scratch + (size_t)kFewScratchPairs * 16, *counts = scratch + (size_t)kFewScratchPairs * 16 + 1024;
        void *chunks = scratch + (size_t)kFewScratchPairs * 16 + 2048, *chunk_count = scratch + (size_t)kFewScratchPairs * 16 + 2048 + (size_t)kFewScratchChunks * 12;
        int32_t rc = tf_prefill_router_group_block(ctx, stream, weights, weights_offset, scales, scales_offset, biases, biases_offset, hidden, hidden_offset,
                                                   effective_scale, effective_scale_offset, per_expert_scale, per_expert_scale_offset, out_indices,
                                                   out_indices_offset, out_weights, out_weights_offset, query_count, num_experts, d, top_k,
                                                   hidden_stride_elements, sorted_pairs, offsets, counts, chunks, chunk_count);
        if (rc != TF_OK) return rc;
        rc = tf_prefill_grouped_routed_moe_resident(ctx, stream, routed_hidden, routed_hidden_offset, routed_hidden_stride_elements, sorted_pairs, chunks,
                                                    chunk_count, kFewScratchChunks, query_count * top_k, expert_pool, expert_pool_stride, num_experts,
                                                    routed_offsets, acts_scratch, route_partials, d, f, top_k, scale_dtype);
        if (rc != TF_OK) return rc;
        return tf_prefill_moe_reduce_token_major(ctx, stream, route_partials, 0, out_weights, out_weights_offset, h2, h2_offset, query_count, top_k, d);
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    float *logits = ctx->prefill_logits;
    hipLaunchKernelGGL(few_logits_kernel<0>, dim3(num_experts, query_count), dim3(256), 0, st, w, s, b, h, hidden_stride_elements, eff, logits,
                       num_experts, (int)d);
    int32_t rc = check_launch(ctx, "prefill_routed_moe_few_tokens logits");
    if (rc != TF_OK) return rc;
    half_t *acts = static_cast<half_t *>(acts_scratch);
    half_t *partials = static_cast<half_t *>(route_partials);
    const dim3 grid1(((f + plan.rt - 1) / plan.rt + 3) / 4, query_count * kFewTopK);
    const size_t lds1 = (size_t)few_image_bytes(d) + (size_t)query_count * num_experts * 4;
    bool launched = false;
#define TF_FEW_P1(RT_, NP_)                                                                                                                  \
    if (!launched && plan.rt == RT_ && plan.np == NP_) {                                                                                     \
        launched = true;                                                                                                                     \
        if (scale_dtype == TF_BF16)                                                                                                          \
            hipLaunchKernelGGL((few_phase1_kernel<RT_, NP_, 0>), grid1, dim3(256), lds1, st, logits, pes, pool, expert_pool_stride, x,       \
                               routed_hidden_stride_elements, acts, oi, ow, query_count, num_experts, d, f, *routed_offsets);                       \
        else                                                                                                                                 \
            hipLaunchKernelGGL((few_phase1_kernel<RT_, NP_, 1>), grid1, dim3(256), lds1, st, logits, pes, pool, expert_pool_stride, x,       \
                               routed_hidden_stride_elements, acts, oi, ow, query_count, num_experts, d, f, *routed_offsets);                       \
    }
    TF_FEW_P1(1, 1) TF_FEW_P1(1, 2) TF_FEW_P1(2, 2) TF_FEW_P1(2, 3) TF_FEW_P1(2, 4) TF_FEW_P1(4, 3) TF_FEW_P1(4, 4)
#undef TF_FEW_P1
    rc = check_launch(ctx, "prefill_routed_moe_few_tokens gate / up");
    if (rc != TF_OK) return rc;
    const dim3 grid2((d + best_rpb - 1) / best_rpb);
#define TF_FEW_DN(NP_, SD_)                                                                                                                  \
    hipLaunchKernelGGL((few_down_kernel<NP_, SD_>), grid2, dim3(64 * kFewDownWaves), 0, st, oi, ow, pool, expert_pool_stride, acts, partials, out, query_count, \
                       d, f, best_rpb, inv_nch, num_experts, *routed_offsets)
    if (scale_dtype == TF_BF16) {
        if (best_np == 1) TF_FEW_DN(1, 0); else if (best_np == 2) TF_FEW_DN(2, 0); else if (best_np == 3) TF_FEW_DN(3, 0); else TF_FEW_DN(4, 0);
    } else {
        if (best_np == 1) TF_FEW_DN(1, 1); else if (best_np == 2) TF_FEW_DN(2, 1); else if (best_np == 3) TF_FEW_DN(3, 1); else TF_FEW_DN(4, 1);
    }
#undef TF_FEW_DN
    return check_launch(ctx, "prefill_routed_moe_few_tokens down + reduce");
}

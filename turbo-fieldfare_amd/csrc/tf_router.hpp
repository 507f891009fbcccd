// Router arithmetic shared by the decode router and the per-token prefill router.
#pragma once

#include "tf_common.hpp"

namespace tfk {

// logits[e] = sum_g [ s * sum(q * x') + b * sum(x') ],  x' = float(hidden) * float(effective_scale).
// One wave per expert row.  NPASS > 0: every operand 16-byte aligned and d <= 1024 * NPASS; the lane's <= NPASS chunks of
// 16 weights are all requested before the first is used, so the row costs one memory round trip.  NPASS == 0: any
// alignment and size, byte/halfword loads in a loop.
__device__ __forceinline__ void router_chunk(const u32x4 w, const u32x4 ha, const u32x4 hb, const u32x4 ea, const u32x4 eb,
                                             float s, float b, float &acc) {
    float dot = 0.0f, sum = 0.0f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
        const uint32_t hw = i < 8 ? ha[i >> 1] : hb[(i - 8) >> 1];
        const uint32_t ew = i < 8 ? ea[i >> 1] : eb[(i - 8) >> 1];
        const uint16_t hbits = (uint16_t)((i & 1) ? (hw >> 16) : (hw & 0xFFFFu));
        const float ev = (i & 1) ? __uint_as_float(ew & 0xFFFF0000u) : __uint_as_float(ew << 16);
        const float xv = f16_to_f32(hbits) * ev;
        const float q = (float)((w[i >> 2] >> (8 * (i & 3))) & 0xFFu);
        dot = fmaf(q, xv, dot);
        sum += xv;
    }
    acc = fmaf(s, dot, acc);
    acc = fmaf(b, sum, acc);
}

template <int SD, int NPASS>
__device__ __forceinline__ float router_row(const uint8_t *w_row, const uint8_t *s_row, const uint8_t *b_row,
                                            const half_t *hidden, const uint16_t *eff, int d, int lane) {
    float acc = 0.0f;
    if constexpr (NPASS > 0) {
        const int chunks = d >> 4;
        u32x4 w[NPASS], ha[NPASS], hb[NPASS], ea[NPASS], eb[NPASS];
        uint16_t sv[NPASS], bv[NPASS];
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const int c = lane + 64 * p;
            w[p] = ha[p] = hb[p] = ea[p] = eb[p] = u32x4{0u, 0u, 0u, 0u};
            sv[p] = bv[p] = 0;
            if (c < chunks) {
                w[p] = load16(w_row + (size_t)c * 16);
                ha[p] = load16(hidden + c * 16);
                hb[p] = load16(hidden + c * 16 + 8);
                ea[p] = load16(eff + c * 16);
                eb[p] = load16(eff + c * 16 + 8);
                sv[p] = *reinterpret_cast<const uint16_t *>(s_row + (c >> 2) * 2);
                bv[p] = *reinterpret_cast<const uint16_t *>(b_row + (c >> 2) * 2);
            }
        }
#pragma unroll
        for (int p = 0; p < NPASS; ++p)
            router_chunk(w[p], ha[p], hb[p], ea[p], eb[p], sb_to_f32<SD>(sv[p]), sb_to_f32<SD>(bv[p]), acc);
    } else {
        const int words = d >> 2;
        for (int wi = lane; wi < words; wi += kWave) {
            const int g = wi >> 4;
            const float s = sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(s_row + g * 2));
            const float b = sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(b_row + g * 2));
            float dot = 0.0f, sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float xv = (float)hidden[wi * 4 + i] * bf16_to_f32(eff[wi * 4 + i]);
                dot = fmaf((float)w_row[wi * 4 + i], xv, dot);
                sum += xv;
            }
            acc = fmaf(s, dot, acc);
            acc = fmaf(b, sum, acc);
        }
    }
    return wave_sum(acc);
}

// The same row by a whole 256-thread block (d <= 4096, every operand 16-byte aligned): thread t takes chunk t of 16 weights,
// so the arithmetic after the one memory round trip is a third of a wave-per-row pass at d = 2816; the four wave sums meet in
// LDS and are added in wave order.  Returns the logit in every thread.  `partial`: 4 floats of LDS.
template <int SD>
__device__ __forceinline__ float router_row_block(const uint8_t *w_row, const uint8_t *s_row, const uint8_t *b_row, const half_t *hidden,
                                                  const uint16_t *eff, int d, float *partial) {
    const int c = threadIdx.x, chunks = d >> 4;
    float acc = 0.0f;
    if (c < chunks) {
        const u32x4 w = load16(w_row + (size_t)c * 16);
        const u32x4 ha = load16(hidden + c * 16), hb = load16(hidden + c * 16 + 8);
        const u32x4 ea = load16(eff + c * 16), eb = load16(eff + c * 16 + 8);
        const uint16_t sv = *reinterpret_cast<const uint16_t *>(s_row + (c >> 2) * 2);
        const uint16_t bv = *reinterpret_cast<const uint16_t *>(b_row + (c >> 2) * 2);
        router_chunk(w, ha, hb, ea, eb, sb_to_f32<SD>(sv), sb_to_f32<SD>(bv), acc);
    }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    return ((partial[0] + partial[1]) + partial[2]) + partial[3];
}

// Top-k over <= 256 fp32 logits by one wave, then softmax over the selected and the per-expert gain.
// Same ordering as the reference's serial insertion (moe.metal:152-171): score descending, ties to the lower index;
// NaN and -inf are never selected; an unfilled position reads index 0 with score -inf.
// Lane l holds candidates l, l+64, l+128, l+192 and their gains; each round takes the wave maximum with DPP and finds
// its lowest expert index with ballots, so a round is a few dozen ALU instructions and no memory traffic.
// router_select_lanes leaves selection i in lane i (i < top_k): its expert index and its routing weight.
// NC = candidates per lane: 2 serves up to 128 experts, 4 up to 256.
// router_select_core: the same on candidates already in registers (cand[j] = logit of expert lane + 64 j, -inf where
// there is no such expert or the logit is NaN; gain[j] its per-expert gain).  cand is consumed.
template <int NC>
__device__ __forceinline__ void router_select_core(float (&cand)[NC], const float (&gain)[NC], uint32_t top_k, int lane,
                                                   uint32_t &sel_index, half_t &sel_weight) {
    float my_score = -INFINITY, my_gain = 0.0f;   // lane i (< top_k) ends up holding the i-th selection
    uint32_t my_idx = 0;
    for (uint32_t i = 0; i < top_k; ++i) {
        float m = cand[0];
#pragma unroll
        for (int j = 1; j < NC; ++j) m = fmaxf(m, cand[j]);
        const float wm = wave_max(m);
        const bool found = wm > -INFINITY;
        int sel_j = NC, sel_lane = 0;
#pragma unroll
        for (int j = NC - 1; j >= 0; --j) {
            const uint64_t mask = __ballot(cand[j] == wm);
            if (mask) { sel_j = j; sel_lane = __builtin_ctzll(mask); }
        }
        float g = 0.0f;
#pragma unroll
        for (int j = 0; j < NC; ++j)
            if (sel_j == j) g = read_lane(gain[j], sel_lane);
        if ((uint32_t)lane == i) {
            my_score = found ? wm : -INFINITY;
            my_idx = found ? (uint32_t)(sel_lane + 64 * sel_j) : 0u;
            my_gain = found ? g : read_lane(gain[0], 0);
        }
        if (found && lane == sel_lane) {
#pragma unroll
            for (int j = 0; j < NC; ++j)
                if (sel_j == j) cand[j] = -INFINITY;
        }
    }
    const float max_s = read_lane(my_score, 0);
    const float ex = (uint32_t)lane < top_k ? expf(my_score - max_s) : 0.0f;
    float sum_exp = 0.0f;   // summed in selection order, like the reference
    for (uint32_t i = 0; i < top_k; ++i) sum_exp += read_lane(ex, (int)i);
    sel_index = my_idx;
    sel_weight = (half_t)((ex / sum_exp) * my_gain);
}

template <int NC>
__device__ __forceinline__ void router_select_lanes(const float *logits, const uint16_t *per_expert_scale, uint32_t num_experts,
                                                    uint32_t top_k, int lane, uint32_t &sel_index, half_t &sel_weight) {
    float cand[NC], gain[NC];
#pragma unroll
    for (int j = 0; j < NC; ++j) {
        const uint32_t e = lane + 64 * j;
        const float v = e < num_experts ? logits[e] : -INFINITY;
        gain[j] = e < num_experts ? bf16_to_f32(per_expert_scale[e]) : 0.0f;
        cand[j] = (v != v) ? -INFINITY : v;
    }
    router_select_core<NC>(cand, gain, top_k, lane, sel_index, sel_weight);
}

__device__ __forceinline__ void router_select_lanes(const float *logits, const uint16_t *per_expert_scale, uint32_t num_experts,
                                                    uint32_t top_k, int lane, uint32_t &sel_index, half_t &sel_weight) {
    if (num_experts <= 128) router_select_lanes<2>(logits, per_expert_scale, num_experts, top_k, lane, sel_index, sel_weight);
    else router_select_lanes<4>(logits, per_expert_scale, num_experts, top_k, lane, sel_index, sel_weight);
}

// Top-8 of <= 256 logits by a whole 256-thread block, by counting: a candidate's position in the order (score descending,
// ties to the lower index) is the number of candidates that beat it, and with 128 experts two threads share a candidate's
// 128 comparisons, so the selection costs the block a few hundred instructions with no serial chain where the one-wave
// selection above walks eight dependent rounds.  The count ignores ties; when any of the first eight positions is claimed
// twice or not at all (equal scores, fewer than eight finite logits) the block says so and the caller falls back to the
// one-wave selection, which is exact in every case.  On success chosen[0..8) holds the expert indices in selection order and
// cand[e] the logit of expert e (NaN read as -inf).  Every thread of the block must call; ends with a barrier.
struct RankSelectLds {
    __attribute__((aligned(16))) float cand[256];
    uint32_t part[2][128];
    __attribute__((aligned(16))) uint32_t claims[8];
};
__device__ __forceinline__ float rank_select_load(const float *logits, uint32_t num_experts) {
    const uint32_t c = num_experts <= 128 ? (threadIdx.x & 127) : threadIdx.x;
    float v = c < num_experts ? logits[c] : -INFINITY;
    return v;
}
__device__ __forceinline__ bool rank_select_block(float my_logit, uint32_t num_experts, RankSelectLds &l, uint32_t *chosen) {
    const bool two_per_candidate = num_experts <= 128;
    const uint32_t c = two_per_candidate ? (threadIdx.x & 127) : threadIdx.x;
    const float v = (my_logit != my_logit) ? -INFINITY : my_logit;
    l.cand[threadIdx.x] = (two_per_candidate && threadIdx.x >= 128) ? -INFINITY : v;
    if (threadIdx.x < 8) l.claims[threadIdx.x] = 0u;
    lds_barrier();
    uint32_t beaten_by = 0;
    if (two_per_candidate) {
        const uint32_t h = (uint32_t)__builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 7));
        const f32x4 *src = reinterpret_cast<const f32x4 *>(l.cand + 64 * h);
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const f32x4 q = src[j];
            beaten_by += (q[0] > v) + (q[1] > v) + (q[2] > v) + (q[3] > v);
        }
        l.part[h][c] = beaten_by;
        lds_barrier();
        beaten_by = l.part[0][c] + l.part[1][c];
    } else {
        const f32x4 *src = reinterpret_cast<const f32x4 *>(l.cand);
#pragma unroll 8
        for (int j = 0; j < 64; ++j) {
            const f32x4 q = src[j];
            beaten_by += (q[0] > v) + (q[1] > v) + (q[2] > v) + (q[3] > v);
        }
    }
    const bool owner = !two_per_candidate || threadIdx.x < 128;
    if (owner && beaten_by < 8u && v > -INFINITY) {
        chosen[beaten_by] = c;
        atomicAdd(&l.claims[beaten_by], 1u);
    }
    lds_barrier();
    const u32x4 c0 = *reinterpret_cast<const u32x4 *>(l.claims), c1 = *reinterpret_cast<const u32x4 *>(l.claims + 4);
    const bool ok = c0[0] == 1u && c0[1] == 1u && c0[2] == 1u && c0[3] == 1u && c1[0] == 1u && c1[1] == 1u && c1[2] == 1u && c1[3] == 1u;
    return __builtin_amdgcn_readfirstlane((int)ok) != 0;
}

// The routing weights of a selection made by rank_select_block, computed by one wave exactly as router_select_core's tail
// does: softmax over the selected scores in selection order, times the per-expert gain.  Lane i < 8 gets selection i.
__device__ __forceinline__ void rank_select_weights(const RankSelectLds &l, const uint32_t *chosen, const uint16_t *per_expert_scale, int lane,
                                                    uint32_t &sel_index, half_t &sel_weight) {
    const uint32_t e = lane < 8 ? chosen[lane] : 0u;
    const float score = lane < 8 ? l.cand[e] : -INFINITY;
    const float gain = bf16_to_f32(per_expert_scale[e]);
    const float max_s = read_lane(score, 0);
    const float ex = lane < 8 ? expf(score - max_s) : 0.0f;
    float sum_exp = 0.0f;
    for (int i = 0; i < 8; ++i) sum_exp += read_lane(ex, i);
    sel_index = e;
    sel_weight = (half_t)((ex / sum_exp) * gain);
}

__device__ __forceinline__ void router_select(const float *logits, const uint16_t *per_expert_scale, uint32_t *out_indices,
                                              half_t *out_weights, uint32_t num_experts, uint32_t top_k, int lane) {
    uint32_t idx;
    half_t weight;
    router_select_lanes(logits, per_expert_scale, num_experts, top_k, lane, idx, weight);
    if ((uint32_t)lane < top_k) {
        out_indices[lane] = idx;
        out_weights[lane] = weight;
    }
}


}  // namespace tfk

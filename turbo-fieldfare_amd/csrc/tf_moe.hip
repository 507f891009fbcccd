// Router (int8 GEMV + top-8 + softmax), routed expert phases 1 and 2, and the int4 shared expert, for gfx950.
#include "../../include/tf_bench.h"
#include "tf_gemv_kernels.hpp"
#include "tf_router.hpp"
#include "tf_rowslice.hpp"

using namespace tfk;

// Router logits of tf_moe_decode_step_static: device memory that exists from load time on, one copy per GPU, so that entry
// point never allocates.  Host code never uses the array's name as an address: tf_ctx_create asks the runtime for the
// address of this device's copy (moe_static_scratch_setup) and every launch passes that pointer.
constexpr uint32_t kStaticMaxExperts = 256;
static __device__ __align__(256) float scratch[kStaticMaxExperts];

// Per-wave timeline of the decode step's kernels for tuning, compiled only with -DTF_STAMPS (never in the shipped library):
// lane 0 of a wave writes the 100 MHz wall clock into slot `slot` of its row in a load-time buffer that
// tf_debug_stamps() hands to the host.
#ifdef TF_STAMPS
constexpr uint32_t kStampWaves = 4096;
static __device__ unsigned long long stamp_buf[3 * kStampWaves * 8];
#define TF_STAMP(kernel_, wave_, slot_)                                                                                   \
    do {                                                                                                                  \
        if ((threadIdx.x & 63) == 0 && (wave_) < kStampWaves) stamp_buf[(((kernel_) * kStampWaves + (wave_)) << 3) + (slot_)] = wall_clock64(); \
    } while (0)
#ifdef TF_STAMPS_NOWAIT
#define TF_STAMP_WAIT() do {} while (0)
#else
#define TF_STAMP_WAIT() asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#endif
extern "C" unsigned long long *tf_debug_stamps(void) {
    void *ptr = nullptr;
    return hipGetSymbolAddress(&ptr, HIP_SYMBOL(stamp_buf)) == hipSuccess ? static_cast<unsigned long long *>(ptr) : nullptr;
}
#else
#define TF_STAMP(kernel_, wave_, slot_) do {} while (0)
#define TF_STAMP_WAIT() do {} while (0)
#endif

namespace tfk {

int32_t moe_static_scratch_setup(tf_ctx *ctx) {
    void *ptr = nullptr;
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // the context's device is current here
    if (e != hipSuccess || !ptr) return fail(ctx, TF_ERR_DEVICE, "moe static scratch: %s", hipGetErrorString(e));
    ctx->static_router_logits = static_cast<float *>(ptr);
    return TF_OK;
}

}  // namespace tfk

namespace {

struct RoutedArg {
    const uint8_t *blob[TF_MAX_STREAMED_EXPERTS];
    const uint8_t *pool;
    uint64_t stride;
    const uint32_t *indices;
    uint32_t num_experts;
};

// Base pointer of the expert serving `slot`: a host-chosen pointer, or pool + stride * indices[slot] with the
// index read on the device.
__device__ __forceinline__ const uint8_t *blob_base(const RoutedArg &r, uint32_t slot) {
    if (r.indices) {
        uint32_t e = r.indices[slot];
        e = e < r.num_experts ? e : r.num_experts - 1;
        return r.pool + (uint64_t)e * r.stride;
    }
    return r.blob[slot];
}

// ------------------------------------------------------------------------------------------------ router
// Two launches, as in the reference (router_gemv_gemma4_r4 then router_topk_select_k8): one wave per expert row writes
// its logit; a single wave then selects.  Both stay on the device; nothing returns to the host.
template <int SD, int NPASS>
__global__ __launch_bounds__(256) void router_logits_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                            const half_t *hidden, const uint16_t *eff, float *logits,
                                                            uint32_t num_experts, int d) {
    const int lane = threadIdx.x & 63;
    const uint32_t e = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (e >= num_experts) return;
    const int groups = d >> 6;
    const float v = router_row<SD, NPASS>(W + (size_t)e * d, S + (size_t)e * groups * 2, B + (size_t)e * groups * 2, hidden, eff, d, lane);
    if (lane == 0) logits[e] = v;
}

// One block per expert row (aligned operands, d <= 4096).  The kernels below are thin shells around `..._body` functions so
// that two independent stages can share a launch (a block takes one role or the other by its index).
template <int SD>
__device__ __forceinline__ void router_logits_block_body(const uint8_t *W, const uint8_t *S, const uint8_t *B, const half_t *hidden,
                                                         const uint16_t *eff, float *logits, int d, uint32_t e, float *partial) {
    TF_STAMP(0, e * 4 + (threadIdx.x >> 6), 0);
    const int groups = d >> 6;
    const float v = router_row_block<SD>(W + (size_t)e * d, S + (size_t)e * groups * 2, B + (size_t)e * groups * 2, hidden, eff, d, partial);
    if (threadIdx.x == 0) logits[e] = v;
    TF_STAMP(0, e * 4 + (threadIdx.x >> 6), 1);
}
template <int SD>
__global__ __launch_bounds__(256) void router_logits_block_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B, const half_t *hidden,
                                                                  const uint16_t *eff, float *logits, int d) {
    __shared__ float partial[4];
    router_logits_block_body<SD>(W, S, B, hidden, eff, logits, d, blockIdx.x, partial);
}

__global__ __launch_bounds__(64) void router_select_kernel(const float *logits, const uint16_t *per_expert_scale,
                                                           uint32_t *out_indices, half_t *out_weights, uint32_t num_experts,
                                                           uint32_t top_k) {
    router_select(logits, per_expert_scale, out_indices, out_weights, num_experts, top_k, threadIdx.x);
}

// ------------------------------------------------------------------------------------------------ phase 1
__device__ __forceinline__ void store_act(half_t *acts, uint32_t index, float gate, float up) {
    acts[index] = (half_t)(gelu_tanh_fast(gate) * up);
}

struct Phase1Geom {
    uint32_t d, f, top_k;
    uint32_t active_count;            // subset variant only
    const uint32_t *active_slots;     // nullptr: all slots
};

__device__ __forceinline__ bool phase1_slot(const Phase1Geom &g, uint32_t unit, uint32_t units_per_slot, uint32_t &slot, uint32_t &tile) {
    const uint32_t a = unit / units_per_slot;
    tile = unit - a * units_per_slot;
    if (g.active_slots) {
        if (a >= g.active_count) return false;
        slot = g.active_slots[a];
    } else {
        if (a >= g.top_k) return false;
        slot = a;
    }
    return slot < g.top_k;
}

// Selection fused into phase 1 (the decode step): every block repeats the top-k over the router's logits (by counting,
// all four waves at once; the one-wave serial selection only when scores tie) while its activation loads are in flight,
// instead of the grid waiting for a selection kernel and then for its indices; block 0 publishes indices and weights for
// phase 2 and for the caller.
struct FusedSelect {
    const float *logits;
    const uint16_t *per_expert_scale;
    uint32_t *out_indices;
    half_t *out_weights;
    uint32_t num_experts;
};

// D > 1024: one wave per RT-row tile of one slot; the gate tile and the up tile share the activations, which the block
// stages once in LDS.  Order of requests: activations, expert lookup, weights; the activations are arranged while the
// weights are in flight (with the fused selection the weights are requested right after the block's barrier).
template <int RT, int NP, int SD, bool FUSED>
__device__ __forceinline__ void phase1_long_body(const RoutedArg &routed, const tf_expert_offsets &off, const half_t *x, half_t *acts,
                                                 const Phase1Geom &g, const FusedSelect &fs, uint32_t block, u32x4 *xa, float *xsum,
                                                 uint32_t *chosen, RankSelectLds &sel) {
    const int lane = threadIdx.x & 63;
    const uint32_t unit = uniform_u32((block * blockDim.x + threadIdx.x) >> 6);
    const uint32_t tiles = (g.f + RT - 1) / RT;
    TF_STAMP(1, unit, 0);
    float my_logit = 0.0f;
    if constexpr (FUSED) my_logit = rank_select_load(fs.logits, fs.num_experts);   // requested first: the selection waits for nothing else
    XStage stage;
    stage.request(x, (int)g.d);
    uint32_t slot = 0, tile = 0;
    const bool live = phase1_slot(g, unit, tiles, slot, tile);
    const uint32_t row0 = tile * RT;
    const size_t w_byte = (size_t)row0 * (g.d >> 1);
    const size_t sb_byte = (size_t)row0 * (g.d >> 6) * 2;
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile tg, tu;
    rs.init_map((int)g.d, lane);
    auto request_weights = [&](const uint8_t *base) {
        rs.load(tg, base + off.gate_W_off + w_byte, base + off.gate_s_off + sb_byte, base + off.gate_b_off + sb_byte, g.f - row0);
        rs.load(tu, base + off.up_W_off + w_byte, base + off.up_s_off + sb_byte, base + off.up_b_off + sb_byte, g.f - row0);
    };
    bool ranked = false;
    if constexpr (FUSED) {
        ranked = rank_select_block(my_logit, fs.num_experts, sel, chosen);
        if (!ranked && uniform_u32(threadIdx.x >> 6) == 0) {
            uint32_t idx;
            half_t weight;
            router_select_lanes(fs.logits, fs.per_expert_scale, fs.num_experts, g.top_k, lane, idx, weight);
            if ((uint32_t)lane < g.top_k) {
                chosen[lane] = idx < fs.num_experts ? idx : fs.num_experts - 1;
                if (block == 0) {
                    fs.out_indices[lane] = idx;
                    fs.out_weights[lane] = weight;
                }
            }
        }
    } else {
        if (live) request_weights(uniform_ptr(blob_base(routed, slot)));
    }
    TF_STAMP(1, unit, 1);
    stage.publish((int)g.d, xa, xsum);
    TF_STAMP(1, unit, 2);
    if (!live) return;
    if constexpr (FUSED) {
        request_weights(routed.pool + (uint64_t)uniform_u32(chosen[slot]) * routed.stride);
        if (ranked && block == 0 && threadIdx.x < 64) {   // the step's outputs, off the path of the weight requests
            uint32_t idx;
            half_t weight;
            rank_select_weights(sel, chosen, fs.per_expert_scale, lane, idx, weight);
            if ((uint32_t)lane < g.top_k) {
                fs.out_indices[lane] = idx;
                fs.out_weights[lane] = weight;
            }
        }
    }
    rs.init_x_lds(xa, xsum, (int)g.d);
    TF_STAMP_WAIT();
    TF_STAMP(1, unit, 3);
    float gate[RT], up[RT];
    rs.template reduce<SD>(tg, gate);
    rs.template reduce<SD>(tu, up);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r)
            if (row0 + r < g.f) store_act(acts, slot * g.f + row0 + r, gate[r], up[r]);
    }
    TF_STAMP(1, unit, 4);
}

template <int RT, int NP, int SD, bool FUSED>
__global__ __launch_bounds__(256) void phase1_long_kernel(RoutedArg routed, tf_expert_offsets off, const half_t *x,
                                                          half_t *acts, Phase1Geom g, FusedSelect fs) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ uint32_t chosen[TF_MAX_STREAMED_EXPERTS];
    __shared__ RankSelectLds sel;
    phase1_long_body<RT, NP, SD, FUSED>(routed, off, x, acts, g, fs, blockIdx.x, xa, xsum, chosen, sel);
}

// D <= 1024: half-wave per row, NPASS passes: 2 * NPASS rows of gate and up per wave.
template <int NPASS, int SD>
__global__ __launch_bounds__(256) void phase1_short_kernel(RoutedArg routed, tf_expert_offsets off, const half_t *x,
                                                           half_t *acts, Phase1Geom g) {
    const int lane = threadIdx.x & 63;
    const uint32_t unit = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint32_t tiles = (g.f + 2 * NPASS - 1) / (2 * NPASS);
    uint32_t slot, tile;
    if (!phase1_slot(g, unit, tiles, slot, tile)) return;
    const uint8_t *base = blob_base(routed, slot);
    const long row0 = (long)tile * 2 * NPASS;
    ShortRows sr;
    sr.init(x, g.d, lane);
    ShortRows::Pair tg[NPASS], tu[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        sr.load(tg[p], base + off.gate_W_off, base + off.gate_s_off, base + off.gate_b_off, row0 + 2 * p, g.f, g.d);
        sr.load(tu[p], base + off.up_W_off, base + off.up_s_off, base + off.up_b_off, row0 + 2 * p, g.f, g.d);
    }
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        float glo, ghi, ulo, uhi;
        sr.template reduce<SD>(tg[p], glo, ghi);
        sr.template reduce<SD>(tu[p], ulo, uhi);
        if (lane == 0) {
            const long r = row0 + 2 * p;
            if (r < g.f) store_act(acts, slot * g.f + (uint32_t)r, glo, ulo);
            if (r + 1 < g.f) store_act(acts, slot * g.f + (uint32_t)r + 1, ghi, uhi);
        }
    }
}

template <int SD>
__global__ __launch_bounds__(256) void phase1_generic_kernel(RoutedArg routed, tf_expert_offsets off, const half_t *x,
                                                             half_t *acts, Phase1Geom g) {
    const int lane = threadIdx.x & 63;
    const uint32_t unit = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    uint32_t slot, r;
    if (!phase1_slot(g, unit, g.f, slot, r)) return;
    const uint8_t *base = blob_base(routed, slot);
    const int groups = g.d >> 6;
    const size_t w_byte = (size_t)r * (g.d >> 1), sb_byte = (size_t)r * groups * 2;
    const float gate = generic_row_dot<SD>(base + off.gate_W_off + w_byte, base + off.gate_s_off + sb_byte, base + off.gate_b_off + sb_byte, x, g.d, lane);
    const float up = generic_row_dot<SD>(base + off.up_W_off + w_byte, base + off.up_s_off + sb_byte, base + off.up_b_off + sb_byte, x, g.d, lane);
    if (lane == 0) store_act(acts, slot * g.f + r, gate, up);
}

// ------------------------------------------------------------------------------------------------ phase 2
// y[r] = half(residual[r] + sum_slot w[slot] * down_slot[r,:] . acts[slot,:]), slots added in order 0..7.
// Block = 8 waves, wave s serves slot s; F <= 1024: 2 * NPASS rows per block.
template <int NPASS, int SD>
__global__ __launch_bounds__(512) void phase2_short_kernel(RoutedArg routed, tf_expert_offsets off, const half_t *acts,
                                                           const half_t *routing_w, const half_t *residual, half_t *y,
                                                           uint32_t d, uint32_t f) {
    __shared__ float partial[8][2 * NPASS];
    const int lane = threadIdx.x & 63;
    const uint32_t slot = uniform_u32(threadIdx.x >> 6);
    const long row0 = (long)blockIdx.x * 2 * NPASS;
    TF_STAMP(2, blockIdx.x * 8 + slot, 0);
    ShortRows sr;
    ShortRows::Pair t[NPASS];
    sr.init_map(f, lane);
    // requests in this order: what does not depend on the expert lookup (activations, routing weight), the lookup,
    // then the weights
    u32x4 xr[4];
#pragma unroll
    for (int dd = 0; dd < 4; ++dd) xr[dd] = load16(acts + (size_t)slot * f + (sr.col < 0 ? 0 : sr.col) * 32 + dd * 8);
    const half_t w16 = routing_w[slot];
    const bool writer = threadIdx.x < 2 * NPASS && row0 + threadIdx.x < d;
    const half_t res16 = writer ? residual[row0 + threadIdx.x] : (half_t)0.0f;   // requested now, needed after the barrier
    const uint8_t *base = uniform_ptr(blob_base(routed, slot));
    TF_STAMP(2, blockIdx.x * 8 + slot, 1);
#pragma unroll
    for (int p = 0; p < NPASS; ++p)
        sr.load(t[p], base + off.down_W_off, base + off.down_s_off, base + off.down_b_off, row0 + 2 * p, d, f);
    sr.xs = arrange_x(xr, sr.xq);
    const float w = (float)w16;
    TF_STAMP_WAIT();
    TF_STAMP(2, blockIdx.x * 8 + slot, 2);
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        float lo, hi;
        sr.template reduce<SD>(t[p], lo, hi);
        if (lane == 0) {
            partial[slot][2 * p] = w * lo;
            partial[slot][2 * p + 1] = w * hi;
        }
    }
    TF_STAMP(2, blockIdx.x * 8 + slot, 3);
    __syncthreads();
    if (writer) {
        float acc = (float)res16;
#pragma unroll
        for (int s = 0; s < 8; ++s) acc += partial[s][threadIdx.x];
        y[row0 + threadIdx.x] = (half_t)acc;
    }
    TF_STAMP(2, blockIdx.x * 8 + slot, 4);
}

// The same projection with an even share of the rows for every block and every lane busy (F <= 1024, 16-byte aligned operands).
// A block takes `rpb` consecutive rows; wave s reads those rows of slot s's matrix as ONE flat stream of 16-byte chunks
// (rows are contiguous: pass p, lane l reads chunk 64 p + l of the block's rows, 1 KiB per load instruction), so at F = 704
// eleven rows fill 242 of the 256 chunk positions of four passes where one row per half-wave fills 22 of 32, and 2816 rows make
// exactly one block for each of 256 CUs.  A lane's chunk lies in row c / nch, column c % nch: the slot's activations are staged
// once per wave in LDS in dot-product order and each pass picks its column there.  Row sums are sums over runs of nch
// consecutive lanes that may cross a pass boundary: every pass is prefix-summed across the wave (six DPP adds), the running
// sums go to LDS indexed by chunk, and lane r takes row r's sum as a difference of two of them.
// The hot arguments lead the list as plain scalars (kernel-argument preloading takes leading scalars only).
constexpr int kFlatMaxRows = 32;
struct BlobPtrs {
    const uint8_t *blob[TF_MAX_STREAMED_EXPERTS];
};
__device__ __forceinline__ float wave_inclusive_scan(float v) {
    v += dpp_f32<0x111>(v);          // row_shr:1 (lanes without a source inside their row of 16 add 0)
    v += dpp_f32<0x112>(v);          // row_shr:2
    v += dpp_f32<0x114>(v);          // row_shr:4
    v += dpp_f32<0x118>(v);          // row_shr:8
    v += dpp_f32<0x142, 0xA>(v);     // row_bcast15 into rows 1 and 3
    v += dpp_f32<0x143, 0xC>(v);     // row_bcast31 into rows 2 and 3
    return v;
}
template <int NP, int SD>
__global__ __launch_bounds__(512) void phase2_flat_kernel(const uint32_t *indices, const uint8_t *pool, uint64_t stride, const half_t *acts,
                                                          const half_t *routing_w, const half_t *residual, half_t *y, uint32_t d, uint32_t f,
                                                          uint32_t rpb, uint32_t inv_nch, uint32_t num_experts, tf_expert_offsets off,
                                                          BlobPtrs blobs) {
    __shared__ __align__(16) u32x4 xa[8][128];        // [slot][word d of column c at d * nch + c]
    __shared__ float xsum[8][32];
    __shared__ float running[8][NP * 64];             // [slot][chunk]: inclusive sums within each pass
    __shared__ float partial[8][kFlatMaxRows];
    const int lane = threadIdx.x & 63;
    const uint32_t slot = uniform_u32(threadIdx.x >> 6);
    const uint32_t row0 = blockIdx.x * rpb;
    const uint32_t rows_here = min(rpb, d - row0);
    const int nch = (int)(f >> 5), groups = (int)(f >> 6), pieces = (int)(f >> 3);
    TF_STAMP(2, blockIdx.x * 8 + slot, 0);
    // what does not depend on the expert lookup goes first: the slot's activations, its routing weight, the residual
    const rsrc_t ra = make_rsrc(acts + (size_t)slot * f, f * 2u);
    u32x4 xr[2];
    xr[0] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, (uint32_t)lane * 16u, 0, 0));
    xr[1] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(ra, (uint32_t)(lane + 64) * 16u, 0, 0));
    const half_t w16 = routing_w[slot];
    const bool writer = threadIdx.x < rows_here;
    const half_t res16 = writer ? residual[row0 + threadIdx.x] : (half_t)0.0f;   // needed after the barrier
    const uint8_t *base;
    if (indices) {
        uint32_t e = indices[slot];
        e = e < num_experts ? e : num_experts - 1;
        base = pool + (uint64_t)e * stride;
    } else {
        base = blobs.blob[slot];
    }
    base = uniform_ptr(base);
    TF_STAMP(2, blockIdx.x * 8 + slot, 1);
    const rsrc_t rw = make_rsrc(base + off.down_W_off + (size_t)row0 * (f >> 1), rows_here * (f >> 1));
    const rsrc_t rs = make_rsrc(base + off.down_s_off + (size_t)row0 * groups * 2, rows_here * (uint32_t)groups * 2u);
    const rsrc_t rb = make_rsrc(base + off.down_b_off + (size_t)row0 * groups * 2, rows_here * (uint32_t)groups * 2u);
    u32x4 w[NP];
    uint16_t sv[NP], bv[NP];
    int col[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        const uint32_t c = 64u * p + (uint32_t)lane;
        const uint32_t r = (c * inv_nch) >> 16;            // c / nch (the host checked the reciprocal for every c < 64 NP)
        const uint32_t cc = c - r * (uint32_t)nch;
        col[p] = (int)cc;
        const uint32_t sboff = (r * (uint32_t)groups + (cc >> 1)) * 2u;   // past the block's rows: past the descriptor, reads zero
        w[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, c * 16u, 0, kStreamOnce));
        sv[p] = __builtin_amdgcn_raw_buffer_load_b16(rs, sboff, 0, 0);
        bv[p] = __builtin_amdgcn_raw_buffer_load_b16(rb, sboff, 0, 0);
    }
    // the wave's own LDS image of its slot's activations (LDS serves one wave's requests in order: no barrier needed)
    XStage::publish_piece(xr[0], lane, pieces, nch, xa[slot], xsum[slot]);
    XStage::publish_piece(xr[1], lane + 64, pieces, nch, xa[slot], xsum[slot]);
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    const float wgt = (float)w16;
    TF_STAMP_WAIT();
    TF_STAMP(2, blockIdx.x * 8 + slot, 2);
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        half2_t xq[16];
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) {
            const u32x4 v = xa[slot][dd * nch + col[p]];
#pragma unroll
            for (int j = 0; j < 4; ++j) xq[4 * dd + j] = as_half2(v[j]);
        }
        const float part = fmaf(sb_to_f32<SD>(sv[p]), chunk_dot(w[p], xq), sb_to_f32<SD>(bv[p]) * xsum[slot][col[p]]);
        running[slot][64 * p + lane] = wave_inclusive_scan(part);
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    if ((uint32_t)lane < rows_here) {
        // row `lane` = chunks first .. last of the stream
        const uint32_t first = (uint32_t)lane * (uint32_t)nch, last = first + (uint32_t)nch - 1u;
        const float *run = running[slot];
        float sum = run[last];
        if ((first >> 6) != (last >> 6)) sum += run[(first | 63u)];            // the row started in the pass before
        if (first & 63u) sum -= run[first - 1u];
        partial[slot][lane] = wgt * sum;
    }
    TF_STAMP(2, blockIdx.x * 8 + slot, 3);
    __syncthreads();
    if (writer) {
        float acc = (float)res16;
#pragma unroll
        for (int s = 0; s < 8; ++s) acc += partial[s][threadIdx.x];
        y[row0 + threadIdx.x] = (half_t)acc;
    }
    TF_STAMP(2, blockIdx.x * 8 + slot, 4);
}

template <int SD>
__global__ __launch_bounds__(512) void phase2_generic_kernel(RoutedArg routed, tf_expert_offsets off, const half_t *acts,
                                                             const half_t *routing_w, const half_t *residual, half_t *y,
                                                             uint32_t d, uint32_t f) {
    __shared__ float partial[8];
    const int lane = threadIdx.x & 63;
    const uint32_t slot = threadIdx.x >> 6;
    const uint32_t r = blockIdx.x;
    const uint8_t *base = blob_base(routed, slot);
    const int groups = f >> 6;
    const float v = generic_row_dot<SD>(base + off.down_W_off + (size_t)r * (f >> 1), base + off.down_s_off + (size_t)r * groups * 2,
                                        base + off.down_b_off + (size_t)r * groups * 2, acts + (size_t)slot * f, f, lane);
    if (lane == 0) partial[slot] = (float)routing_w[slot] * v;
    __syncthreads();
    if (threadIdx.x == 0) {
        float acc = (float)residual[r];
#pragma unroll
        for (int s = 0; s < 8; ++s) acc += partial[s];
        y[r] = (half_t)acc;
    }
}

// ------------------------------------------------------------------------------------------------ shared expert
// gate and up tiles share the activations; both sums are rounded to fp16 (the reference's two GEMVs write fp16)
// before GeGLU (gelu_mul_fp16), and all three vectors land in the caller's scratch buffers.
struct SharedGateUpArgs {
    const uint8_t *gW, *gS, *gB, *uW, *uS, *uB;
    const half_t *x;
    half_t *gate_out, *up_out, *act_out;
    uint32_t f;
    int d;
};
template <int RT, int NP, int SD>
__device__ __forceinline__ void shared_gate_up_long_body(const SharedGateUpArgs &a, uint32_t block, u32x4 *xa, float *xsum) {
    const uint8_t *gW = a.gW, *gS = a.gS, *gB = a.gB, *uW = a.uW, *uS = a.uS, *uB = a.uB;
    const half_t *x = a.x;
    half_t *gate_out = a.gate_out, *up_out = a.up_out, *act_out = a.act_out;
    const uint32_t f = a.f;
    const int d = a.d;
    const int lane = threadIdx.x & 63;
    const uint32_t tile = uniform_u32((block * blockDim.x + threadIdx.x) >> 6);
    const uint32_t row0 = tile * RT;
    const bool live = row0 < f;
    XStage stage;
    stage.request(x, d);
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile tg, tu;
    rs.init_map(d, lane);
    if (live) {
        const size_t w_byte = (size_t)row0 * (d >> 1);
        const size_t sb_byte = (size_t)row0 * (d >> 6) * 2;
        rs.load(tg, gW + w_byte, gS + sb_byte, gB + sb_byte, f - row0);
        rs.load(tu, uW + w_byte, uS + sb_byte, uB + sb_byte, f - row0);
    }
    stage.publish(d, xa, xsum);
    if (!live) return;
    rs.init_x_lds(xa, xsum, d);
    float gate[RT], up[RT];
    rs.template reduce<SD>(tg, gate);
    rs.template reduce<SD>(tu, up);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            if (row0 + r >= f) continue;
            const half_t g16 = (half_t)gate[r], u16 = (half_t)up[r];
            gate_out[row0 + r] = g16;
            up_out[row0 + r] = u16;
            act_out[row0 + r] = (half_t)(gelu_tanh((float)g16) * (float)u16);
        }
    }
}

template <int RT, int NP, int SD>
__global__ __launch_bounds__(256) void shared_gate_up_long_kernel(SharedGateUpArgs a) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    shared_gate_up_long_body<RT, NP, SD>(a, blockIdx.x, xa, xsum);
}

// ------------------------------------------------------------------------------------------------ two stages, one launch
// The shared expert does not depend on the router or the routed experts (the reference commits it on a command buffer of its
// own).  In a chain of launches on one stream it can ride along: its gate / up rows as extra blocks of the router launch, its
// down rows as extra blocks of the routed phase 1, so that the decoder layer has two launches fewer and their work overlaps.
// A block takes one role by its index; the arithmetic of either role is that of the stand-alone kernel.
struct RouterArgs {
    const uint8_t *W, *S, *B;
    const half_t *hidden;
    const uint16_t *eff;
    float *logits;
    uint32_t num_experts;
    int d;
};
template <int RT, int NP, int SD>
__global__ __launch_bounds__(256) void router_and_shared_gate_up_kernel(RouterArgs r, SharedGateUpArgs sh) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ float partial[4];
    if (blockIdx.x < r.num_experts) {
        router_logits_block_body<0>(r.W, r.S, r.B, r.hidden, r.eff, r.logits, r.d, blockIdx.x, partial);
        return;
    }
    shared_gate_up_long_body<RT, NP, SD>(sh, blockIdx.x - r.num_experts, xa, xsum);
}

// The same launch with the post-attention setup (FusedPostAttentionSetup: residual add, the norms that make dense_x, routed_x
// and router_x) repeated by every block in its prologue instead of a launch of its own ahead of this one: a block requests
// its weights, then the attention output, the residual stream and the norm weights (27 KB out of L2), computes the two
// row reductions and keeps the one vector it multiplies with in LDS - router blocks router_x, shared-expert blocks dense_x.
// Block 0 also writes the four vectors to memory: the new residual stream and routed_x for the launches that follow, dense_x
// and router_x for the caller.  Thread t of the setup owns the same 8-element pieces as thread t of the staging code, and the
// arithmetic is PostAttnRow's, so every value equals what the stand-alone setup kernel writes.  hidden_out must not be the
// residual stream that the other blocks are still reading.
struct PostAttnFuseArgs {
    const half_t *hidden, *attn;
    half_t *hidden_out, *dense_x, *routed_x, *router_x;
    const uint16_t *w_post_attn, *w_pre_ffn, *w_pre_ffn2;
    float eps;
};
template <int RT, int NP, int SD>
__global__ __launch_bounds__(256) void post_attn_router_and_shared_gate_up_kernel(PostAttnFuseArgs pa, RouterArgs r, SharedGateUpArgs sh) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ float partial[4];
    __shared__ float norm_partial[8];
    const int d = r.d;
    const RowSlice<true> rs{(uint32_t)d};
    float at[kPerThread], w[kPerThread];
    PostAttnRow<true> pr;
    if (blockIdx.x < r.num_experts) {
        // ---- router role: thread c multiplies chunk c (16 values) of the expert's row
        const uint32_t e = blockIdx.x;
        const int c = threadIdx.x, chunks = d >> 4, groups = d >> 6;
        // the rows of the setup first: loads return in the order of their requests
        rs.load_f16(pa.attn, at);
        rs.load_bf16(pa.w_post_attn, w);
        rs.load_f16(pa.hidden, pr.h);
        float w2[kPerThread], w3[kPerThread];
        if (e == 0) {
            rs.load_bf16(pa.w_pre_ffn, w2);
            rs.load_bf16(pa.w_pre_ffn2, w3);
        }
        u32x4 wv = {0u, 0u, 0u, 0u}, ea = wv, eb = wv;
        uint16_t sv = 0, bv = 0;
        if (c < chunks) {
            wv = load16(r.W + (size_t)e * d + (size_t)c * 16);
            ea = load16(r.eff + c * 16);
            eb = load16(r.eff + c * 16 + 8);
            sv = *reinterpret_cast<const uint16_t *>(r.S + (size_t)e * groups * 2 + (c >> 2) * 2);
            bv = *reinterpret_cast<const uint16_t *>(r.B + (size_t)e * groups * 2 + (c >> 2) * 2);
        }
        pr.finish(rs, at, w, pa.eps, norm_partial);
        if (e == 0) rs.store_f16(pa.hidden_out, pr.h);
#pragma unroll
        for (int j = 0; j < kPerThread; ++j) {
            const float hn = pr.h[j] * pr.inv;
            if (e == 0) {
                w2[j] = round_half(hn * w2[j]);
                w3[j] = round_half(hn * w3[j]);
            }
            pr.h[j] = round_half(hn);
        }
        if (e == 0) {
            rs.store_f16(pa.dense_x, w2);
            rs.store_f16(pa.routed_x, w3);
            rs.store_f16(pa.router_x, pr.h);
        }
        half_t *row = reinterpret_cast<half_t *>(xa);   // router_x as a plain fp16 row
#pragma unroll
        for (int p = 0; p < 2; ++p)
            if (rs.live(8 * p)) *reinterpret_cast<u32x4 *>(row + rs.index(8 * p)) = pack_half8(pr.h + 8 * p);
        __syncthreads();
        float acc = 0.0f;
        if (c < chunks) {
            const u32x4 ha = *reinterpret_cast<const u32x4 *>(row + c * 16), hb = *reinterpret_cast<const u32x4 *>(row + c * 16 + 8);
            router_chunk(wv, ha, hb, ea, eb, sb_to_f32<0>(sv), sb_to_f32<0>(bv), acc);
        }
        acc = wave_sum(acc);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
        __syncthreads();
        if (threadIdx.x == 0) r.logits[e] = ((partial[0] + partial[1]) + partial[2]) + partial[3];
        return;
    }
    // ---- shared expert's gate / up role: shared_gate_up_long_body with dense_x made here
    const int lane = threadIdx.x & 63;
    const uint32_t tile = uniform_u32(((blockIdx.x - r.num_experts) * blockDim.x + threadIdx.x) >> 6);
    const uint32_t row0 = tile * RT;
    const bool live = row0 < sh.f;
    float w2[kPerThread];
    rs.load_f16(pa.attn, at);
    rs.load_bf16(pa.w_post_attn, w);
    rs.load_f16(pa.hidden, pr.h);
    rs.load_bf16(pa.w_pre_ffn, w2);
    RowStream<RT, NP> stream;
    typename RowStream<RT, NP>::Tile tg, tu;
    stream.init_map(d, lane);
    if (live) {
        const size_t w_byte = (size_t)row0 * (d >> 1);
        const size_t sb_byte = (size_t)row0 * (d >> 6) * 2;
        stream.load(tg, sh.gW + w_byte, sh.gS + sb_byte, sh.gB + sb_byte, sh.f - row0);
        stream.load(tu, sh.uW + w_byte, sh.uS + sb_byte, sh.uB + sb_byte, sh.f - row0);
    }
    pr.finish(rs, at, w, pa.eps, norm_partial);
#pragma unroll
    for (int j = 0; j < kPerThread; ++j) w2[j] = round_half(pr.h[j] * pr.inv * w2[j]);
#pragma unroll
    for (int p = 0; p < 2; ++p) XStage::publish_piece(pack_half8(w2 + 8 * p), threadIdx.x + 256 * p, d >> 3, d >> 5, xa, xsum);
    __syncthreads();
    if (!live) return;
    stream.init_x_lds(xa, xsum, d);
    float gate[RT], up[RT];
    stream.template reduce<SD>(tg, gate);
    stream.template reduce<SD>(tu, up);
    if (lane == 0) {
#pragma unroll
        for (int r_ = 0; r_ < RT; ++r_) {
            if (row0 + r_ >= sh.f) continue;
            const half_t g16 = (half_t)gate[r_], u16 = (half_t)up[r_];
            sh.gate_out[row0 + r_] = g16;
            sh.up_out[row0 + r_] = u16;
            sh.act_out[row0 + r_] = (half_t)(gelu_tanh((float)g16) * (float)u16);
        }
    }
}

// One RT-row tile of y = W x per wave (fp16 out): the row streamer of the GEMV entry points, one tile a wave.
struct GemvTileArgs {
    const uint8_t *W, *S, *B;
    const half_t *x;
    half_t *y;
    uint32_t m;
    int k;
};
template <int RT, int NP, int SD>
__device__ __forceinline__ void gemv_tile_body(const GemvTileArgs &a, uint32_t block, u32x4 *xa, float *xsum) {
    const int lane = threadIdx.x & 63;
    const uint32_t tile = uniform_u32((block * blockDim.x + threadIdx.x) >> 6);
    const uint32_t row0 = tile * RT;
    const bool live = row0 < a.m;
    XStage stage;
    stage.request(a.x, a.k);
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile t;
    rs.init_map(a.k, lane);
    if (live) rs.load(t, a.W + (size_t)row0 * (a.k >> 1), a.S + (size_t)row0 * (a.k >> 6) * 2, a.B + (size_t)row0 * (a.k >> 6) * 2, a.m - row0);
    stage.publish(a.k, xa, xsum);
    if (!live) return;
    rs.init_x_lds(xa, xsum, a.k);
    float out[RT];
    rs.template reduce<SD>(t, out);
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < RT; ++r)
            if (row0 + r < a.m) a.y[row0 + r] = (half_t)out[r];
    }
}
template <int RT, int NP, int SD>
__global__ __launch_bounds__(256) void phase1_and_shared_down_kernel(RoutedArg routed, tf_expert_offsets off, const half_t *x, half_t *acts,
                                                                     Phase1Geom g, FusedSelect fs, uint32_t moe_blocks, GemvTileArgs down) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ uint32_t chosen[TF_MAX_STREAMED_EXPERTS];
    __shared__ RankSelectLds sel;
    if (blockIdx.x < moe_blocks) {
        phase1_long_body<RT, NP, SD, true>(routed, off, x, acts, g, fs, blockIdx.x, xa, xsum, chosen, sel);
        return;
    }
    gemv_tile_body<RT, NP, SD>(down, blockIdx.x - moe_blocks, xa, xsum);
}

bool routed_to_arg(const tf_routed_blobs *routed, uint32_t top_k, RoutedArg &arg, bool &all16) {
    all16 = true;
    arg.pool = nullptr;
    arg.stride = 0;
    arg.indices = nullptr;
    arg.num_experts = 0;
    for (uint32_t i = 0; i < TF_MAX_STREAMED_EXPERTS; ++i) arg.blob[i] = nullptr;
    if (routed->indices) {
        if (!routed->pool || routed->num_experts == 0) return false;
        arg.pool = static_cast<const uint8_t *>(routed->pool);
        arg.stride = routed->pool_stride;
        arg.indices = routed->indices;
        arg.num_experts = routed->num_experts;
        all16 = aligned16(arg.pool) && (arg.stride % 16 == 0);
        return true;
    }
    for (uint32_t i = 0; i < top_k; ++i) {
        if (!routed->blobs[i]) return false;
        arg.blob[i] = static_cast<const uint8_t *>(routed->blobs[i]);
        all16 = all16 && aligned16(arg.blob[i]);
    }
    return true;
}

bool offsets_even(const tf_expert_offsets &o) {
    return ((o.gate_W_off | o.gate_s_off | o.gate_b_off | o.up_W_off | o.up_s_off | o.up_b_off | o.down_W_off | o.down_s_off | o.down_b_off) & 1u) == 0;
}

// fused != nullptr (decode step): the expert indices are not read from routed->indices but selected inside the
// kernel from fused->logits; returns TF_ERR_UNAVAILABLE when the operands do not allow the fused kernel.
int32_t phase1_entry(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed, const tf_expert_offsets *off, const void *x,
                     void *acts, const uint32_t *active_slots, uint32_t active_count, bool subset, uint32_t d, uint32_t f,
                     uint32_t top_k, tf_dtype sd, const FusedSelect *fused = nullptr, int mark_event = -1,
                     const GemvTileArgs *ride = nullptr, bool *ride_taken = nullptr) {
    if (ride_taken) *ride_taken = false;
    TF_REQUIRE(ctx, ctx && routed && off && x && acts, TF_ERR_INVALID_ARGUMENT, "moe_phase1: null argument");
    TF_REQUIRE(ctx, top_k == TF_MAX_STREAMED_EXPERTS, TF_ERR_INVALID_ARGUMENT, "moe_phase1: topK must be 8, got %u", top_k);
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0 && f > 0, TF_ERR_INVALID_ARGUMENT, "moe_phase1: d must be a multiple of 64 and f positive");
    TF_REQUIRE(ctx, sd == TF_BF16 || sd == TF_FP16, TF_ERR_INVALID_ARGUMENT, "moe_phase1: scale dtype must be bf16 or fp16");
    TF_REQUIRE(ctx, offsets_even(*off) && aligned(x, 2) && aligned(acts, 2), TF_ERR_INVALID_ARGUMENT, "moe_phase1: misaligned operand");
    if (subset) {
        if (active_count == 0) return TF_OK;
        TF_REQUIRE(ctx, active_slots != nullptr && active_count <= top_k, TF_ERR_INVALID_ARGUMENT, "moe_phase1_subset: bad active slots");
    }
    RoutedArg arg;
    bool all16;
    TF_REQUIRE(ctx, routed_to_arg(routed, top_k, arg, all16), TF_ERR_INVALID_ARGUMENT, "moe_phase1: routed blobs incomplete");
    Phase1Geom g{d, f, top_k, subset ? active_count : 0u, subset ? active_slots : nullptr};
    const uint32_t n_slots = subset ? active_count : top_k;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t *xh = static_cast<const half_t *>(x);
    half_t *ah = static_cast<half_t *>(acts);
    const bool fast = all16 && aligned16(x) && (off->gate_W_off % 16 == 0) && (off->up_W_off % 16 == 0);
    const int SD = sd == TF_BF16 ? 0 : 1;
    if (fused && !(fast && d > 1024 && d <= (uint32_t)XStage::kMaxK && plan_long_rows((int)d).rt > 0)) return TF_ERR_UNAVAILABLE;
    if (fast && d <= 1024) {
        constexpr int NPASS = 2;
        const uint32_t units = n_slots * ((f + 2 * NPASS - 1) / (2 * NPASS));
        const dim3 grid((units + 3) / 4);
        if (SD == 0) hipLaunchKernelGGL((phase1_short_kernel<NPASS, 0>), grid, dim3(256), 0, st, arg, *off, xh, ah, g);
        else hipLaunchKernelGGL((phase1_short_kernel<NPASS, 1>), grid, dim3(256), 0, st, arg, *off, xh, ah, g);
        return check_launch(ctx, "moe_phase1_short");
    }
    const LongPlan plan = plan_long_rows((int)d);
    const FusedSelect no_select = {nullptr, nullptr, nullptr, nullptr, 0};
    if (fast && d > 1024 && plan.rt > 0) {
        const uint32_t units = n_slots * ((f + plan.rt - 1) / plan.rt);
        const dim3 grid((units + 3) / 4);
        if (fused && mark_event >= 0 && ctx->step_timing) (void)hipEventRecord(ctx->step_events[mark_event], st);
        // the shared expert's down rows ride along as extra blocks when both row widths take the same tile shape
        if (fused && ride && plan.rt == 2 && plan.np == 3) {
            const uint32_t down_blocks = ((ride->m + 1) / 2 + 3) / 4;
            const dim3 both(grid.x + down_blocks);
            if (SD == 0) hipLaunchKernelGGL((phase1_and_shared_down_kernel<2, 3, 0>), both, dim3(256), 0, st, arg, *off, xh, ah, g, *fused, grid.x, *ride);
            else hipLaunchKernelGGL((phase1_and_shared_down_kernel<2, 3, 1>), both, dim3(256), 0, st, arg, *off, xh, ah, g, *fused, grid.x, *ride);
            if (ride_taken) *ride_taken = true;
            return check_launch(ctx, "moe_phase1_long + shared down");
        }
#define TF_P1_LAUNCH(RT_, NP_, SD_)                                                                                  \
    do {                                                                                                             \
        if (fused) hipLaunchKernelGGL((phase1_long_kernel<RT_, NP_, SD_, true>), grid, dim3(256), 0, st, arg, *off, xh, ah, g, *fused); \
        else hipLaunchKernelGGL((phase1_long_kernel<RT_, NP_, SD_, false>), grid, dim3(256), 0, st, arg, *off, xh, ah, g, no_select);    \
    } while (0)
#define TF_P1_CASE(RT_, NP_)                                                                                         \
    if (plan.rt == RT_ && plan.np == NP_) {                                                                          \
        if (SD == 0) TF_P1_LAUNCH(RT_, NP_, 0);                                                                      \
        else TF_P1_LAUNCH(RT_, NP_, 1);                                                                              \
        return check_launch(ctx, "moe_phase1_long");                                                                 \
    }
        TF_P1_CASE(1, 1) TF_P1_CASE(1, 2) TF_P1_CASE(1, 3) TF_P1_CASE(1, 4)
        TF_P1_CASE(2, 1) TF_P1_CASE(2, 2) TF_P1_CASE(2, 3) TF_P1_CASE(2, 4)
        TF_P1_CASE(4, 1) TF_P1_CASE(4, 2) TF_P1_CASE(4, 3) TF_P1_CASE(4, 4)
#undef TF_P1_CASE
#undef TF_P1_LAUNCH
    }
    const uint32_t units = n_slots * f;
    const dim3 grid((units + 3) / 4);
    if (SD == 0) hipLaunchKernelGGL((phase1_generic_kernel<0>), grid, dim3(256), 0, st, arg, *off, xh, ah, g);
    else hipLaunchKernelGGL((phase1_generic_kernel<1>), grid, dim3(256), 0, st, arg, *off, xh, ah, g);
    return check_launch(ctx, "moe_phase1_generic");
}

// ------------------------------------------------------------------------------------------------ shared expert, 8-bit
// shared_int8_gate_up_act_simd (Metal/Quant/dequant_int8.metal:100-157): one wave per row takes the gate row and the up
// row against the same activations; act[row] = half(gelu_tanh(float(half(gate))) * float(half(up))).
// A chunk = 16 weights (one byte each) against 16 activations.  The weights become fp16 pairs once (byte b -> the half
// 0x6400 | b = 1024 + b, minus 1024: exact), then every pair of products is one packed dot instruction with an fp32 sum;
// 255 * x is exact in fp32.  Expanded weights serve every activation row they meet, and the sum of a row's activations
// serves gate and up.
struct Int8Weights {
    half2_t q[8];
};
__device__ __forceinline__ Int8Weights int8_expand(const u32x4 w) {
    const half2_t bias = {(half_t)1024.0f, (half_t)1024.0f};
    Int8Weights e;
#pragma unroll
    for (int j = 0; j < 8; ++j)
        e.q[j] = as_half2(__builtin_amdgcn_perm(0x64646464u, w[j >> 1], (j & 1) ? 0x04030402u : 0x04010400u)) - bias;
    return e;
}
__device__ __forceinline__ float int8_sum(const u32x4 xa, const u32x4 xb) {
    const half2_t ones = {(half_t)1.0f, (half_t)1.0f};
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) sum = __builtin_amdgcn_fdot2(as_half2(j < 4 ? xa[j] : xb[j - 4]), ones, sum, false);
    return sum;
}
__device__ __forceinline__ void int8_chunk(const Int8Weights &e, const u32x4 xa, const u32x4 xb, float sum, float s, float b, float &acc) {
    float dot = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) dot = __builtin_amdgcn_fdot2(e.q[j], as_half2(j < 4 ? xa[j] : xb[j - 4]), dot, false);
    acc = fmaf(s, dot, acc);
    acc = fmaf(b, sum, acc);
}

// MODE > 0: 16-byte aligned rows and activations, k <= 1024 * MODE: the lane's chunks of both rows are all requested before
// the first is used.  MODE == 0: aligned, any k.  MODE < 0: any alignment (16-bit loads).
template <int SD, int MODE>
__global__ __launch_bounds__(256) void shared8_gate_up_kernel(const uint8_t *gW, const uint8_t *gS, const uint8_t *gB, const uint8_t *uW,
                                                              const uint8_t *uS, const uint8_t *uB, const half_t *x, half_t *act, uint32_t m, int k) {
    const int lane = threadIdx.x & 63;
    const uint32_t row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (row >= m) return;
    const int groups = k >> 6, chunks = k >> 4;
    const uint8_t *gw = gW + (size_t)row * k, *uw = uW + (size_t)row * k;
    const uint8_t *gs = gS + (size_t)row * groups * 2, *gb = gB + (size_t)row * groups * 2;
    const uint8_t *us = uS + (size_t)row * groups * 2, *ub = uB + (size_t)row * groups * 2;
    float gate = 0.0f, up = 0.0f;
    if constexpr (MODE > 0) {
        u32x4 wg[MODE], wu[MODE], xa[MODE], xb[MODE];
        uint16_t sg[MODE], bg[MODE], su[MODE], bu[MODE];
#pragma unroll
        for (int p = 0; p < MODE; ++p) {
            const int c = lane + 64 * p;
            wg[p] = wu[p] = xa[p] = xb[p] = u32x4{0u, 0u, 0u, 0u};
            sg[p] = bg[p] = su[p] = bu[p] = 0;
            if (c < chunks) {
                wg[p] = load16(gw + (size_t)c * 16);
                wu[p] = load16(uw + (size_t)c * 16);
                xa[p] = load16(x + c * 16);
                xb[p] = load16(x + c * 16 + 8);
                sg[p] = *reinterpret_cast<const uint16_t *>(gs + (c >> 2) * 2);
                bg[p] = *reinterpret_cast<const uint16_t *>(gb + (c >> 2) * 2);
                su[p] = *reinterpret_cast<const uint16_t *>(us + (c >> 2) * 2);
                bu[p] = *reinterpret_cast<const uint16_t *>(ub + (c >> 2) * 2);
            }
        }
#pragma unroll
        for (int p = 0; p < MODE; ++p) {
            const float sum = int8_sum(xa[p], xb[p]);
            int8_chunk(int8_expand(wg[p]), xa[p], xb[p], sum, sb_to_f32<SD>(sg[p]), sb_to_f32<SD>(bg[p]), gate);
            int8_chunk(int8_expand(wu[p]), xa[p], xb[p], sum, sb_to_f32<SD>(su[p]), sb_to_f32<SD>(bu[p]), up);
        }
        gate = wave_sum(gate);
        up = wave_sum(up);
    } else if constexpr (MODE == 0) {
        for (int c = lane; c < chunks; c += kWave) {
            const u32x4 xa = load16(x + c * 16), xb = load16(x + c * 16 + 8);
            const float sum = int8_sum(xa, xb);
            int8_chunk(int8_expand(load16(gw + (size_t)c * 16)), xa, xb, sum, sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(gs + (c >> 2) * 2)),
                       sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(gb + (c >> 2) * 2)), gate);
            int8_chunk(int8_expand(load16(uw + (size_t)c * 16)), xa, xb, sum, sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(us + (c >> 2) * 2)),
                       sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(ub + (c >> 2) * 2)), up);
        }
        gate = wave_sum(gate);
        up = wave_sum(up);
    } else {
        gate = generic_row_dot8<SD>(gw, gs, gb, x, k, lane);
        up = generic_row_dot8<SD>(uw, us, ub, x, k, lane);
    }
    if (lane == 0) {
        const half_t g16 = (half_t)gate, u16 = (half_t)up;
        act[row] = (half_t)(gelu_tanh((float)g16) * (float)u16);
    }
}

// A block of rows: a wave takes one weight row (gate and up, or one down row) against kSharedRows activation rows at a time,
// with the chunk assignment and the order of operations of the single-row kernels, so every row comes out as the single-row
// chain leaves it, bit for bit, while a weight row is fetched once per kSharedRows rows instead of once per row.
constexpr int kSharedRows = 4;

// gate / up + activation: acts[t, row]; x rows x_stride elements apart
template <int SD, int NPASS>
__global__ __launch_bounds__(256) void shared8_gate_up_rows_kernel(const uint8_t *gW, const uint8_t *gS, const uint8_t *gB, const uint8_t *uW,
                                                                   const uint8_t *uS, const uint8_t *uB, const half_t *x, uint32_t x_stride,
                                                                   half_t *acts, uint32_t m, int k, uint32_t tokens) {
    const int lane = threadIdx.x & 63;
    const uint32_t row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, t0 = blockIdx.y * kSharedRows;
    if (row >= m) return;
    const int groups = k >> 6, chunks = k >> 4;
    u32x4 wg[NPASS], wu[NPASS], xa[kSharedRows][NPASS], xb[kSharedRows][NPASS];
    float sg[NPASS], bg[NPASS], su[NPASS], bu[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int c = lane + 64 * p;
        wg[p] = wu[p] = u32x4{0u, 0u, 0u, 0u};
        uint16_t s0 = 0, b0 = 0, s1 = 0, b1 = 0;
        if (c < chunks) {
            wg[p] = load16(gW + (size_t)row * k + (size_t)c * 16);
            wu[p] = load16(uW + (size_t)row * k + (size_t)c * 16);
            s0 = *reinterpret_cast<const uint16_t *>(gS + ((size_t)row * groups + (c >> 2)) * 2);
            b0 = *reinterpret_cast<const uint16_t *>(gB + ((size_t)row * groups + (c >> 2)) * 2);
            s1 = *reinterpret_cast<const uint16_t *>(uS + ((size_t)row * groups + (c >> 2)) * 2);
            b1 = *reinterpret_cast<const uint16_t *>(uB + ((size_t)row * groups + (c >> 2)) * 2);
        }
        sg[p] = sb_to_f32<SD>(s0);
        bg[p] = sb_to_f32<SD>(b0);
        su[p] = sb_to_f32<SD>(s1);
        bu[p] = sb_to_f32<SD>(b1);
#pragma unroll
        for (int t = 0; t < kSharedRows; ++t) {
            xa[t][p] = xb[t][p] = u32x4{0u, 0u, 0u, 0u};
            if (c < chunks && t0 + t < tokens) {
                const half_t *xr = x + (size_t)(t0 + t) * x_stride + c * 16;
                xa[t][p] = load16(xr);
                xb[t][p] = load16(xr + 8);
            }
        }
    }
    Int8Weights eg[NPASS], eu[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        eg[p] = int8_expand(wg[p]);
        eu[p] = int8_expand(wu[p]);
    }
#pragma unroll
    for (int t = 0; t < kSharedRows; ++t) {
        float gate = 0.0f, up = 0.0f;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) {
            const float sum = int8_sum(xa[t][p], xb[t][p]);
            int8_chunk(eg[p], xa[t][p], xb[t][p], sum, sg[p], bg[p], gate);
            int8_chunk(eu[p], xa[t][p], xb[t][p], sum, su[p], bu[p], up);
        }
        gate = wave_sum(gate);
        up = wave_sum(up);
        if (lane == 0 && t0 + t < tokens) {
            const half_t g16 = (half_t)gate, u16 = (half_t)up;
            acts[(size_t)(t0 + t) * m + row] = (half_t)(gelu_tanh((float)g16) * (float)u16);
        }
    }
}

// down: y[t, row] = half(W[row, :] . acts[t, :]); acts rows k elements apart, y rows y_stride apart
template <int SD, int NPASS, int ROWS = kSharedRows>
__global__ __launch_bounds__(256) void gemv8_rows_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B, const half_t *acts, half_t *y,
                                                         uint32_t y_stride, uint32_t m, int k, uint32_t tokens) {
    constexpr int kSharedRows = ROWS;      // activation rows per weight row fetch (1: the single-row chain)
    const int lane = threadIdx.x & 63;
    const uint32_t row = (blockIdx.x * blockDim.x + threadIdx.x) >> 6, t0 = blockIdx.y * kSharedRows;
    if (row >= m) return;
    const int groups = k >> 6, chunks = k >> 4;
    u32x4 w[NPASS], xa[kSharedRows][NPASS], xb[kSharedRows][NPASS];
    float sv[NPASS], bv[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        const int c = lane + 64 * p;
        w[p] = u32x4{0u, 0u, 0u, 0u};
        uint16_t s0 = 0, b0 = 0;
        if (c < chunks) {
            w[p] = load16(W + (size_t)row * k + (size_t)c * 16);
            s0 = *reinterpret_cast<const uint16_t *>(S + ((size_t)row * groups + (c >> 2)) * 2);
            b0 = *reinterpret_cast<const uint16_t *>(B + ((size_t)row * groups + (c >> 2)) * 2);
        }
        sv[p] = sb_to_f32<SD>(s0);
        bv[p] = sb_to_f32<SD>(b0);
#pragma unroll
        for (int t = 0; t < kSharedRows; ++t) {
            xa[t][p] = xb[t][p] = u32x4{0u, 0u, 0u, 0u};
            if (c < chunks && t0 + t < tokens) {
                const half_t *xr = acts + (size_t)(t0 + t) * k + c * 16;
                xa[t][p] = load16(xr);
                xb[t][p] = load16(xr + 8);
            }
        }
    }
    Int8Weights e[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) e[p] = int8_expand(w[p]);
#pragma unroll
    for (int t = 0; t < kSharedRows; ++t) {
        float acc = 0.0f;
#pragma unroll
        for (int p = 0; p < NPASS; ++p) int8_chunk(e[p], xa[t][p], xb[t][p], int8_sum(xa[t][p], xb[t][p]), sv[p], bv[p], acc);
        acc = wave_sum(acc);
        if (lane == 0 && t0 + t < tokens) y[(size_t)(t0 + t) * y_stride + row] = (half_t)acc;
    }
}

bool projection_ok(const tf_projection *p) {
    return p->weights && p->scales && p->biases && p->cols % TF_GROUP_SIZE == 0 && p->cols > 0 && p->rows > 0 &&
           aligned(at(p->scales, p->scales_offset), 2) && aligned(at(p->biases, p->biases_offset), 2);
}

// Router stage 1: validates the whole router call and writes the logits into the context's scratch.
int32_t router_logits_entry(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                            uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *hidden,
                            const void *effective_scale, uint64_t effective_scale_offset, const void *per_expert_scale,
                            uint64_t per_expert_scale_offset, void *out_indices, void *out_weights, uint32_t num_experts,
                            uint32_t d, uint32_t top_k, float *logits, const SharedGateUpArgs *ride = nullptr, int ride_sd = 0,
                            bool *ride_taken = nullptr, const PostAttnFuseArgs *post = nullptr) {
    if (ride_taken) *ride_taken = false;
    TF_REQUIRE(ctx, ctx && weights && scales && biases && hidden && effective_scale && per_expert_scale && out_indices && out_weights,
               TF_ERR_INVALID_ARGUMENT, "router_gemma4: null argument");
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "router_gemma4: d must be a multiple of 64, got %u", d);
    TF_REQUIRE(ctx, num_experts > 0 && num_experts <= 256, TF_ERR_INVALID_ARGUMENT, "router_gemma4: numExperts must be in 1...256, got %u", num_experts);
    TF_REQUIRE(ctx, top_k == TF_MAX_STREAMED_EXPERTS, TF_ERR_INVALID_ARGUMENT, "router_gemma4: topK must be 8, got %u", top_k);
    const uint8_t *w = at(weights, weights_offset);
    const uint8_t *s = at(scales, scales_offset);
    const uint8_t *b = at(biases, biases_offset);
    const uint8_t *eff = at(effective_scale, effective_scale_offset);
    const uint8_t *pes = at(per_expert_scale, per_expert_scale_offset);
    TF_REQUIRE(ctx, aligned(s, 2) && aligned(b, 2) && aligned(eff, 2) && aligned(pes, 2) && aligned(hidden, 2) &&
                   aligned(out_indices, 4) && aligned(out_weights, 2),
               TF_ERR_INVALID_ARGUMENT, "router_gemma4: misaligned operand");
    const bool fast = aligned16(w) && aligned16(hidden) && aligned16(eff) && d <= 4096;
    const int npass = fast ? (int)((d / 16 + 63) / 64) : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the post-attention setup in this launch's prologue needs this launch to be the one kernel below (the caller checked)
    TF_REQUIRE(ctx, !post || (fast && ride), TF_ERR_INVALID_ARGUMENT, "router_gemma4: the fused post-attention setup does not apply to these operands");
    if (fast && ride) {
        // the shared expert's gate / up rows as extra blocks of this launch (two-row tiles of three passes: the caller checked)
        const RouterArgs ra = {w, s, b, static_cast<const half_t *>(hidden), reinterpret_cast<const uint16_t *>(eff), logits, num_experts, (int)d};
        const uint32_t shared_blocks = ((ride->f + 1) / 2 + 3) / 4;
        if (post) {
            if (ride_sd == 0) hipLaunchKernelGGL((post_attn_router_and_shared_gate_up_kernel<2, 3, 0>), dim3(num_experts + shared_blocks), dim3(256), 0, st, *post, ra, *ride);
            else hipLaunchKernelGGL((post_attn_router_and_shared_gate_up_kernel<2, 3, 1>), dim3(num_experts + shared_blocks), dim3(256), 0, st, *post, ra, *ride);
            if (ride_taken) *ride_taken = true;
            return check_launch(ctx, "post-attention setup + router_gemma4 logits + shared gate/up");
        }
        if (ride_sd == 0) hipLaunchKernelGGL((router_and_shared_gate_up_kernel<2, 3, 0>), dim3(num_experts + shared_blocks), dim3(256), 0, st, ra, *ride);
        else hipLaunchKernelGGL((router_and_shared_gate_up_kernel<2, 3, 1>), dim3(num_experts + shared_blocks), dim3(256), 0, st, ra, *ride);
        if (ride_taken) *ride_taken = true;
        return check_launch(ctx, "router_gemma4 logits + shared gate/up");
    }
    if (fast) {
        hipLaunchKernelGGL((router_logits_block_kernel<0>), dim3(num_experts), dim3(256), 0, st, w, s, b, static_cast<const half_t *>(hidden),
                           reinterpret_cast<const uint16_t *>(eff), logits, (int)d);
        return check_launch(ctx, "router_gemma4 logits");
    }
    const dim3 grid((num_experts + 3) / 4);
#define TF_ROUTER(NP_)                                                                                                        \
    hipLaunchKernelGGL((router_logits_kernel<0, NP_>), grid, dim3(256), 0, st, w, s, b, static_cast<const half_t *>(hidden),  \
                       reinterpret_cast<const uint16_t *>(eff), logits, num_experts, (int)d)
    switch (npass) {
        case 1: TF_ROUTER(1); break;
        case 2: TF_ROUTER(2); break;
        case 3: TF_ROUTER(3); break;
        case 4: TF_ROUTER(4); break;
        default: TF_ROUTER(0); break;
    }
#undef TF_ROUTER
    return check_launch(ctx, "router_gemma4 logits");
}

// Router stage 2: one wave selects from the logits.
int32_t router_select_entry(tf_ctx *ctx, tf_stream stream, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                            void *out_indices, void *out_weights, uint32_t num_experts, uint32_t top_k, const float *logits) {
    hipLaunchKernelGGL(router_select_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), logits,
                       reinterpret_cast<const uint16_t *>(at(per_expert_scale, per_expert_scale_offset)),
                       static_cast<uint32_t *>(out_indices), static_cast<half_t *>(out_weights), num_experts, top_k);
    return check_launch(ctx, "router_gemma4 select");
}

// Every precondition of the step's three stages (router, phase 1, phase 2), checked without launching anything: a refused
// step leaves every buffer as it was.  The stage entries repeat these checks when they are called on their own.
int32_t decode_step_check(tf_ctx *ctx, const void *router_weights, uint64_t router_weights_offset, const void *router_scales,
                          uint64_t router_scales_offset, const void *router_biases, uint64_t router_biases_offset, const void *router_x,
                          const void *effective_scale, uint64_t effective_scale_offset, const void *per_expert_scale,
                          uint64_t per_expert_scale_offset, const void *expert_pool, uint32_t num_experts, const tf_expert_offsets *routed_offsets,
                          const void *x, const void *acts, const void *residual, const void *y, const void *out_indices, const void *out_weights,
                          uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: null context");
    TF_REQUIRE(ctx, router_weights && router_scales && router_biases && router_x && effective_scale && per_expert_scale && expert_pool &&
                   routed_offsets && x && acts && residual && y && out_indices && out_weights,
               TF_ERR_INVALID_ARGUMENT, "moe_decode_step: null argument");
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: d must be a multiple of 64, got %u", d);
    TF_REQUIRE(ctx, f > 0 && f % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: f must be a multiple of 64, got %u", f);
    TF_REQUIRE(ctx, num_experts > 0 && num_experts <= 256, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: numExperts must be in 1...256, got %u", num_experts);
    TF_REQUIRE(ctx, top_k == TF_MAX_STREAMED_EXPERTS, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: topK must be 8, got %u", top_k);
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: scale dtype must be bf16 or fp16");
    (void)router_weights_offset;   // 8-bit weights: any byte offset
    TF_REQUIRE(ctx, aligned(at(router_scales, router_scales_offset), 2) && aligned(at(router_biases, router_biases_offset), 2) &&
                   aligned(at(effective_scale, effective_scale_offset), 2) && aligned(at(per_expert_scale, per_expert_scale_offset), 2) &&
                   aligned(router_x, 2) && aligned(out_indices, 4) && aligned(out_weights, 2) && offsets_even(*routed_offsets) && aligned(x, 2) &&
                   aligned(acts, 2) && aligned(residual, 2) && aligned(y, 2),
               TF_ERR_INVALID_ARGUMENT, "moe_decode_step: misaligned operand");
    return TF_OK;
}

// router logits -> (selection + phase 1) -> phase 2 on one stream; `logits` is the num_experts-float scratch between the launches
// The shared expert riding along with the decode step's launches (see router_and_shared_gate_up_kernel).
struct SharedRide {
    SharedGateUpArgs gate_up;
    GemvTileArgs down;
};

int32_t decode_step_impl(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                           const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                           uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                           uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                           const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                           const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                           void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype, float *logits,
                         bool may_time, const SharedRide *ride = nullptr, const PostAttnFuseArgs *post = nullptr, uint32_t stages = 3) {
    int32_t rc = decode_step_check(ctx, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                                   router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                                   per_expert_scale_offset, expert_pool, num_experts, routed_offsets, x, acts, residual, y, out_indices,
                                   out_weights, d, f, top_k, scale_dtype);
    if (rc != TF_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const bool timed = may_time && ctx->step_timing;
    auto mark = [&](int i) {
        if (timed) (void)hipEventRecord(ctx->step_events[i], st);
    };
    mark(0);
    const int ride_sd = scale_dtype == TF_BF16 ? 0 : 1;
    bool rode = false;
    rc = router_logits_entry(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset,
                                     router_biases, router_biases_offset, router_x, effective_scale, effective_scale_offset,
                                     per_expert_scale, per_expert_scale_offset, out_indices, out_weights, num_experts, d, top_k, logits,
                                     ride ? &ride->gate_up : nullptr, ride_sd, &rode, post);
    if (rc != TF_OK || stages < 2) return rc;
    if (ride && !rode) {   // the router took another kernel: the shared expert's gate / up rows get their own launch
        if (ride_sd == 0) hipLaunchKernelGGL((shared_gate_up_long_kernel<2, 3, 0>), dim3(((ride->gate_up.f + 1) / 2 + 3) / 4), dim3(256), 0, st, ride->gate_up);
        else hipLaunchKernelGGL((shared_gate_up_long_kernel<2, 3, 1>), dim3(((ride->gate_up.f + 1) / 2 + 3) / 4), dim3(256), 0, st, ride->gate_up);
        rc = check_launch(ctx, "shared_gate_up");
        if (rc != TF_OK) return rc;
    }
    tf_routed_blobs routed = {};
    routed.pool = expert_pool;
    routed.pool_stride = expert_pool_stride;
    routed.indices = static_cast<const uint32_t *>(out_indices);
    routed.num_experts = num_experts;
    // Three launches when the vector path applies: logits, phase 1 with the selection repeated by every wave, phase 2.
    const FusedSelect fused = {logits, reinterpret_cast<const uint16_t *>(at(per_expert_scale, per_expert_scale_offset)),
                               static_cast<uint32_t *>(out_indices), static_cast<half_t *>(out_weights), num_experts};
    rode = false;
    rc = phase1_entry(ctx, stream, &routed, routed_offsets, x, acts, nullptr, 0, false, d, f, top_k, scale_dtype, &fused, timed ? 1 : -1,
                      ride ? &ride->down : nullptr, &rode);
    if (ride && !rode && (rc == TF_OK || rc == TF_ERR_UNAVAILABLE)) {   // phase 1 took another kernel: the down rows get their own launch
        const int32_t rc_down = launch_gemv4(ctx, st, ride->down.W, ride->down.S, ride->down.B, ride->down.x, ride->down.y, ride->down.m,
                                             (uint32_t)ride->down.k, scale_dtype, TF_FP16);
        if (rc_down != TF_OK) return rc_down;
    }
    if (rc == TF_ERR_UNAVAILABLE) {
        rc = router_select_entry(ctx, stream, per_expert_scale, per_expert_scale_offset, out_indices, out_weights, num_experts, top_k, logits);
        if (rc != TF_OK) return rc;
        mark(1);
        rc = phase1_entry(ctx, stream, &routed, routed_offsets, x, acts, nullptr, 0, false, d, f, top_k, scale_dtype);
    }
    if (rc != TF_OK || stages < 3) return rc;
    mark(2);
    rc = tf_moe_phase2_down_reduce(ctx, stream, &routed, routed_offsets, acts, out_weights, residual, y, d, f, top_k, scale_dtype);
    mark(3);
    mark(4);
    if (timed && rc == TF_OK) ctx->step_timed = true;
    return rc;
}

}  // namespace

namespace tfk {

int32_t shared8_block(tf_ctx *ctx, hipStream_t st, const tf_projection *gate, const tf_projection *up, const tf_projection *down, const void *x,
                      uint32_t x_stride_elements, void *y, uint32_t y_stride_elements, uint32_t rows, void *acts, tf_dtype scale_dtype) {
    const uint32_t f = gate->rows, d = gate->cols;
    const uint8_t *gw = at(gate->weights, gate->weights_offset), *uw = at(up->weights, up->weights_offset);
    const uint8_t *dw = at(down->weights, down->weights_offset);
    // every chunk of every row 16-byte aligned: the single-row kernels then take the same (vector) path row by row
    const bool ok = projection_ok(gate) && projection_ok(up) && projection_ok(down) && aligned16(gw) && aligned16(uw) && aligned16(dw) &&
                    aligned16(x) && aligned16(acts) && x_stride_elements % 8 == 0 && d <= 4096 && f <= 4096 && rows <= 65535 * (uint32_t)kSharedRows &&
                    (scale_dtype == TF_BF16 || scale_dtype == TF_FP16);
    if (!ok) return TF_ERR_UNAVAILABLE;
    const uint8_t *gs = at(gate->scales, gate->scales_offset), *gb = at(gate->biases, gate->biases_offset);
    const uint8_t *us = at(up->scales, up->scales_offset), *ub = at(up->biases, up->biases_offset);
    const uint8_t *ds = at(down->scales, down->scales_offset), *db = at(down->biases, down->biases_offset);
    const half_t *xp = static_cast<const half_t *>(x);
    half_t *ap = static_cast<half_t *>(acts), *yp = static_cast<half_t *>(y);
    const uint32_t groups_of_rows = (rows + kSharedRows - 1) / kSharedRows;
    const int sd = scale_dtype == TF_BF16 ? 0 : 1;
#define TF_SH8_ROWS(SD_, NP_)                                                                                                          \
    hipLaunchKernelGGL((shared8_gate_up_rows_kernel<SD_, NP_>), dim3((f + 3) / 4, groups_of_rows), dim3(256), 0, st, gw, gs, gb, uw, us, ub, xp, \
                       x_stride_elements, ap, f, (int)d, rows)
#define TF_GEMV8_ROWS(SD_, NP_)                                                                                                        \
    hipLaunchKernelGGL((gemv8_rows_kernel<SD_, NP_>), dim3((d + 3) / 4, groups_of_rows), dim3(256), 0, st, dw, ds, db, ap, yp,         \
                       y_stride_elements, d, (int)f, rows)
#define TF_PICK(MACRO_, K_)                                                                                                            \
    do {                                                                                                                               \
        const int np = ((K_) + 1023) / 1024;                                                                                           \
        if (sd == 0) {                                                                                                                 \
            if (np == 1) MACRO_(0, 1); else if (np == 2) MACRO_(0, 2); else if (np == 3) MACRO_(0, 3); else MACRO_(0, 4);              \
        } else {                                                                                                                       \
            if (np == 1) MACRO_(1, 1); else if (np == 2) MACRO_(1, 2); else if (np == 3) MACRO_(1, 3); else MACRO_(1, 4);              \
        }                                                                                                                              \
    } while (0)
    TF_PICK(TF_SH8_ROWS, d);
    int32_t rc = check_launch(ctx, "shared_int8_gate_up_act rows");
    if (rc != TF_OK) return rc;
    TF_PICK(TF_GEMV8_ROWS, f);
#undef TF_PICK
#undef TF_GEMV8_ROWS
#undef TF_SH8_ROWS
    return check_launch(ctx, "int8 gemv rows");
}

}  // namespace tfk

extern "C" {

int32_t tf_router_gemma4(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                         uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *hidden,
                         const void *effective_scale, uint64_t effective_scale_offset, const void *per_expert_scale,
                         uint64_t per_expert_scale_offset, void *out_indices, void *out_weights, uint32_t num_experts,
                         uint32_t d, uint32_t top_k) {
    int32_t rc = router_logits_entry(ctx, stream, weights, weights_offset, scales, scales_offset, biases, biases_offset, hidden,
                                     effective_scale, effective_scale_offset, per_expert_scale, per_expert_scale_offset,
                                     out_indices, out_weights, num_experts, d, top_k, ctx ? ctx->router_logits : nullptr);
    if (rc != TF_OK) return rc;
    return router_select_entry(ctx, stream, per_expert_scale, per_expert_scale_offset, out_indices, out_weights, num_experts, top_k,
                               ctx->router_logits);
}

int32_t tf_moe_phase1_gate_up_act(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed, const tf_expert_offsets *routed_offsets,
                                  const void *x, void *acts, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    return phase1_entry(ctx, stream, routed, routed_offsets, x, acts, nullptr, 0, false, d, f, top_k, scale_dtype);
}

int32_t tf_moe_phase1_gate_up_act_subset(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed, const tf_expert_offsets *routed_offsets,
                                         const void *x, void *acts, const uint32_t *active_slots, uint32_t active_count,
                                         uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    return phase1_entry(ctx, stream, routed, routed_offsets, x, acts, active_slots, active_count, true, d, f, top_k, scale_dtype);
}

int32_t tf_moe_phase2_down_reduce(tf_ctx *ctx, tf_stream stream, const tf_routed_blobs *routed, const tf_expert_offsets *routed_offsets,
                                  const void *acts, const void *routing_weights, const void *residual, void *y, uint32_t d,
                                  uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx && routed && routed_offsets && acts && routing_weights && residual && y, TF_ERR_INVALID_ARGUMENT, "moe_phase2: null argument");
    TF_REQUIRE(ctx, top_k == TF_MAX_STREAMED_EXPERTS, TF_ERR_INVALID_ARGUMENT, "moe_phase2: topK must be 8, got %u", top_k);
    TF_REQUIRE(ctx, f > 0 && f % TF_GROUP_SIZE == 0 && d > 0, TF_ERR_INVALID_ARGUMENT, "moe_phase2: f must be a multiple of 64 and d positive");
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "moe_phase2: scale dtype must be bf16 or fp16");
    TF_REQUIRE(ctx, offsets_even(*routed_offsets) && aligned(acts, 2) && aligned(routing_weights, 2) && aligned(residual, 2) && aligned(y, 2),
               TF_ERR_INVALID_ARGUMENT, "moe_phase2: misaligned operand");
    RoutedArg arg;
    bool all16;
    TF_REQUIRE(ctx, routed_to_arg(routed, top_k, arg, all16), TF_ERR_INVALID_ARGUMENT, "moe_phase2: routed blobs incomplete");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t *ah = static_cast<const half_t *>(acts);
    const half_t *wh = static_cast<const half_t *>(routing_weights);
    const half_t *rh = static_cast<const half_t *>(residual);
    half_t *yh = static_cast<half_t *>(y);
    // acts rows start at slot * f halves: 16-byte aligned when f % 8 == 0, which f % 64 == 0 guarantees
    const bool fast = all16 && aligned16(acts) && (routed_offsets->down_W_off % 16 == 0) && f <= 1024;
    if (fast) {
        // rows per block and passes: fewest passes on the busiest CU (blocks are dealt out evenly), then fullest lanes
        const uint32_t nch = f / 32;
        int best_np = 0;
        uint32_t best_rpb = 0;
        double best_cost = 0.0;
        for (int np = 1; np <= 4; ++np) {
            const uint32_t rpb = std::min<uint32_t>((uint32_t)(64 * np) / nch, (uint32_t)kFlatMaxRows);
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
        // c / nch as a multiply and a shift, checked for every chunk position a lane can hold
        const uint32_t inv_nch = (65536u + nch - 1) / nch;
        bool inv_ok = best_np > 0;
        for (uint32_t c = 0; inv_ok && c < 64u * (uint32_t)best_np; ++c) inv_ok = ((c * inv_nch) >> 16) == c / nch;
        if (inv_ok) {
            const dim3 grid((d + best_rpb - 1) / best_rpb);
            BlobPtrs blobs;
            for (uint32_t i = 0; i < TF_MAX_STREAMED_EXPERTS; ++i) blobs.blob[i] = arg.blob[i];
#define TF_P2_FLAT(NP_, SD_)                                                                                                          \
    hipLaunchKernelGGL((phase2_flat_kernel<NP_, SD_>), grid, dim3(512), 0, st, arg.indices, arg.pool, arg.stride, ah, wh, rh, yh, d, f, \
                       best_rpb, inv_nch, arg.num_experts, *routed_offsets, blobs)
            if (scale_dtype == TF_BF16) {
                if (best_np == 1) TF_P2_FLAT(1, 0); else if (best_np == 2) TF_P2_FLAT(2, 0); else if (best_np == 3) TF_P2_FLAT(3, 0); else TF_P2_FLAT(4, 0);
            } else {
                if (best_np == 1) TF_P2_FLAT(1, 1); else if (best_np == 2) TF_P2_FLAT(2, 1); else if (best_np == 3) TF_P2_FLAT(3, 1); else TF_P2_FLAT(4, 1);
            }
#undef TF_P2_FLAT
            return check_launch(ctx, "moe_phase2_flat");
        }
        constexpr int NPASS = 4;
        const dim3 grid((d + 2 * NPASS - 1) / (2 * NPASS));
        if (scale_dtype == TF_BF16) hipLaunchKernelGGL((phase2_short_kernel<NPASS, 0>), grid, dim3(512), 0, st, arg, *routed_offsets, ah, wh, rh, yh, d, f);
        else hipLaunchKernelGGL((phase2_short_kernel<NPASS, 1>), grid, dim3(512), 0, st, arg, *routed_offsets, ah, wh, rh, yh, d, f);
        return check_launch(ctx, "moe_phase2_short");
    }
    if (scale_dtype == TF_BF16) hipLaunchKernelGGL((phase2_generic_kernel<0>), dim3(d), dim3(512), 0, st, arg, *routed_offsets, ah, wh, rh, yh, d, f);
    else hipLaunchKernelGGL((phase2_generic_kernel<1>), dim3(d), dim3(512), 0, st, arg, *routed_offsets, ah, wh, rh, yh, d, f);
    return check_launch(ctx, "moe_phase2_generic");
}

int32_t tf_moe_decode_step(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                           const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                           uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                           uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                           const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                           const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                           void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "moe_decode_step: null context");
    return decode_step_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                            router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                            per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, x, acts, residual, y,
                            out_indices, out_weights, d, f, top_k, scale_dtype, ctx->router_logits, true);
}

// include/tf_bench.h: the first `stages` launches of tf_moe_decode_step (1: router logits, 2: + selection and phase 1, 3: the step)
int32_t tf_bench_moe_decode_step_stages(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                                        const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                                        uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                                        uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                        const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                        const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                                        void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                        uint32_t stages) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "bench_moe_decode_step_stages: null context");
    TF_REQUIRE(ctx, stages >= 1 && stages <= 3, TF_ERR_INVALID_ARGUMENT, "bench_moe_decode_step_stages: stages must be 1, 2 or 3, got %u", stages);
    return decode_step_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                            router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                            per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, x, acts, residual, y,
                            out_indices, out_weights, d, f, top_k, scale_dtype, ctx->router_logits, false, nullptr, nullptr, stages);
}

int32_t tf_moe_decode_step_static(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                                  const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                                  uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                                  uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                  const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                  const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                                  void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "moe_decode_step_static: null context");
    TF_REQUIRE(ctx, num_experts <= kStaticMaxExperts, TF_ERR_SCRATCH_TOO_SMALL,
               "moe_decode_step_static: %u experts exceed the %u router logits of the static scratch", num_experts, kStaticMaxExperts);
    TF_REQUIRE(ctx, ctx->static_router_logits != nullptr, TF_ERR_DEVICE, "moe_decode_step_static: static scratch was not set up on this device");
    // every logit that is read has been written by this call's router launch, so nothing needs clearing between calls
    return decode_step_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                            router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                            per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, x, acts, residual, y,
                            out_indices, out_weights, d, f, top_k, scale_dtype, ctx->static_router_logits, false);
}

}  // extern "C"

namespace {

// tf_moe_decode_step_shared; with `post` (the post-attention setup that makes router_x, x and shared_x) the setup runs in the
// prologue of the first launch when that launch is the shared one (post->hidden_out must then differ from post->hidden),
// as a launch of its own ahead of everything otherwise.
struct PostAttnCall {
    const void *hidden, *attn;
    void *hidden_out;
    const void *w_post_attn, *w_pre_ffn, *w_pre_ffn2;
    uint64_t w_post_attn_offset, w_pre_ffn_offset, w_pre_ffn2_offset;
    float eps;
};
int32_t decode_step_shared_impl(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                                const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                                uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                                uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                                void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                const void *shared_x, const tf_projection *shared_gate, const tf_projection *shared_up,
                                const tf_projection *shared_down, void *shared_y, void *shared_scratch_gate, void *shared_scratch_up,
                                void *shared_scratch_act, const PostAttnCall *post) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "moe_decode_step_shared: null context");
    TF_REQUIRE(ctx, shared_x && shared_gate && shared_up && shared_down && shared_y && shared_scratch_gate && shared_scratch_up && shared_scratch_act,
               TF_ERR_INVALID_ARGUMENT, "moe_decode_step_shared: null shared-expert argument");
    TF_REQUIRE(ctx, shared_gate->rows == shared_up->rows && shared_gate->cols == shared_up->cols && shared_down->rows == shared_gate->cols &&
                   shared_down->cols == shared_gate->rows,
               TF_ERR_DIMENSION_MISMATCH, "SharedExpert dimension mismatch: gate=(%u,%u) up=(%u,%u) down=(%u,%u)", shared_gate->rows,
               shared_gate->cols, shared_up->rows, shared_up->cols, shared_down->rows, shared_down->cols);
    const uint32_t sf = shared_gate->rows, sdim = shared_gate->cols;
    const tf_projection *proj[3] = {shared_gate, shared_up, shared_down};
    bool proj_ok = true, proj16 = true;
    for (int i = 0; i < 3; ++i) {
        proj_ok = proj_ok && projection_ok(proj[i]) && proj[i]->rows > 0 && aligned(at(proj[i]->weights, proj[i]->weights_offset), 2);
        proj16 = proj16 && proj_ok && aligned16(at(proj[i]->weights, proj[i]->weights_offset));
    }
    TF_REQUIRE(ctx, proj_ok, TF_ERR_INVALID_ARGUMENT,
               "moe_decode_step_shared: a projection needs its three buffers, 2-byte aligned, and N a positive multiple of 64");
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "moe_decode_step_shared: scale dtype must be bf16 or fp16");
    // the shared expert rides along when its row widths take the row streamers' two-row tiles of three passes (the production
    // widths 2816 and 2112 do) and its operands the vector path; otherwise it runs first, as its own launches, same results
    const LongPlan plan_up = plan_long_rows((int)sdim), plan_down = plan_long_rows((int)sf);
    const bool ride_ok = proj16 && aligned16(shared_x) && aligned16(shared_scratch_act) && aligned(shared_scratch_gate, 2) && aligned(shared_scratch_up, 2) &&
                         aligned(shared_y, 2) && sdim > 1024 && sdim <= (uint32_t)XStage::kMaxK && sf > 1024 && sf <= (uint32_t)XStage::kMaxK &&
                         plan_up.rt == 2 && plan_up.np == 3 && plan_down.rt == 2 && plan_down.np == 3;
    // the routed step's own preconditions before anything is launched (the setup and the shared expert may run as launches
    // of their own below): a refused call leaves the residual stream and every other buffer untouched
    {
        const int32_t rc = decode_step_check(ctx, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                                             router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                                             per_expert_scale_offset, expert_pool, num_experts, routed_offsets, x, acts, residual, y, out_indices,
                                             out_weights, d, f, top_k, scale_dtype);
        if (rc != TF_OK) return rc;
    }
    // the setup inside the first launch: that launch must be the block-per-expert router with the shared rows riding along,
    // every row and norm weight must move in 16-byte pieces, and nobody may write what other blocks still read
    PostAttnFuseArgs fuse = {};
    bool fuse_ok = false;
    if (post) {
        TF_REQUIRE(ctx, post->hidden && post->attn && post->hidden_out && post->w_post_attn && post->w_pre_ffn && post->w_pre_ffn2 && router_x && x,
                   TF_ERR_INVALID_ARGUMENT, "moe_decode_step_shared_post_attn: null argument");
        TF_REQUIRE(ctx, sdim == d, TF_ERR_DIMENSION_MISMATCH, "moe_decode_step_shared_post_attn: the shared expert reads %u values, the layer has %u", sdim, d);
        fuse = {static_cast<const half_t *>(post->hidden), static_cast<const half_t *>(post->attn), static_cast<half_t *>(post->hidden_out),
                static_cast<half_t *>(const_cast<void *>(shared_x)), static_cast<half_t *>(const_cast<void *>(x)),
                static_cast<half_t *>(const_cast<void *>(router_x)),
                reinterpret_cast<const uint16_t *>(at(post->w_post_attn, post->w_post_attn_offset)),
                reinterpret_cast<const uint16_t *>(at(post->w_pre_ffn, post->w_pre_ffn_offset)),
                reinterpret_cast<const uint16_t *>(at(post->w_pre_ffn2, post->w_pre_ffn2_offset)), post->eps};
        // four output rows and two input rows of d halves each: no output may overlap an input or another output
        const void *rows[6] = {fuse.hidden_out, fuse.dense_x, fuse.routed_x, fuse.router_x, fuse.hidden, fuse.attn};
        const uintptr_t row_bytes = (uintptr_t)d * 2;
        bool distinct = true;
        for (int i = 0; i < 4; ++i)
            for (int j = i + 1; j < 6; ++j) {
                const uintptr_t a = (uintptr_t)rows[i], b = (uintptr_t)rows[j];
                distinct = distinct && (a + row_bytes <= b || b + row_bytes <= a);
            }
        const bool router_fast = router_weights && effective_scale && aligned16(at(router_weights, router_weights_offset)) &&
                                 aligned16(at(effective_scale, effective_scale_offset)) && d <= 4096 && d % TF_GROUP_SIZE == 0 && num_experts > 0 &&
                                 num_experts <= 256;
        fuse_ok = ride_ok && router_fast && distinct && aligned16(fuse.hidden) && aligned16(fuse.attn) && aligned16(fuse.hidden_out) &&
                  aligned16(fuse.dense_x) && aligned16(fuse.routed_x) && aligned16(fuse.router_x) && aligned16(fuse.w_post_attn) &&
                  aligned16(fuse.w_pre_ffn) && aligned16(fuse.w_pre_ffn2);
        if (!fuse_ok) {
            const int32_t rc = post_attn_setup_to(ctx, stream, post->hidden, post->hidden_out, post->attn, const_cast<void *>(shared_x), const_cast<void *>(x),
                                                  const_cast<void *>(router_x), post->w_post_attn, post->w_post_attn_offset, post->w_pre_ffn,
                                                  post->w_pre_ffn_offset, post->w_pre_ffn2, post->w_pre_ffn2_offset, d, post->eps);
            if (rc != TF_OK) return rc;
        }
    }
    if (!ride_ok) {
        const int32_t rc = tf_shared_expert_int4(ctx, stream, shared_x, 0, (uint64_t)sdim * 2, shared_gate, shared_up, shared_down, shared_y, 0,
                                                 (uint64_t)sdim * 2, shared_scratch_gate, 0, (uint64_t)sf * 2, shared_scratch_up, 0, (uint64_t)sf * 2,
                                                 shared_scratch_act, 0, (uint64_t)sf * 2, 4, scale_dtype);
        if (rc != TF_OK) return rc;
        return decode_step_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                                router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                                per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, x, acts, residual, y,
                                out_indices, out_weights, d, f, top_k, scale_dtype, ctx->router_logits, true);
    }
    SharedRide ride;
    ride.gate_up = {at(shared_gate->weights, shared_gate->weights_offset), at(shared_gate->scales, shared_gate->scales_offset),
                    at(shared_gate->biases, shared_gate->biases_offset), at(shared_up->weights, shared_up->weights_offset),
                    at(shared_up->scales, shared_up->scales_offset), at(shared_up->biases, shared_up->biases_offset),
                    static_cast<const half_t *>(shared_x), static_cast<half_t *>(shared_scratch_gate), static_cast<half_t *>(shared_scratch_up),
                    static_cast<half_t *>(shared_scratch_act), sf, (int)sdim};
    ride.down = {at(shared_down->weights, shared_down->weights_offset), at(shared_down->scales, shared_down->scales_offset),
                 at(shared_down->biases, shared_down->biases_offset), static_cast<const half_t *>(shared_scratch_act), static_cast<half_t *>(shared_y),
                 shared_down->rows, (int)shared_down->cols};
    return decode_step_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                            router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                            per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, x, acts, residual, y,
                            out_indices, out_weights, d, f, top_k, scale_dtype, ctx->router_logits, true, &ride, fuse_ok ? &fuse : nullptr);
}

}  // namespace

extern "C" {

int32_t tf_moe_decode_step_shared(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                                  const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                                  uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                                  uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                  const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                  const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                                  void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                  const void *shared_x, const tf_projection *shared_gate, const tf_projection *shared_up,
                                  const tf_projection *shared_down, void *shared_y, void *shared_scratch_gate, void *shared_scratch_up,
                                  void *shared_scratch_act) {
    return decode_step_shared_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                                   router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                                   per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, x, acts, residual, y,
                                   out_indices, out_weights, d, f, top_k, scale_dtype, shared_x, shared_gate, shared_up, shared_down, shared_y,
                                   shared_scratch_gate, shared_scratch_up, shared_scratch_act, nullptr);
}

int32_t tf_moe_decode_step_shared_post_attn(tf_ctx *ctx, tf_stream stream, const void *hidden, const void *attn, void *hidden_out,
                                            const void *post_attention_weight, uint64_t post_attention_weight_offset,
                                            const void *pre_ffn_weight, uint64_t pre_ffn_weight_offset, const void *pre_ffn2_weight,
                                            uint64_t pre_ffn2_weight_offset, float eps, const void *router_weights,
                                            uint64_t router_weights_offset, const void *router_scales, uint64_t router_scales_offset,
                                            const void *router_biases, uint64_t router_biases_offset, void *router_x,
                                            const void *effective_scale, uint64_t effective_scale_offset, const void *per_expert_scale,
                                            uint64_t per_expert_scale_offset, const void *expert_pool, uint64_t expert_pool_stride,
                                            uint32_t num_experts, const tf_expert_offsets *routed_offsets, void *routed_x, void *acts,
                                            const void *residual, void *y, void *out_indices, void *out_weights, uint32_t d, uint32_t f,
                                            uint32_t top_k, tf_dtype scale_dtype, void *dense_x, const tf_projection *shared_gate,
                                            const tf_projection *shared_up, const tf_projection *shared_down, void *shared_y,
                                            void *shared_scratch_gate, void *shared_scratch_up, void *shared_scratch_act) {
    const PostAttnCall post = {hidden, attn, hidden_out, post_attention_weight, pre_ffn_weight, pre_ffn2_weight, post_attention_weight_offset,
                               pre_ffn_weight_offset, pre_ffn2_weight_offset, eps};
    return decode_step_shared_impl(ctx, stream, router_weights, router_weights_offset, router_scales, router_scales_offset, router_biases,
                                   router_biases_offset, router_x, effective_scale, effective_scale_offset, per_expert_scale,
                                   per_expert_scale_offset, expert_pool, expert_pool_stride, num_experts, routed_offsets, routed_x, acts, residual, y,
                                   out_indices, out_weights, d, f, top_k, scale_dtype, dense_x, shared_gate, shared_up, shared_down, shared_y,
                                   shared_scratch_gate, shared_scratch_up, shared_scratch_act, &post);
}

int32_t tf_shared_expert_int4(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, uint64_t x_length,
                              const tf_projection *gate, const tf_projection *up, const tf_projection *down, void *y,
                              uint64_t y_offset, uint64_t y_length, void *scratch_gate, uint64_t scratch_gate_offset,
                              uint64_t scratch_gate_length, void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                              void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length, uint32_t weight_bits,
                              tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "shared_expert: null context");
    // SharedExpertRuntime (SharedExpertInt4.swift:96-137): 8-bit weights take the 8-bit wrapper, which needs scratchAct only
    if (weight_bits == 8)
        return tf_shared_expert_int8(ctx, stream, x, x_offset, x_length, gate, up, down, y, y_offset, y_length, scratch_act, scratch_act_offset,
                                     scratch_act_length, scale_dtype);
    TF_REQUIRE(ctx, weight_bits == 4, TF_ERR_UNSUPPORTED_BITS, "SharedExpert unsupported weight bits: %u", weight_bits);
    TF_REQUIRE(ctx, x && gate && up && down && y && scratch_gate && scratch_up && scratch_act, TF_ERR_INVALID_ARGUMENT, "shared_expert: null argument");
    TF_REQUIRE(ctx, gate->rows == up->rows && gate->cols == up->cols && down->rows == gate->cols && down->cols == gate->rows,
               TF_ERR_DIMENSION_MISMATCH, "SharedExpert dimension mismatch: gate=(%u,%u) up=(%u,%u) down=(%u,%u)", gate->rows,
               gate->cols, up->rows, up->cols, down->rows, down->cols);
    const uint64_t required = (uint64_t)gate->rows * 2;
    TF_REQUIRE(ctx, scratch_gate_offset + required <= scratch_gate_length && scratch_up_offset + required <= scratch_up_length &&
                   scratch_act_offset + required <= scratch_act_length,
               TF_ERR_SCRATCH_TOO_SMALL, "SharedExpert scratch too small: need %llu bytes per intermediate buffer", (unsigned long long)required);
    TF_REQUIRE(ctx, x_offset + (uint64_t)gate->cols * 2 <= x_length, TF_ERR_SCRATCH_TOO_SMALL, "SharedExpert scratch too small: input range exceeds x buffer");
    TF_REQUIRE(ctx, y_offset + (uint64_t)down->rows * 2 <= y_length, TF_ERR_SCRATCH_TOO_SMALL, "SharedExpert scratch too small: output range exceeds y buffer");
    const tf_projection *proj[3] = {gate, up, down};
    for (int i = 0; i < 3; ++i) {
        TF_REQUIRE(ctx, proj[i]->weights && proj[i]->scales && proj[i]->biases, TF_ERR_INVALID_ARGUMENT, "shared_expert: null projection buffer");
        TF_REQUIRE(ctx, proj[i]->cols % TF_GROUP_SIZE == 0 && proj[i]->cols > 0 && proj[i]->rows > 0, TF_ERR_INVALID_ARGUMENT,
                   "shared_expert: N must be a multiple of 64");
        TF_REQUIRE(ctx, aligned(at(proj[i]->weights, proj[i]->weights_offset), 2) && aligned(at(proj[i]->scales, proj[i]->scales_offset), 2) &&
                       aligned(at(proj[i]->biases, proj[i]->biases_offset), 2),
                   TF_ERR_INVALID_ARGUMENT, "shared_expert: projection offsets must be 2-byte aligned");
    }
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "shared_expert: scale dtype must be bf16 or fp16");
    TF_REQUIRE(ctx, x_offset % 2 == 0 && y_offset % 2 == 0 && scratch_gate_offset % 2 == 0 && scratch_up_offset % 2 == 0 && scratch_act_offset % 2 == 0,
               TF_ERR_INVALID_ARGUMENT, "shared_expert: offsets must be 2-byte aligned");

    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint8_t *xp = at(x, x_offset);
    uint8_t *sg = at(scratch_gate, scratch_gate_offset), *su = at(scratch_up, scratch_up_offset), *sa = at(scratch_act, scratch_act_offset);
    const uint8_t *gw = at(gate->weights, gate->weights_offset), *uw = at(up->weights, up->weights_offset);
    const uint32_t f = gate->rows, d = gate->cols;
    const LongPlan plan = plan_long_rows((int)d);
    const bool fused = d > 1024 && plan.rt > 0 && aligned16(gw) && aligned16(uw) && aligned16(xp);
    int32_t rc = TF_OK;
    if (fused) {
        const uint32_t tiles = (f + plan.rt - 1) / plan.rt;
        const dim3 grid((tiles + 3) / 4);
        const uint8_t *gs = at(gate->scales, gate->scales_offset), *gb = at(gate->biases, gate->biases_offset);
        const uint8_t *us = at(up->scales, up->scales_offset), *ub = at(up->biases, up->biases_offset);
        bool launched = false;
        const SharedGateUpArgs sga = {gw, gs, gb, uw, us, ub, reinterpret_cast<const half_t *>(xp), reinterpret_cast<half_t *>(sg),
                                      reinterpret_cast<half_t *>(su), reinterpret_cast<half_t *>(sa), f, (int)d};
#define TF_SH_CASE(RT_, NP_)                                                                                                    \
    if (!launched && plan.rt == RT_ && plan.np == NP_) {                                                                        \
        launched = true;                                                                                                        \
        if (scale_dtype == TF_BF16) hipLaunchKernelGGL((shared_gate_up_long_kernel<RT_, NP_, 0>), grid, dim3(256), 0, st, sga); \
        else hipLaunchKernelGGL((shared_gate_up_long_kernel<RT_, NP_, 1>), grid, dim3(256), 0, st, sga);                        \
    }
        TF_SH_CASE(1, 1) TF_SH_CASE(1, 2) TF_SH_CASE(1, 3) TF_SH_CASE(1, 4)
        TF_SH_CASE(2, 1) TF_SH_CASE(2, 2) TF_SH_CASE(2, 3) TF_SH_CASE(2, 4)
        TF_SH_CASE(4, 1) TF_SH_CASE(4, 2) TF_SH_CASE(4, 3) TF_SH_CASE(4, 4)
#undef TF_SH_CASE
        rc = check_launch(ctx, "shared_gate_up");
        if (rc != TF_OK) return rc;
    } else {
        rc = launch_gemv4(ctx, st, gw, at(gate->scales, gate->scales_offset), at(gate->biases, gate->biases_offset), xp, sg, f, d, scale_dtype, TF_FP16);
        if (rc != TF_OK) return rc;
        rc = launch_gemv4(ctx, st, uw, at(up->scales, up->scales_offset), at(up->biases, up->biases_offset), xp, su, f, d, scale_dtype, TF_FP16);
        if (rc != TF_OK) return rc;
        rc = launch_gelu_mul(ctx, st, sg, su, sa, f);
        if (rc != TF_OK) return rc;
    }
    return launch_gemv4(ctx, st, at(down->weights, down->weights_offset), at(down->scales, down->scales_offset),
                        at(down->biases, down->biases_offset), sa, at(y, y_offset), down->rows, down->cols, scale_dtype, TF_FP16);
}

int32_t tf_shared_expert_int8_phase1(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, uint64_t x_length, const tf_projection *gate,
                                     const tf_projection *up, void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length,
                                     tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: null context");
    TF_REQUIRE(ctx, x && gate && up && scratch_act, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: null argument");
    TF_REQUIRE(ctx, gate->rows == up->rows && gate->cols == up->cols, TF_ERR_DIMENSION_MISMATCH,
               "SharedExpertInt8 dimension mismatch: gate/up shapes differ: gate=(%u,%u) up=(%u,%u)", gate->rows, gate->cols, up->rows, up->cols);
    TF_REQUIRE(ctx, scratch_act_offset + (uint64_t)gate->rows * 2 <= scratch_act_length, TF_ERR_SCRATCH_TOO_SMALL,
               "SharedExpertInt8 scratch too small: scratchAct offset %llu + needed %llu exceeds length %llu", (unsigned long long)scratch_act_offset,
               (unsigned long long)gate->rows * 2, (unsigned long long)scratch_act_length);
    TF_REQUIRE(ctx, x_offset + (uint64_t)gate->cols * 2 <= x_length, TF_ERR_SCRATCH_TOO_SMALL,
               "SharedExpertInt8 scratch too small: x offset %llu + needed %llu exceeds length %llu", (unsigned long long)x_offset,
               (unsigned long long)gate->cols * 2, (unsigned long long)x_length);
    TF_REQUIRE(ctx, projection_ok(gate) && projection_ok(up), TF_ERR_INVALID_ARGUMENT,
               "shared_expert_int8: a projection needs its three buffers, 2-byte aligned scales and biases, and N a multiple of 64");
    TF_REQUIRE(ctx, scale_dtype == TF_BF16 || scale_dtype == TF_FP16, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: scale dtype must be bf16 or fp16");
    TF_REQUIRE(ctx, x_offset % 2 == 0 && scratch_act_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: offsets must be 2-byte aligned");
    const uint8_t *gw = at(gate->weights, gate->weights_offset), *uw = at(up->weights, up->weights_offset);
    const uint8_t *gs = at(gate->scales, gate->scales_offset), *gb = at(gate->biases, gate->biases_offset);
    const uint8_t *us = at(up->scales, up->scales_offset), *ub = at(up->biases, up->biases_offset);
    const half_t *xp = reinterpret_cast<const half_t *>(at(x, x_offset));
    half_t *act = reinterpret_cast<half_t *>(at(scratch_act, scratch_act_offset));
    const uint32_t m = gate->rows, k = gate->cols;
    const bool fast = aligned16(gw) && aligned16(uw) && aligned16(xp);   // k % 64 == 0 keeps every row aligned
    const int mode = !fast ? -1 : k <= 1024 ? 1 : k <= 2048 ? 2 : k <= 3072 ? 3 : k <= 4096 ? 4 : 0;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const dim3 grid((m + 3) / 4);
#define TF_SH8(MODE_)                                                                                                                  \
    case MODE_:                                                                                                                        \
        if (scale_dtype == TF_BF16)                                                                                                    \
            hipLaunchKernelGGL((shared8_gate_up_kernel<0, MODE_>), grid, dim3(256), 0, st, gw, gs, gb, uw, us, ub, xp, act, m, (int)k); \
        else                                                                                                                           \
            hipLaunchKernelGGL((shared8_gate_up_kernel<1, MODE_>), grid, dim3(256), 0, st, gw, gs, gb, uw, us, ub, xp, act, m, (int)k); \
        break;
    switch (mode) {
        TF_SH8(1) TF_SH8(2) TF_SH8(3) TF_SH8(4) TF_SH8(0)
        default:
            if (scale_dtype == TF_BF16)
                hipLaunchKernelGGL((shared8_gate_up_kernel<0, -1>), grid, dim3(256), 0, st, gw, gs, gb, uw, us, ub, xp, act, m, (int)k);
            else
                hipLaunchKernelGGL((shared8_gate_up_kernel<1, -1>), grid, dim3(256), 0, st, gw, gs, gb, uw, us, ub, xp, act, m, (int)k);
            break;
    }
#undef TF_SH8
    return check_launch(ctx, "shared_int8_gate_up_act");
}

int32_t tf_shared_expert_int8_down(tf_ctx *ctx, tf_stream stream, const tf_projection *down, void *y, uint64_t y_offset, uint64_t y_length,
                                   const void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: null context");
    TF_REQUIRE(ctx, down && y && scratch_act, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: null argument");
    TF_REQUIRE(ctx, scratch_act_offset + (uint64_t)down->cols * 2 <= scratch_act_length, TF_ERR_SCRATCH_TOO_SMALL,
               "SharedExpertInt8 scratch too small: scratchAct offset %llu + needed %llu exceeds length %llu", (unsigned long long)scratch_act_offset,
               (unsigned long long)down->cols * 2, (unsigned long long)scratch_act_length);
    TF_REQUIRE(ctx, y_offset + (uint64_t)down->rows * 2 <= y_length, TF_ERR_SCRATCH_TOO_SMALL,
               "SharedExpertInt8 scratch too small: y offset %llu + needed %llu exceeds length %llu", (unsigned long long)y_offset,
               (unsigned long long)down->rows * 2, (unsigned long long)y_length);
    // aligned operands: the row kernel of the block form with one row, so a block equals its rows one by one bit for bit
    const uint8_t *dw = at(down->weights, down->weights_offset);
    const half_t *ap = reinterpret_cast<const half_t *>(at(scratch_act, scratch_act_offset));
    if (projection_ok(down) && aligned16(dw) && aligned16(ap) && down->cols <= 4096 && y_offset % 2 == 0 &&
        (scale_dtype == TF_BF16 || scale_dtype == TF_FP16)) {
        const uint8_t *ds = at(down->scales, down->scales_offset), *db = at(down->biases, down->biases_offset);
        half_t *yp = reinterpret_cast<half_t *>(at(y, y_offset));
        hipStream_t st = static_cast<hipStream_t>(stream);
        const uint32_t m = down->rows, k = down->cols;
        const int np = (int)((k + 1023) / 1024);
#define TF_DOWN8(SD_, NP_) hipLaunchKernelGGL((gemv8_rows_kernel<SD_, NP_, 1>), dim3((m + 3) / 4, 1), dim3(256), 0, st, dw, ds, db, ap, yp, m, m, (int)k, 1u)
        if (scale_dtype == TF_BF16) {
            if (np == 1) TF_DOWN8(0, 1); else if (np == 2) TF_DOWN8(0, 2); else if (np == 3) TF_DOWN8(0, 3); else TF_DOWN8(0, 4);
        } else {
            if (np == 1) TF_DOWN8(1, 1); else if (np == 2) TF_DOWN8(1, 2); else if (np == 3) TF_DOWN8(1, 3); else TF_DOWN8(1, 4);
        }
#undef TF_DOWN8
        return check_launch(ctx, "shared_int8_down");
    }
    return tf_dequant_int8_gemv(ctx, stream, down->weights, down->weights_offset, down->scales, down->scales_offset, down->biases,
                                down->biases_offset, scratch_act, scratch_act_offset, y, y_offset, down->rows, down->cols, scale_dtype, TF_FP16);
}

int32_t tf_shared_expert_int8(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, uint64_t x_length, const tf_projection *gate,
                              const tf_projection *up, const tf_projection *down, void *y, uint64_t y_offset, uint64_t y_length,
                              void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: null context");
    TF_REQUIRE(ctx, x && gate && up && down && y && scratch_act, TF_ERR_INVALID_ARGUMENT, "shared_expert_int8: null argument");
    TF_REQUIRE(ctx, gate->rows == up->rows && gate->cols == up->cols, TF_ERR_DIMENSION_MISMATCH,
               "SharedExpertInt8 dimension mismatch: gate/up shapes differ: gate=(%u,%u) up=(%u,%u)", gate->rows, gate->cols, up->rows, up->cols);
    TF_REQUIRE(ctx, down->rows == gate->cols && down->cols == gate->rows, TF_ERR_DIMENSION_MISMATCH,
               "SharedExpertInt8 dimension mismatch: down expected (%u,%u), got (%u,%u)", gate->cols, gate->rows, down->rows, down->cols);
    TF_REQUIRE(ctx, y_offset + (uint64_t)down->rows * 2 <= y_length, TF_ERR_SCRATCH_TOO_SMALL,
               "SharedExpertInt8 scratch too small: y offset %llu + needed %llu exceeds length %llu", (unsigned long long)y_offset,
               (unsigned long long)down->rows * 2, (unsigned long long)y_length);
    const int32_t rc = tf_shared_expert_int8_phase1(ctx, stream, x, x_offset, x_length, gate, up, scratch_act, scratch_act_offset,
                                                    scratch_act_length, scale_dtype);
    if (rc != TF_OK) return rc;
    return tf_shared_expert_int8_down(ctx, stream, down, y, y_offset, y_length, scratch_act, scratch_act_offset, scratch_act_length, scale_dtype);
}


}  // extern "C"

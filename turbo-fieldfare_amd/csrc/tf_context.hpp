// Host-side context shared by the C ABI entry points (not part of the public header).
#pragma once

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/tf_kernels.h"

struct tf_ctx {
    int device = 0;
    int num_cus = 0;
    int stream_blocks_per_cu = 2;       // 256-thread blocks per CU launched by the persistent row streamers
    // wrapper-owned scratch, as the reference's kernel classes own theirs
    float *router_logits = nullptr;     // 256 floats (MoE.swift:92-99)
    float *static_router_logits = nullptr;   // this device's copy of the load-time scratch of tf_moe_decode_step_static
    void *head_x_normed = nullptr;      // kMaxHeadD halves (LMHeadChainInt4.swift:38-51)
    float *head_summaries = nullptr;    // kMaxHeadWaves x {value, index bits}
    float *head_logits = nullptr;       // fp32 logits of the unaligned lm_head path, limits.max_vocab of them
    size_t head_logits_count = 0;
    uint32_t *group_scratch = nullptr;  // kGroupSegments x 256 per-segment expert counts of the device pair grouping
    uint8_t *few_scratch = nullptr;     // kFewScratchBytes: sorted pairs, per-expert tables and work list of tf_prefill_routed_moe_few_tokens
    float *prefill_logits = nullptr;    // [tokens, experts] router logits (+ partial planes) of the multi-token router
    size_t prefill_logits_count = 0;
    void *sample_scratch = nullptr;     // argmax cells, softmax partials, top-k pair buffers of the samplers
    size_t sample_scratch_bytes = 0;
    void *shared_block_acts = nullptr;  // [rows, intermediate] fp16 activations of the block shared expert
    size_t shared_block_acts_bytes = 0;
    void *attn_scratch = nullptr;       // split-KV partial states of decode and block attention (m, d, o per head and chunk)
    size_t attn_scratch_bytes = 0;
    // what the five buffers above are sized for; only tf_ctx_create and tf_ctx_reserve allocate them
    tf_scratch_limits limits = {0, 0, 0, 0, 0, 0, 0};
    // optional device-time bracketing of the decode step's three launches
    bool step_timing = false;
    bool step_timed = false;            // a step has been recorded since timing was enabled
    hipEvent_t step_events[5] = {nullptr, nullptr, nullptr, nullptr, nullptr};
    char last_error[512] = {0};
};

namespace tfk {

constexpr uint32_t kMaxHeadD = 16384;
constexpr uint32_t kMaxHeadWaves = 16384;
constexpr uint32_t kGroupSegments = 64;   // token segments the device pair grouping counts and places independently
// what tf_prefill_routed_moe_few_tokens keeps between its launches when it runs the grouped kernels: up to 256 sorted pairs
// (16 bytes each), per-expert offsets and counts (256 x 4 bytes each), a work list of up to 264 chunks (12 bytes each), its length
constexpr uint32_t kFewScratchPairs = 256, kFewScratchChunks = 264;
constexpr size_t kFewScratchBytes = (size_t)kFewScratchPairs * 16 + 2 * 256 * 4 + (size_t)kFewScratchChunks * 12 + 16;

inline int32_t fail(tf_ctx *ctx, int32_t status, const char *fmt, ...) {
    if (ctx) {
        va_list ap;
        va_start(ap, fmt);
        vsnprintf(ctx->last_error, sizeof(ctx->last_error), fmt, ap);
        va_end(ap);
    }
    return status;
}

inline int32_t check_launch(tf_ctx *ctx, const char *what) {
    const hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "%s: %s", what, hipGetErrorString(e));
    return TF_OK;
}

inline const uint8_t *at(const void *base, uint64_t off) { return static_cast<const uint8_t *>(base) + off; }
inline uint8_t *at(void *base, uint64_t off) { return static_cast<uint8_t *>(base) + off; }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline bool aligned(const void *p, unsigned a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1u)) == 0; }

// Wrapper scratch is sized once (tf_ctx_create, tf_ctx_reserve); an entry point that finds it too small enqueues nothing.
inline int32_t scratch_too_small(tf_ctx *ctx, const char *who, size_t need, size_t have) {
    return fail(ctx, TF_ERR_SCRATCH_TOO_SMALL, "%s: needs %zu bytes of wrapper scratch, the context holds %zu: raise the limits with tf_ctx_reserve",
                who, need, have);
}

// Looks up this device's copy of the load-time router-logit scratch (tf_moe.hip); the context's device must be current.
int32_t moe_static_scratch_setup(tf_ctx *ctx);

// Sizes of the wrapper scratch as functions of the limits, each defined beside the entry points that use the buffer.
size_t sample_scratch_bytes_for(uint32_t vocab);                                    // tf_sampling.hip
size_t sample_scratch_clear_bytes();                                                // leading bytes that must start at zero
size_t prefill_logits_floats_for(uint32_t tokens, uint32_t experts);                // tf_prefill.hip
size_t attention_scratch_floats_for(int num_cus, uint32_t q_heads, uint32_t head_dim, uint32_t block_tokens);   // tf_attention.hip

// The 8-bit shared expert over a block of rows (tf_moe.hip), for the block entry of the shared expert (tf_qmm.hip): two
// launches, every row bit-identical to the single-row chain.  acts: [rows, intermediate] fp16 scratch.  TF_ERR_UNAVAILABLE when
// the operands do not allow it (alignment, K > 4096): the caller runs the rows one by one.
int32_t shared8_block(tf_ctx *ctx, hipStream_t st, const tf_projection *gate, const tf_projection *up, const tf_projection *down, const void *x,
                      uint32_t x_stride_elements, void *y, uint32_t y_stride_elements, uint32_t rows, void *acts, tf_dtype scale_dtype);

}  // namespace tfk

#define TF_REQUIRE(ctx, cond, status, ...) \
    do {                                    \
        if (!(cond)) return tfk::fail((ctx), (status), __VA_ARGS__); \
    } while (0)

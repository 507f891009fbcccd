// Context lifetime, error strings and stream synchronisation of the C ABI.
#include "tf_context.hpp"

#include <stdlib.h>

#include <new>

using namespace tfk;

extern "C" {

uint32_t tf_abi_version(void) { return 1u; }

const char *tf_status_string(int32_t status) {
    switch (status) {
        case TF_OK: return "ok";
        case TF_ERR_INVALID_ARGUMENT: return "invalid argument";
        case TF_ERR_UNAVAILABLE: return "unavailable for this shape or alignment";
        case TF_ERR_DIMENSION_MISMATCH: return "dimension mismatch";
        case TF_ERR_SCRATCH_TOO_SMALL: return "scratch too small";
        case TF_ERR_UNSUPPORTED_BITS: return "unsupported weight bits";
        case TF_ERR_NO_DEVICE: return "no device";
        case TF_ERR_DEVICE: return "device error";
        case TF_ERR_OUT_OF_MEMORY: return "out of device memory";
        default: return "unknown status";
    }
}

const char *tf_last_error(const tf_ctx *ctx) { return ctx ? ctx->last_error : "null context"; }

int32_t tf_ctx_create(int32_t device, tf_ctx **out_ctx) {
    if (!out_ctx) return TF_ERR_INVALID_ARGUMENT;
    *out_ctx = nullptr;
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count <= 0 || device < 0 || device >= count) return TF_ERR_NO_DEVICE;
    if (hipSetDevice(device) != hipSuccess) return TF_ERR_NO_DEVICE;
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return TF_ERR_NO_DEVICE;
    tf_ctx *ctx = new (std::nothrow) tf_ctx();
    if (!ctx) return TF_ERR_OUT_OF_MEMORY;
    ctx->device = device;
    ctx->num_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    bool ok = hipMalloc(&ctx->router_logits, 256 * sizeof(float)) == hipSuccess;
    ok = ok && hipMemset(ctx->router_logits, 0, 256 * sizeof(float)) == hipSuccess;
    ok = ok && hipMalloc(&ctx->head_x_normed, kMaxHeadD * 2) == hipSuccess;
    // argmax summaries + 64 64-bit argmax cells and a ticket counter behind them (start at 0; every call leaves them at 0)
    const size_t summary_bytes = ((size_t)kMaxHeadWaves * 2 + 128 + 4) * sizeof(float);
    ok = ok && hipMalloc(&ctx->head_summaries, summary_bytes) == hipSuccess;
    ok = ok && hipMemset(ctx->head_summaries, 0, summary_bytes) == hipSuccess;
    ok = ok && hipMalloc(&ctx->group_scratch, (size_t)kGroupSegments * 256 * sizeof(uint32_t)) == hipSuccess;
    ok = ok && hipMalloc(&ctx->few_scratch, kFewScratchBytes) == hipSuccess;
    // the reference's model (Infrastructure/ModelIO/ModelTypes.swift:78-100) at the largest block sizes this library is run at
    const tf_scratch_limits defaults = {262144u, 2048u, 256u, 2112u, 16u, 512u, 128u};
    ok = ok && tf_ctx_reserve(ctx, &defaults) == TF_OK;
    ok = ok && moe_static_scratch_setup(ctx) == TF_OK;
    if (const char *env = getenv("TF_STREAM_BLOCKS_PER_CU")) {
        const int v = atoi(env);
        if (v >= 1 && v <= 8) ctx->stream_blocks_per_cu = v;
    }
    if (!ok) {
        tf_ctx_destroy(ctx);
        return TF_ERR_OUT_OF_MEMORY;
    }
    *out_ctx = ctx;
    return TF_OK;
}

void tf_ctx_destroy(tf_ctx *ctx) {
    if (!ctx) return;
    if (ctx->router_logits) (void)hipFree(ctx->router_logits);
    if (ctx->head_x_normed) (void)hipFree(ctx->head_x_normed);
    if (ctx->head_summaries) (void)hipFree(ctx->head_summaries);
    if (ctx->head_logits) (void)hipFree(ctx->head_logits);
    if (ctx->group_scratch) (void)hipFree(ctx->group_scratch);
    if (ctx->few_scratch) (void)hipFree(ctx->few_scratch);
    if (ctx->prefill_logits) (void)hipFree(ctx->prefill_logits);
    if (ctx->sample_scratch) (void)hipFree(ctx->sample_scratch);
    if (ctx->shared_block_acts) (void)hipFree(ctx->shared_block_acts);
    if (ctx->attn_scratch) (void)hipFree(ctx->attn_scratch);
    for (hipEvent_t e : ctx->step_events)
        if (e) (void)hipEventDestroy(e);
    delete ctx;
}

namespace {

// Grows one wrapper buffer; kernels of earlier calls may still use the old one, so the device is drained first.
bool regrow(void **buf, size_t *have, size_t need, size_t unit) {
    if (*have * unit >= need) return true;
    if (*buf) {
        if (hipDeviceSynchronize() != hipSuccess) return false;
        (void)hipFree(*buf);
        *buf = nullptr;
        *have = 0;
    }
    if (need == 0) return true;
    if (hipMalloc(buf, need) != hipSuccess) return false;
    *have = need / unit;
    return true;
}

}  // namespace

int32_t tf_ctx_reserve(tf_ctx *ctx, const tf_scratch_limits *limits) {
    TF_REQUIRE(ctx, ctx && limits, TF_ERR_INVALID_ARGUMENT, "ctx_reserve: null argument");
    if (hipSetDevice(ctx->device) != hipSuccess) return fail(ctx, TF_ERR_NO_DEVICE, "ctx_reserve: cannot select device %d", ctx->device);
    tf_scratch_limits want = ctx->limits;   // limits only ever grow
    want.max_vocab = limits->max_vocab > want.max_vocab ? limits->max_vocab : want.max_vocab;
    want.max_block_tokens = limits->max_block_tokens > want.max_block_tokens ? limits->max_block_tokens : want.max_block_tokens;
    want.max_experts = limits->max_experts > want.max_experts ? limits->max_experts : want.max_experts;
    want.max_shared_intermediate = limits->max_shared_intermediate > want.max_shared_intermediate ? limits->max_shared_intermediate : want.max_shared_intermediate;
    want.max_q_heads = limits->max_q_heads > want.max_q_heads ? limits->max_q_heads : want.max_q_heads;
    want.max_head_dim = limits->max_head_dim > want.max_head_dim ? limits->max_head_dim : want.max_head_dim;
    want.max_attention_block_tokens = limits->max_attention_block_tokens > want.max_attention_block_tokens ? limits->max_attention_block_tokens : want.max_attention_block_tokens;
    bool ok = regrow(reinterpret_cast<void **>(&ctx->head_logits), &ctx->head_logits_count, (size_t)want.max_vocab * sizeof(float), sizeof(float));
    ok = ok && regrow(reinterpret_cast<void **>(&ctx->prefill_logits), &ctx->prefill_logits_count,
                      prefill_logits_floats_for(want.max_block_tokens, want.max_experts) * sizeof(float), sizeof(float));
    const size_t sample_before = ctx->sample_scratch_bytes;
    ok = ok && regrow(&ctx->sample_scratch, &ctx->sample_scratch_bytes, sample_scratch_bytes_for(want.max_vocab), 1);
    if (ok && ctx->sample_scratch_bytes != sample_before && ctx->sample_scratch)
        ok = hipMemset(ctx->sample_scratch, 0, sample_scratch_clear_bytes()) == hipSuccess;   // cells and ticket start at zero
    ok = ok && regrow(&ctx->shared_block_acts, &ctx->shared_block_acts_bytes, (size_t)want.max_block_tokens * want.max_shared_intermediate * 2, 1);
    ok = ok && regrow(&ctx->attn_scratch, &ctx->attn_scratch_bytes,
                      attention_scratch_floats_for(ctx->num_cus, want.max_q_heads, want.max_head_dim, want.max_attention_block_tokens) * sizeof(float), 1);
    if (!ok) return fail(ctx, TF_ERR_OUT_OF_MEMORY, "ctx_reserve: out of device memory");
    ctx->limits = want;
    return TF_OK;
}

int32_t tf_ctx_scratch_limits(const tf_ctx *ctx, tf_scratch_limits *out_limits) {
    if (!ctx || !out_limits) return TF_ERR_INVALID_ARGUMENT;
    *out_limits = ctx->limits;
    return TF_OK;
}

int32_t tf_stream_synchronize(tf_ctx *ctx, tf_stream stream) {
    const hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "stream synchronize: %s", hipGetErrorString(e));
    return TF_OK;
}

int32_t tf_ctx_set_step_timing(tf_ctx *ctx, int32_t enabled) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "step timing: null context");
    if (enabled) {
        for (hipEvent_t &e : ctx->step_events) {
            if (e) continue;
            const hipError_t err = hipEventCreate(&e);
            if (err != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "step timing: %s", hipGetErrorString(err));
        }
    }
    ctx->step_timing = enabled != 0;
    ctx->step_timed = false;
    return TF_OK;
}

int32_t tf_ctx_last_step_timing(tf_ctx *ctx, float out_us[4]) {
    TF_REQUIRE(ctx, ctx && out_us, TF_ERR_INVALID_ARGUMENT, "step timing: null argument");
    TF_REQUIRE(ctx, ctx->step_timing && ctx->step_timed, TF_ERR_UNAVAILABLE, "step timing: no decode step recorded while timing was enabled");
    hipError_t err = hipEventSynchronize(ctx->step_events[4]);
    for (int i = 0; i < 4 && err == hipSuccess; ++i) {
        float ms = 0.0f;
        err = hipEventElapsedTime(&ms, ctx->step_events[i], ctx->step_events[i + 1]);
        out_us[i] = ms * 1e3f;
    }
    if (err != hipSuccess) return fail(ctx, TF_ERR_DEVICE, "step timing: %s", hipGetErrorString(err));
    return TF_OK;
}

const float *tf_router_logits(const tf_ctx *ctx) { return ctx ? ctx->router_logits : nullptr; }
const float *tf_prefill_router_logits(const tf_ctx *ctx) { return ctx ? ctx->prefill_logits : nullptr; }

}  // extern "C"

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
    if (ctx->prefill_logits) (void)hipFree(ctx->prefill_logits);
    if (ctx->sample_scratch) (void)hipFree(ctx->sample_scratch);
    if (ctx->shared_block_acts) (void)hipFree(ctx->shared_block_acts);
    if (ctx->attn_scratch) (void)hipFree(ctx->attn_scratch);
    for (hipEvent_t e : ctx->step_events)
        if (e) (void)hipEventDestroy(e);
    delete ctx;
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

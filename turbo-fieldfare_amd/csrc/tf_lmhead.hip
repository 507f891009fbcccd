// Tied int4 output head for gfx950: final RMSNorm -> vocab-sized int4 GEMV -> greedy argmax without materialising
// logits, and the logits variant for samplers.
#include "tf_argmax.hpp"
#include "tf_gemv_kernels.hpp"

using namespace tfk;

namespace {

// Persistent row streamer: every wave walks tiles wave, wave + nwaves, ... of RT rows and keeps the best finite logit it
// has seen (rows ascend within a wave, so a strict comparison keeps the lowest index among equals).  With FUSE_NORM each
// block normalises the hidden vector itself (rmsnorm_bf16w needs no kernel of its own).  Each block folds its best
// {value, index} into one of kHeadCells 64-bit cells with a single atomic max on the key
// (orderable(value) << 32 | ~index): larger value wins, equal values resolve to the lower index, 0 means "nothing finite".
// The block that finishes last turns the cells into the token and clears them for the next call.
template <int RT, int NP, int SD, bool FUSE_NORM>
__global__ __launch_bounds__(256, 4) void head_greedy_long_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                               const half_t *x, const uint16_t *norm_w, float eps,
                                                               unsigned long long *cells, uint32_t *out_token, long v_rows,
                                                               int k) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ float partial[4];
    const int lane = threadIdx.x & 63;
    const int wib = threadIdx.x >> 6;
    const long wave = uniform_int((int)(((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6));
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    const long ntiles = (v_rows + RT - 1) / RT;
    Best best{-INFINITY, 0xFFFFFFFFu};
    const size_t tile_bytes = (size_t)RT * (k >> 1);
    const size_t sb_bytes = (size_t)RT * (k >> 6) * 2;
    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile ta, tb;
    rs.init_map(k, lane);
    auto request = [&](typename RowStream<RT, NP>::Tile &t, long at) {
        rs.load(t, W + at * tile_bytes, S + at * sb_bytes, B + at * sb_bytes, v_rows - at * RT);
    };
    // requests in this order: the activations, then the first two tiles; the activations are normalised and staged in
    // LDS while the tiles are in flight
    long t0 = wave, t1 = wave + nwaves;
    if constexpr (FUSE_NORM) {
        XNormStage stage;
        stage.request(x, norm_w, k);
        if (t0 < ntiles) request(ta, t0);
        if (t1 < ntiles) request(tb, t1);
        stage.publish(eps, k, xa, xsum, partial);
    } else {
        XStage stage;
        stage.request(x, k);
        if (t0 < ntiles) request(ta, t0);
        if (t1 < ntiles) request(tb, t1);
        stage.publish(k, xa, xsum);
    }
    // rows ascend within a wave, so a strict comparison keeps the lowest index among equals
    auto consider = [&](const typename RowStream<RT, NP>::Tile &t, long at) {
        float out[RT];
        rs.template reduce<SD>(t, out);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            const long row = at * RT + r;
            const float z = out[r];
            if (row < v_rows && __builtin_isfinite(z) && z > best.v) {
                best.v = z;
                best.idx = (uint32_t)row;
            }
        }
    };
    if (t0 < ntiles) {
        rs.init_x_lds(xa, xsum, k);
        for (;;) {
            consider(ta, t0);
            t0 += 2 * nwaves;
            if (t0 < ntiles) request(ta, t0);
            if (t1 >= ntiles) break;
            consider(tb, t1);
            t1 += 2 * nwaves;
            if (t1 < ntiles) request(tb, t1);
            if (t0 >= ntiles) break;
        }
    }
    if (lane == 0) { sv[wib] = best.v; si[wib] = best.idx; }
    fold_block_best(sv, si, cells, out_token);
}

// Fallback first stage: argmax summaries over an fp32 logits vector (one summary per block).
__global__ __launch_bounds__(256) void logits_partial_argmax_kernel(const float *logits, float *summaries, long v_rows) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    Best best{-INFINITY, 0xFFFFFFFFu};
    for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < v_rows; i += (long)gridDim.x * blockDim.x) {
        const float z = logits[i];
        if (__builtin_isfinite(z)) better(best, z, (uint32_t)i);
    }
    wave_best_pair(best.v, best.idx);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best.v; si[threadIdx.x >> 6] = best.idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        Best b{sv[0], si[0]};
        for (int w = 1; w < 4; ++w) better(b, sv[w], si[w]);
        summaries[2 * blockIdx.x] = b.v;
        summaries[2 * blockIdx.x + 1] = __uint_as_float(b.idx);
    }
}

// Global argmax over the summaries: highest value, lowest index among equals, token 0 when nothing was finite
// (lm_head_greedy_int4_rows_reduce, Metal/Sampling/logit.metal:740-787).
__global__ __launch_bounds__(256) void head_reduce_kernel(const float *summaries, uint32_t *out_token, uint32_t count) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    Best best{-INFINITY, 0xFFFFFFFFu};
    for (uint32_t i = threadIdx.x; i < count; i += blockDim.x)
        better(best, summaries[2 * i], __float_as_uint(summaries[2 * i + 1]));
    wave_best_pair(best.v, best.idx);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best.v; si[threadIdx.x >> 6] = best.idx; }
    __syncthreads();
    if (threadIdx.x == 0) {
        Best b{sv[0], si[0]};
        for (int w = 1; w < 4; ++w) better(b, sv[w], si[w]);
        out_token[0] = b.idx == 0xFFFFFFFFu ? 0u : b.idx;
    }
}

int32_t validate_head(tf_ctx *ctx, const char *who, const void *hidden, uint64_t hidden_offset, const void *norm_weight,
                      uint64_t norm_offset, const void *weights, uint64_t weights_offset, const void *scales,
                      uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *out, uint32_t d,
                      uint32_t vocab, tf_dtype sd) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "%s: null context", who);
    TF_REQUIRE(ctx, hidden && norm_weight && weights && scales && biases && out, TF_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    TF_REQUIRE(ctx, d > 0 && d <= kMaxHeadD, TF_ERR_INVALID_ARGUMENT, "%s: d=%u exceeds wrapper maxD=%u", who, d, kMaxHeadD);
    TF_REQUIRE(ctx, vocab > 0, TF_ERR_INVALID_ARGUMENT, "%s: vocab must be positive", who);
    TF_REQUIRE(ctx, d % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "%s: d must be a multiple of 64", who);
    TF_REQUIRE(ctx, aligned(at(weights, weights_offset), 2), TF_ERR_INVALID_ARGUMENT, "%s needs a 2-aligned weightsOffset", who);
    TF_REQUIRE(ctx, aligned(at(hidden, hidden_offset), 2) && aligned(at(norm_weight, norm_offset), 2) &&
                   aligned(at(scales, scales_offset), 2) && aligned(at(biases, biases_offset), 2),
               TF_ERR_INVALID_ARGUMENT, "%s: misaligned operand", who);
    TF_REQUIRE(ctx, sd == TF_BF16 || sd == TF_FP16, TF_ERR_INVALID_ARGUMENT, "%s: scale dtype must be bf16 or fp16", who);
    return TF_OK;
}

}  // namespace

extern "C" {

int32_t tf_lm_head_greedy_int4(tf_ctx *ctx, tf_stream stream, const void *hidden, uint64_t hidden_offset, const void *norm_weight,
                               uint64_t norm_offset, const void *weights, uint64_t weights_offset, const void *scales,
                               uint64_t scales_offset, const void *biases, uint64_t biases_offset, void *out_token, uint32_t d,
                               uint32_t vocab, float rms_eps, tf_dtype scale_dtype) {
    int32_t rc = validate_head(ctx, "lm_head_greedy_int4", hidden, hidden_offset, norm_weight, norm_offset, weights, weights_offset,
                               scales, scales_offset, biases, biases_offset, out_token, d, vocab, scale_dtype);
    if (rc != TF_OK) return rc;
    TF_REQUIRE(ctx, aligned(out_token, 4), TF_ERR_INVALID_ARGUMENT, "lm_head_greedy_int4: misaligned out_token");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint8_t *w = at(weights, weights_offset);
    const uint8_t *s = at(scales, scales_offset);
    const uint8_t *b = at(biases, biases_offset);
    const half_t *hid = reinterpret_cast<const half_t *>(at(hidden, hidden_offset));
    const uint16_t *nw = reinterpret_cast<const uint16_t *>(at(norm_weight, norm_offset));
    const half_t *xn = static_cast<const half_t *>(ctx->head_x_normed);
    const LongPlan plan = plan_long_rows((int)d, 2);   // up to two rows a tile: a row's sum is then independent of its place in the tile
    const bool rows_fast = aligned16(w) && d > 1024 && plan.rt > 0;
    const bool fuse_norm = rows_fast && aligned16(hid) && aligned16(nw) && d <= (uint32_t)kMaxFusedNormD;
    if (!fuse_norm) {
        rc = launch_rmsnorm_bf16w(ctx, st, hid, nw, ctx->head_x_normed, d, rms_eps);
        if (rc != TF_OK) return rc;
    }
    uint32_t n_summaries = 0;
    if (rows_fast) {
        const long ntiles = ((long)vocab + plan.rt - 1) / plan.rt;
        const long max_blocks = (long)ctx->num_cus * ctx->stream_blocks_per_cu;
        const uint32_t grid = (uint32_t)std::max<long>(1, std::min<long>((ntiles + 3) / 4, max_blocks));
        unsigned long long *cells = reinterpret_cast<unsigned long long *>(ctx->head_summaries + 2 * kMaxHeadWaves);
        bool launched = false;
#define TF_HEAD_LAUNCH(RT_, NP_, SD_, FN_)                                                                              \
    hipLaunchKernelGGL((head_greedy_long_kernel<RT_, NP_, SD_, FN_>), dim3(grid), dim3(256), 0, st, w, s, b,            \
                       FN_ ? hid : xn, nw, rms_eps, cells, static_cast<uint32_t *>(out_token), (long)vocab, (int)d)
#define TF_HEAD_CASE(RT_, NP_)                                                                                          \
    if (!launched && plan.rt == RT_ && plan.np == NP_) {                                                                \
        launched = true;                                                                                                \
        if (scale_dtype == TF_BF16) { if (fuse_norm) TF_HEAD_LAUNCH(RT_, NP_, 0, true); else TF_HEAD_LAUNCH(RT_, NP_, 0, false); } \
        else { if (fuse_norm) TF_HEAD_LAUNCH(RT_, NP_, 1, true); else TF_HEAD_LAUNCH(RT_, NP_, 1, false); }             \
    }
        TF_HEAD_CASE(1, 1) TF_HEAD_CASE(1, 2) TF_HEAD_CASE(1, 3) TF_HEAD_CASE(1, 4)
        TF_HEAD_CASE(2, 1) TF_HEAD_CASE(2, 2) TF_HEAD_CASE(2, 3) TF_HEAD_CASE(2, 4)
        TF_HEAD_CASE(4, 1) TF_HEAD_CASE(4, 2) TF_HEAD_CASE(4, 3) TF_HEAD_CASE(4, 4)
#undef TF_HEAD_CASE
#undef TF_HEAD_LAUNCH
        return check_launch(ctx, "lm_head_greedy rows");
    } else {
        // short or unaligned rows: fp32 logits into wrapper-owned scratch, then a two-stage argmax
        if (ctx->head_logits_count < vocab)
            return scratch_too_small(ctx, "lm_head_greedy_int4 (unaligned rows)", (size_t)vocab * sizeof(float), ctx->head_logits_count * sizeof(float));
        rc = launch_gemv4(ctx, st, w, s, b, xn, ctx->head_logits, vocab, d, scale_dtype, TF_FP32);
        if (rc != TF_OK) return rc;
        const uint32_t grid = (uint32_t)std::min<long>(((long)vocab + 255) / 256, 1024);
        n_summaries = grid;
        hipLaunchKernelGGL(logits_partial_argmax_kernel, dim3(grid), dim3(256), 0, st, ctx->head_logits, ctx->head_summaries, (long)vocab);
        rc = check_launch(ctx, "lm_head_greedy partial argmax");
        if (rc != TF_OK) return rc;
    }
    hipLaunchKernelGGL(head_reduce_kernel, dim3(1), dim3(256), 0, st, ctx->head_summaries, static_cast<uint32_t *>(out_token), n_summaries);
    return check_launch(ctx, "lm_head_greedy reduce");
}

int32_t tf_lm_head_logits_int4(tf_ctx *ctx, tf_stream stream, const void *hidden, uint64_t hidden_offset, const void *norm_weight,
                               uint64_t norm_offset, const void *weights, uint64_t weights_offset, const void *scales,
                               uint64_t scales_offset, const void *biases, uint64_t biases_offset, void *logits,
                               uint64_t logits_offset, uint32_t d, uint32_t vocab, float rms_eps, tf_dtype scale_dtype,
                               tf_dtype out_dtype) {
    int32_t rc = validate_head(ctx, "lm_head_logits_int4", hidden, hidden_offset, norm_weight, norm_offset, weights, weights_offset,
                               scales, scales_offset, biases, biases_offset, logits, d, vocab, scale_dtype);
    if (rc != TF_OK) return rc;
    TF_REQUIRE(ctx, out_dtype == TF_FP16 || out_dtype == TF_FP32, TF_ERR_INVALID_ARGUMENT, "lm_head_logits_int4: logits must be fp16 or fp32");
    TF_REQUIRE(ctx, aligned(at(logits, logits_offset), out_dtype == TF_FP16 ? 2 : 4), TF_ERR_INVALID_ARGUMENT, "lm_head_logits_int4: misaligned logits");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint8_t *w = at(weights, weights_offset);
    if (gemv4_can_fuse_norm(w, at(hidden, hidden_offset), at(norm_weight, norm_offset), d))
        return launch_gemv4(ctx, st, w, at(scales, scales_offset), at(biases, biases_offset), at(hidden, hidden_offset),
                            at(logits, logits_offset), vocab, d, scale_dtype, out_dtype, at(norm_weight, norm_offset), rms_eps);
    rc = launch_rmsnorm_bf16w(ctx, st, at(hidden, hidden_offset), at(norm_weight, norm_offset), ctx->head_x_normed, d, rms_eps);
    if (rc != TF_OK) return rc;
    return launch_gemv4(ctx, st, w, at(scales, scales_offset), at(biases, biases_offset), ctx->head_x_normed,
                        at(logits, logits_offset), vocab, d, scale_dtype, out_dtype);
}

}  // extern "C"

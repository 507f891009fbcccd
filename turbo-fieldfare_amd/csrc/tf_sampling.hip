// What sits either side of the tied int4 output head: the embedding row lookup (same table), the soft-capped softmax over
// the vocabulary, and the samplers (greedy, Gumbel-max, top-k / top-p / temperature with inverse-CDF draw).
// The reference runs each of these in a single threadgroup; here the vocabulary-sized passes are spread over the chip and
// meet through per-block partials (softmax), an atomic argmax fold (greedy, Gumbel) or sorted tiles (top-k).
#include "tf_argmax.hpp"
#include "tf_context.hpp"
#include "tf_rowdot.hpp"

using namespace tfk;

namespace {

// fp32 -> fp16 with the fp32 value pinned first, so that the multiply producing it is rounded to fp32 as in the
// reference and not fused into the conversion
__device__ __forceinline__ half_t to_half_pinned(float v) {
    asm volatile("" : "+v"(v));
    return (half_t)v;
}

// ------------------------------------------------------------------------------------------------ embedding rows
// out[t, i] = half((q * s + b) * out_scale) for row tokens[t] of the int4 table; one thread per 8 elements (one word).
__global__ __launch_bounds__(256) void embed_lookup_kernel(const uint8_t *table, const uint16_t *scales, const uint16_t *biases,
                                                           const uint32_t *tokens, uint32_t single_token, half_t *out, uint32_t rows,
                                                           uint32_t d, float out_scale, uint32_t table_rows) {
    const uint32_t t = blockIdx.y;
    const uint32_t word = blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= rows || word * 8u >= d) return;
    uint32_t token = tokens ? tokens[t] : single_token;
    token = token < table_rows ? token : table_rows - 1;
    const uint32_t groups = d >> 6;
    const uint16_t *wp = reinterpret_cast<const uint16_t *>(table + (size_t)token * (d >> 1) + (size_t)word * 4);
    const uint32_t w = (uint32_t)wp[0] | ((uint32_t)wp[1] << 16);
    const float s = bf16_to_f32(scales[(size_t)token * groups + (word >> 3)]);
    const float b = bf16_to_f32(biases[(size_t)token * groups + (word >> 3)]);
    half_t *dst = out + (size_t)t * d + (size_t)word * 8;
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[i] = to_half_pinned(((float)((w >> (4 * i)) & 0xFu) * s + b) * out_scale);
}

// ------------------------------------------------------------------------------------------------ soft-capped softmax
// z = softcap * tanh(x / softcap); probs = exp(z - max z) / sum exp(z - max z).  First launch: per-block (max, sum) by
// the online rule; second launch: every block merges the partials (a few hundred values) and normalises its share.
constexpr uint32_t kSoftmaxMaxBlocks = 256;

__device__ __forceinline__ float softcapped(float x, float softcap) { return softcap * tanhf(x / softcap); }

// merge (m2, d2) into (m, d): d counts exp(z - m)
__device__ __forceinline__ void merge_md(float &m, float &d, float m2, float d2) {
    const float mn = fmaxf(m, m2);
    const float a = (m == -INFINITY) ? 0.0f : d * expf(m - mn);
    const float b = (m2 == -INFINITY) ? 0.0f : d2 * expf(m2 - mn);
    m = mn;
    d = a + b;
}

// reduces (m, d) over a 256-thread block; every thread gets the result.  scratch: 8 floats of LDS.
__device__ __forceinline__ void block_merge_md(float &m, float &d, float *scratch) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const float m2 = __shfl_xor(m, off, kWave);
        const float d2 = __shfl_xor(d, off, kWave);
        merge_md(m, d, m2, d2);
    }
    __syncthreads();
    if ((threadIdx.x & 63) == 0) {
        scratch[threadIdx.x >> 6] = m;
        scratch[4 + (threadIdx.x >> 6)] = d;
    }
    __syncthreads();
    m = scratch[0];
    d = scratch[4];
#pragma unroll
    for (int w = 1; w < 4; ++w) merge_md(m, d, scratch[w], scratch[4 + w]);
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_partials_kernel(const T *logits, float *partials, uint32_t v, float softcap) {
    __shared__ float scratch[8];
    float m = -INFINITY, d = 0.0f;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < v; i += gridDim.x * blockDim.x) {
        const float z = softcapped((float)logits[i], softcap);
        const float mn = fmaxf(m, z);
        const float scale = (m == -INFINITY) ? 0.0f : expf(m - mn);
        d = d * scale + expf(z - mn);
        m = mn;
    }
    block_merge_md(m, d, scratch);
    if (threadIdx.x == 0) {
        partials[2 * blockIdx.x] = m;
        partials[2 * blockIdx.x + 1] = d;
    }
}

template <typename T>
__global__ __launch_bounds__(256) void softmax_normalize_kernel(const T *logits, const float *partials, uint32_t n_partials, half_t *probs,
                                                                uint32_t v, float softcap) {
    __shared__ float scratch[8];
    float m = -INFINITY, d = 0.0f;
    if (threadIdx.x < n_partials) {
        m = partials[2 * threadIdx.x];
        d = partials[2 * threadIdx.x + 1];
    }
    block_merge_md(m, d, scratch);
    const float inv_d = 1.0f / d;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < v; i += gridDim.x * blockDim.x)
        probs[i] = to_half_pinned(expf(softcapped((float)logits[i], softcap) - m) * inv_d);
}

// ------------------------------------------------------------------------------------------------ samplers
__device__ __forceinline__ uint64_t xorshift64(uint64_t &s) {
    s ^= s << 13;
    s ^= s >> 7;
    s ^= s << 17;
    return s * 2685821657736338717ull;
}
__device__ __forceinline__ float uniform01(uint64_t &s) { return (float)(uint32_t)(xorshift64(s) >> 40) * (1.0f / 16777216.0f); }

// counter-based Gumbel noise for (seed, position, row)
__device__ __forceinline__ float gumbel_for(uint64_t seed, uint32_t position, uint32_t row) {
    uint64_t x = seed ^ ((uint64_t)position * 0xD2B74407B1CE6E93ull) ^ (uint64_t)row;
    x = x + 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    x = x ^ (x >> 31);
    const float u = ((float)(uint32_t)(x >> 40) + 0.5f) * (1.0f / 16777216.0f);
    return -logf(-logf(u));
}

// GUMBEL false: argmax of the probabilities (temperature 0).  GUMBEL true: argmax of log(p) / T + Gumbel noise over the
// entries with p > 0, which draws from p^(1/T) / Z.  Ties go to the lowest index; nothing eligible gives token 0.
template <bool GUMBEL>
__global__ __launch_bounds__(256) void sample_argmax_kernel(const half_t *probs, uint32_t v, float inv_t, uint64_t seed, uint32_t position,
                                                            unsigned long long *cells, uint32_t *out_token) {
    __shared__ float sv[4];
    __shared__ uint32_t si[4];
    Best best{-INFINITY, 0xFFFFFFFFu};
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < v; i += gridDim.x * blockDim.x) {
        const float p = (float)probs[i];
        if constexpr (GUMBEL) {
            if (!(p > 0.0f)) continue;
            const float s = inv_t * logf(p) + gumbel_for(seed, position, i);
            if (s > best.v) { best.v = s; best.idx = i; }
        } else {
            if (p > best.v) { best.v = p; best.idx = i; }
        }
    }
    wave_best_pair(best.v, best.idx);
    if ((threadIdx.x & 63) == 0) { sv[threadIdx.x >> 6] = best.v; si[threadIdx.x >> 6] = best.idx; }
    fold_block_best(sv, si, cells, out_token);
}

// ---- top-k through sorted tiles
// A tile is 1024 (value, index) pairs sorted by (value descending, index ascending) with a bitonic network in LDS; its
// first KEEP pairs go on to the next stage.  Pairs that must never be chosen carry (-inf, 0xFFFFFFFF): slots past the
// input, NaN and -inf probabilities.
constexpr uint32_t kTile = 1024;

__device__ __forceinline__ bool pair_better(float lv, uint32_t li, float rv, uint32_t ri) { return lv > rv || (lv == rv && li < ri); }

__device__ __forceinline__ void sort_tile(float *values, uint32_t *indices) {
    for (uint32_t width = 2; width <= kTile; width <<= 1) {
        for (uint32_t stride = width >> 1; stride > 0; stride >>= 1) {
            __syncthreads();
            for (uint32_t i = threadIdx.x; i < kTile; i += 256) {
                const uint32_t partner = i ^ stride;
                if (partner <= i) continue;
                const float lv = values[i], rv = values[partner];
                const uint32_t li = indices[i], ri = indices[partner];
                const bool descending = (i & width) == 0;
                const bool swap = descending ? pair_better(rv, ri, lv, li) : pair_better(lv, li, rv, ri);
                if (swap) {
                    values[i] = rv;
                    indices[i] = ri;
                    values[partner] = lv;
                    indices[partner] = li;
                }
            }
        }
    }
    __syncthreads();
}

// source: fp16 probabilities (in_values == nullptr) or the pairs of an earlier stage
__device__ __forceinline__ void load_tile(const half_t *probs, const float *in_values, const uint32_t *in_indices, uint32_t base,
                                          uint32_t count, float *values, uint32_t *indices) {
    for (uint32_t i = threadIdx.x; i < kTile; i += 256) {
        const uint32_t source = base + i;
        float val = -INFINITY;
        uint32_t idx = 0xFFFFFFFFu;
        if (source < count) {
            val = in_values ? in_values[source] : (float)probs[source];
            idx = in_values ? in_indices[source] : source;
            if (!(val > -INFINITY)) {
                val = -INFINITY;
                idx = 0xFFFFFFFFu;
            }
        }
        values[i] = val;
        indices[i] = idx;
    }
}

template <uint32_t KEEP>
__global__ __launch_bounds__(256) void topk_tile_kernel(const half_t *probs, const float *in_values, const uint32_t *in_indices,
                                                        float *out_values, uint32_t *out_indices, uint32_t count) {
    __shared__ float values[kTile];
    __shared__ uint32_t indices[kTile];
    load_tile(probs, in_values, in_indices, blockIdx.x * kTile, count, values, indices);
    sort_tile(values, indices);
    for (uint32_t i = threadIdx.x; i < KEEP; i += 256) {
        out_values[blockIdx.x * KEEP + i] = values[i];
        out_indices[blockIdx.x * KEEP + i] = indices[i];
    }
}

// Running sums of values[0..n) in index order, one fp32 add per element (thread 0; n <= 256), left in sums[] for the whole
// block: sums[i] is what a sequential accumulation holds after element i, so a search over sums[] finds exactly the element a
// sequential walk would stop at.  Ends with a barrier.
__device__ __forceinline__ void running_sums(const float *values, uint32_t n, float *sums) {
    if (threadIdx.x == 0) {
        float acc = 0.0f;
        for (uint32_t i = 0; i < n; ++i) {
            acc += values[i];
            sums[i] = acc;
        }
    }
    __syncthreads();
}

// Smallest candidate any thread of the block offers (threads without one offer `none`), through one LDS word.  Two barriers.
__device__ __forceinline__ uint32_t block_first(uint32_t candidate, uint32_t none, uint32_t *word) {
    if (threadIdx.x == 0) *word = none;
    __syncthreads();
    if (candidate < none) atomicMin(word, candidate);
    __syncthreads();
    const uint32_t found = *word;
    __syncthreads();
    return found;
}

// Last tile: sort, then thread t looks after slot t of the k best (k <= 256 = the block).  Results follow the reference's
// sampler (Metal/Sampling/logit.metal:564-606): the usable prefix ends at the first slot that is padding or not finite; the
// top-p cut keeps the shortest prefix whose mass (probabilities still carry their full-vocabulary normalisation) reaches top_p;
// survivors are reweighted by p^(1/T); the draw is the inverse CDF of the seeded xorshift64* uniform.  The sums that decide
// the cut and the draw are accumulated in index order (running_sums); the slots are tested and reweighted side by side.
__global__ __launch_bounds__(256) void topk_final_kernel(const half_t *probs, const float *in_values, const uint32_t *in_indices, uint32_t count,
                                                         uint32_t k, float temperature, float top_p, uint64_t seed, uint32_t *out_token) {
    __shared__ float values[kTile];
    __shared__ uint32_t indices[kTile];
    __shared__ float sums[256];
    __shared__ uint32_t word;
    load_tile(probs, in_values, in_indices, 0, count, values, indices);
    sort_tile(values, indices);
    const uint32_t t = threadIdx.x;
    const bool unusable = t < k && (indices[t] == 0xFFFFFFFFu || !__builtin_isfinite(values[t]));
    uint32_t n = block_first(unusable ? t : k, k, &word);
    if (top_p > 0.0f && top_p < 1.0f) {
        running_sums(values, n, sums);
        n = block_first(t < n && sums[t] >= top_p ? t + 1 : n, n, &word);
    }
    if (temperature != 1.0f) {
        if (t < n) values[t] = powf(values[t], 1.0f / temperature);
        __syncthreads();
    }
    running_sums(values, n, sums);
    uint64_t rng = seed;
    (void)xorshift64(rng);
    const float u = uniform01(rng) * (n > 0 ? sums[n - 1] : 0.0f);
    const uint32_t slot = block_first(t < n && u <= sums[t] ? t : n, n, &word);
    if (t == 0) {
        const uint32_t token = indices[slot < n ? slot : 0];
        out_token[0] = token == 0xFFFFFFFFu ? 0u : token;
    }
}

// Wrapper-owned scratch of the samplers: [argmax cells + ticket | softmax partials | two pair buffers].
struct SampleScratch {
    unsigned long long *cells;
    float *partials;
    float *values[2];
    uint32_t *indices[2];
};

constexpr size_t kCellBytes = (kHeadCells + 1) * sizeof(unsigned long long);
constexpr size_t kPartialBytes = kSoftmaxMaxBlocks * 2 * sizeof(float);

size_t sample_need(uint32_t pair_capacity) {
    const size_t pairs = ((size_t)pair_capacity + 255) / 256 * 256;
    return kCellBytes + kPartialBytes + pairs * 16;
}

int32_t sample_scratch(tf_ctx *ctx, uint32_t pair_capacity, SampleScratch &out) {
    const size_t need = sample_need(pair_capacity);
    if (ctx->sample_scratch_bytes < need) return scratch_too_small(ctx, "sampler", need, ctx->sample_scratch_bytes);
    uint8_t *base = static_cast<uint8_t *>(ctx->sample_scratch);
    const size_t have_pairs = (ctx->sample_scratch_bytes - kCellBytes - kPartialBytes) / 16;
    out.cells = reinterpret_cast<unsigned long long *>(base);
    out.partials = reinterpret_cast<float *>(base + kCellBytes);
    uint8_t *pair_base = base + kCellBytes + kPartialBytes;
    out.values[0] = reinterpret_cast<float *>(pair_base);
    out.values[1] = reinterpret_cast<float *>(pair_base + have_pairs * 4);
    out.indices[0] = reinterpret_cast<uint32_t *>(pair_base + have_pairs * 8);
    out.indices[1] = reinterpret_cast<uint32_t *>(pair_base + have_pairs * 12);
    return TF_OK;
}

uint32_t spread_blocks(const tf_ctx *ctx, uint32_t v, uint32_t cap) {
    const uint32_t by_work = (v + 2047) / 2048;             // at least 8 elements per thread
    uint32_t blocks = by_work < cap ? by_work : cap;
    const uint32_t chip = (uint32_t)ctx->num_cus * 2;
    blocks = blocks < chip ? blocks : chip;
    return blocks > 0 ? blocks : 1;
}

// the k best of probs[0..v) -> one token; k <= 256
int32_t launch_truncating_sampler(tf_ctx *ctx, hipStream_t st, const half_t *probs, uint32_t v, uint32_t k, float temperature, float top_p,
                                  uint64_t seed, uint32_t *out_token, const char *who) {
    if (v <= kTile) {
        hipLaunchKernelGGL(topk_final_kernel, dim3(1), dim3(256), 0, st, probs, (const float *)nullptr, (const uint32_t *)nullptr, v, k, temperature,
                           top_p, seed, out_token);
        return check_launch(ctx, who);
    }
    const uint32_t keep = k <= 64 ? 64u : 256u;
    const uint32_t tiles0 = (v + kTile - 1) / kTile;
    SampleScratch sc;
    const int32_t rc = sample_scratch(ctx, tiles0 * keep, sc);
    if (rc != TF_OK) return rc;
    uint32_t count = v, tiles = tiles0;
    int cur = 0;
    bool first = true;
    while (true) {
        const float *iv = first ? nullptr : sc.values[cur ^ 1];
        const uint32_t *ii = first ? nullptr : sc.indices[cur ^ 1];
        if (keep == 64) hipLaunchKernelGGL(topk_tile_kernel<64>, dim3(tiles), dim3(256), 0, st, probs, iv, ii, sc.values[cur], sc.indices[cur], count);
        else hipLaunchKernelGGL(topk_tile_kernel<256>, dim3(tiles), dim3(256), 0, st, probs, iv, ii, sc.values[cur], sc.indices[cur], count);
        count = tiles * keep;
        first = false;
        if (count <= kTile) break;
        tiles = (count + kTile - 1) / kTile;
        cur ^= 1;
    }
    hipLaunchKernelGGL(topk_final_kernel, dim3(1), dim3(256), 0, st, probs, sc.values[cur], sc.indices[cur], count, k, temperature, top_p, seed,
                       out_token);
    return check_launch(ctx, who);
}

}  // namespace

namespace tfk {

// the truncating samplers keep up to 256 candidates of every 1024-element tile of the first pass
size_t sample_scratch_bytes_for(uint32_t vocab) { return sample_need((vocab + kTile - 1) / kTile * 256u); }
size_t sample_scratch_clear_bytes() { return kCellBytes; }

}  // namespace tfk

extern "C" {

int32_t tf_embed_lookup_int4(tf_ctx *ctx, tf_stream stream, const void *table, uint64_t table_offset, const void *scales,
                             uint64_t scales_offset, const void *biases, uint64_t biases_offset, void *out, uint64_t out_offset,
                             uint32_t token_id, uint32_t d, float out_scale, uint32_t table_rows) {
    TF_REQUIRE(ctx, ctx && table && scales && biases && out, TF_ERR_INVALID_ARGUMENT, "embed_lookup_int4: null argument");
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "embed_lookup_int4: D must be a multiple of 64, got %u", d);
    TF_REQUIRE(ctx, token_id < table_rows, TF_ERR_INVALID_ARGUMENT, "embed_lookup_int4: token %u out of range (%u rows)", token_id, table_rows);
    const uint8_t *tb = at(table, table_offset);
    const uint8_t *sc = at(scales, scales_offset);
    const uint8_t *bi = at(biases, biases_offset);
    uint8_t *o = at(out, out_offset);
    TF_REQUIRE(ctx, aligned(tb, 2) && aligned(sc, 2) && aligned(bi, 2) && aligned(o, 2), TF_ERR_INVALID_ARGUMENT, "embed_lookup_int4: misaligned operand");
    hipLaunchKernelGGL(embed_lookup_kernel, dim3((d / 8 + 255) / 256, 1), dim3(256), 0, static_cast<hipStream_t>(stream), tb,
                       reinterpret_cast<const uint16_t *>(sc), reinterpret_cast<const uint16_t *>(bi), (const uint32_t *)nullptr, token_id,
                       reinterpret_cast<half_t *>(o), 1u, d, out_scale, table_rows);
    return check_launch(ctx, "embed_lookup_int4");
}

int32_t tf_prefill_embed_lookup_int4_block(tf_ctx *ctx, tf_stream stream, const void *table, uint64_t table_offset, const void *scales,
                                           uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *tokens,
                                           uint64_t tokens_offset, void *out, uint64_t out_offset, uint32_t t, uint32_t d, float out_scale,
                                           uint32_t table_rows) {
    TF_REQUIRE(ctx, ctx && table && scales && biases && tokens && out, TF_ERR_INVALID_ARGUMENT, "prefill_embed_lookup_int4_block: null argument");
    TF_REQUIRE(ctx, d > 0 && d % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "prefill_embed_lookup_int4_block: D must be a multiple of 64, got %u", d);
    TF_REQUIRE(ctx, t > 0 && t <= 65535 && table_rows > 0, TF_ERR_INVALID_ARGUMENT, "prefill_embed_lookup_int4_block: t must be in 1...65535 and the table non-empty");
    const uint8_t *tb = at(table, table_offset);
    const uint8_t *sc = at(scales, scales_offset);
    const uint8_t *bi = at(biases, biases_offset);
    const uint8_t *tk = at(tokens, tokens_offset);
    uint8_t *o = at(out, out_offset);
    TF_REQUIRE(ctx, aligned(tb, 2) && aligned(sc, 2) && aligned(bi, 2) && aligned(o, 2) && aligned(tk, 4), TF_ERR_INVALID_ARGUMENT,
               "prefill_embed_lookup_int4_block: misaligned operand");
    hipLaunchKernelGGL(embed_lookup_kernel, dim3((d / 8 + 255) / 256, t), dim3(256), 0, static_cast<hipStream_t>(stream), tb,
                       reinterpret_cast<const uint16_t *>(sc), reinterpret_cast<const uint16_t *>(bi), reinterpret_cast<const uint32_t *>(tk), 0u,
                       reinterpret_cast<half_t *>(o), t, d, out_scale, table_rows);
    return check_launch(ctx, "prefill_embed_lookup_int4_block");
}

int32_t tf_logit_softcap_softmax(tf_ctx *ctx, tf_stream stream, const void *logits, void *probs, uint32_t v, float softcap,
                                 tf_dtype logits_dtype) {
    TF_REQUIRE(ctx, ctx && logits && probs, TF_ERR_INVALID_ARGUMENT, "logit_softcap_softmax: null argument");
    TF_REQUIRE(ctx, v > 0, TF_ERR_INVALID_ARGUMENT, "logit_softcap_softmax: V must be positive");
    TF_REQUIRE(ctx, softcap > 0.0f, TF_ERR_INVALID_ARGUMENT, "logit_softcap_softmax: softcap must be positive");
    TF_REQUIRE(ctx, logits_dtype == TF_FP16 || logits_dtype == TF_FP32, TF_ERR_INVALID_ARGUMENT, "logit_softcap_softmax: logits must be fp16 or fp32");
    TF_REQUIRE(ctx, aligned(logits, logits_dtype == TF_FP16 ? 2 : 4) && aligned(probs, 2), TF_ERR_INVALID_ARGUMENT, "logit_softcap_softmax: misaligned operand");
    SampleScratch sc;
    const int32_t rc = sample_scratch(ctx, 0, sc);
    if (rc != TF_OK) return rc;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t blocks = spread_blocks(ctx, v, kSoftmaxMaxBlocks);
    half_t *ph = static_cast<half_t *>(probs);
    if (logits_dtype == TF_FP16) {
        const half_t *lh = static_cast<const half_t *>(logits);
        hipLaunchKernelGGL(softmax_partials_kernel<half_t>, dim3(blocks), dim3(256), 0, st, lh, sc.partials, v, softcap);
        hipLaunchKernelGGL(softmax_normalize_kernel<half_t>, dim3(spread_blocks(ctx, v, 1024)), dim3(256), 0, st, lh, sc.partials, blocks, ph, v, softcap);
    } else {
        const float *lf = static_cast<const float *>(logits);
        hipLaunchKernelGGL(softmax_partials_kernel<float>, dim3(blocks), dim3(256), 0, st, lf, sc.partials, v, softcap);
        hipLaunchKernelGGL(softmax_normalize_kernel<float>, dim3(spread_blocks(ctx, v, 1024)), dim3(256), 0, st, lf, sc.partials, blocks, ph, v, softcap);
    }
    return check_launch(ctx, "logit_softcap_softmax");
}

int32_t tf_sample(tf_ctx *ctx, tf_stream stream, const void *probs, void *out_token, uint32_t v, float temperature, uint32_t top_k,
                  float top_p, uint64_t seed, uint32_t position) {
    TF_REQUIRE(ctx, ctx && probs && out_token, TF_ERR_INVALID_ARGUMENT, "sample: null argument");
    TF_REQUIRE(ctx, v > 0, TF_ERR_INVALID_ARGUMENT, "sample: V must be positive");
    TF_REQUIRE(ctx, aligned(probs, 2) && aligned(out_token, 4), TF_ERR_INVALID_ARGUMENT, "sample: misaligned operand");
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t *ph = static_cast<const half_t *>(probs);
    uint32_t *tok = static_cast<uint32_t *>(out_token);
    const bool greedy = temperature <= 0.0f;
    if (greedy || (top_k == 0u && (top_p <= 0.0f || top_p >= 1.0f))) {
        SampleScratch sc;
        const int32_t rc = sample_scratch(ctx, 0, sc);
        if (rc != TF_OK) return rc;
        const uint32_t blocks = spread_blocks(ctx, v, 1024);
        if (greedy) hipLaunchKernelGGL(sample_argmax_kernel<false>, dim3(blocks), dim3(256), 0, st, ph, v, 0.0f, seed, position, sc.cells, tok);
        else hipLaunchKernelGGL(sample_argmax_kernel<true>, dim3(blocks), dim3(256), 0, st, ph, v, 1.0f / temperature, seed, position, sc.cells, tok);
        return check_launch(ctx, "sample");
    }
    uint32_t k = top_k == 0u ? v : top_k;
    k = k < 256u ? k : 256u;       // the reference's working set (kSampleTopMaxK)
    k = k < v ? k : v;
    return launch_truncating_sampler(ctx, st, ph, v, k, temperature, top_p, seed, tok, "sample");
}

int32_t tf_sample_topk64(tf_ctx *ctx, tf_stream stream, const void *probs, void *out_token, uint32_t vocab, float temperature, float top_p,
                         uint64_t seed) {
    TF_REQUIRE(ctx, ctx && probs && out_token, TF_ERR_INVALID_ARGUMENT, "sample_topk64: null argument");
    TF_REQUIRE(ctx, vocab > 0 && vocab <= 262144, TF_ERR_INVALID_ARGUMENT, "sample_topk64: unsupported vocabulary %u", vocab);
    TF_REQUIRE(ctx, temperature > 0.0f, TF_ERR_INVALID_ARGUMENT, "sample_topk64: temperature must be positive (greedy decoding takes the argmax path)");
    TF_REQUIRE(ctx, aligned(probs, 2) && aligned(out_token, 4), TF_ERR_INVALID_ARGUMENT, "sample_topk64: misaligned operand");
    return launch_truncating_sampler(ctx, static_cast<hipStream_t>(stream), static_cast<const half_t *>(probs), vocab, 64u < vocab ? 64u : vocab,
                                     temperature, top_p, seed, static_cast<uint32_t *>(out_token), "sample_topk64");
}

}  // extern "C"

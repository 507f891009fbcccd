// Affine int4/int8 dequantization and GEMV for gfx950, plus the two small primitives on the same path
// (gelu_mul_fp16, rmsnorm_bf16w).
#include "tf_gemv_kernels.hpp"
#include "tf_rowslice.hpp"

using namespace tfk;

namespace {

// ------------------------------------------------------------------------------------------------ dequantize
// out[r, c] = float(q) * scale + bias, bit-exact with the CPU statement: the product q*scale is exact in fp32
// (<= 8 bits x <= 11 bits), so a fused or an unfused multiply-add round identically.
template <int BITS, int SD>
__global__ __launch_bounds__(256) void dequantize_kernel(const uint8_t *w, const uint16_t *s, const uint16_t *b,
                                                         float *out, uint32_t m, uint32_t n) {
    const uint64_t total_pairs = (uint64_t)m * (n >> 1);
    const uint32_t groups = n >> 6;
    for (uint64_t i = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total_pairs;
         i += (uint64_t)gridDim.x * blockDim.x) {
        const uint64_t r = i / (n >> 1);
        const uint32_t c = (uint32_t)(i - r * (n >> 1)) * 2;
        const float scale = sb_to_f32<SD>(s[r * groups + (c >> 6)]);
        const float bias = sb_to_f32<SD>(b[r * groups + (c >> 6)]);
        uint32_t q0, q1;
        if constexpr (BITS == 4) {
            const uint8_t byte = w[i];
            q0 = byte & 0x0Fu;
            q1 = byte >> 4;
        } else {
            q0 = w[r * n + c];
            q1 = w[r * n + c + 1];
        }
        out[r * n + c] = (float)q0 * scale + bias;
        out[r * n + c + 1] = (float)q1 * scale + bias;
    }
}

template <typename OutT>
__device__ __forceinline__ void store_out(OutT *y, long row, float v) {
    y[row] = (OutT)v;
}

// ------------------------------------------------------------------------------------------------ GEMV kernels
// Persistent: every wave walks tiles wave, wave + nwaves, ... of RT rows through two tile buffers used alternately: a
// buffer is refilled as soon as it has been reduced, so one tile is always in flight while the other is reduced.
// The activations are requested first, then the first two tiles, and are staged in LDS (in chunk order, once per block)
// while the tiles are in flight.  FUSE_NORM: x is the raw hidden vector and the block normalises it on the way
// (rmsnorm_bf16w with weight norm_w).  k <= XStage::kMaxK.
template <int RT, int NP, int SD, typename OutT, bool FUSE_NORM>
__global__ __launch_bounds__(256, 4) void gemv4_long_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                            const half_t *x, const uint16_t *norm_w, float eps, OutT *y,
                                                            long m, int k) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ float partial[4];
    const int lane = threadIdx.x & 63;
    const long wave = uniform_int((int)(((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6));
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    const long ntiles = (m + RT - 1) / RT;
    const size_t tile_bytes = (size_t)RT * (k >> 1);
    const size_t sb_bytes = (size_t)RT * (k >> 6) * 2;

    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile ta, tb;
    rs.init_map(k, lane);
    auto request = [&](typename RowStream<RT, NP>::Tile &t, long at) {
        rs.load(t, W + at * tile_bytes, S + at * sb_bytes, B + at * sb_bytes, m - at * RT);
    };
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
    if (t0 >= ntiles) return;
    rs.init_x_lds(xa, xsum, k);
    auto emit = [&](const typename RowStream<RT, NP>::Tile &t, long at) {
        float out[RT];
        rs.template reduce<SD>(t, out);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
                if (at * RT + r < m) store_out(y, at * RT + r, out[r]);
        }
    };
    for (;;) {
        emit(ta, t0);
        t0 += 2 * nwaves;
        if (t0 < ntiles) request(ta, t0);
        if (t1 >= ntiles) break;
        emit(tb, t1);
        t1 += 2 * nwaves;
        if (t1 < ntiles) request(tb, t1);
        if (t0 >= ntiles) break;
    }
}

// The same streamer over up to three matrices that share the activations (the q, k and v projections of one token):
// one launch, one staging of x; a tile never straddles two matrices.  Output fp16.
struct GemvSegments {
    const uint8_t *W[3], *S[3], *B[3];
    half_t *y[3];
    uint32_t rows[3];
    uint32_t tile_end[3];   // running total of tiles up to and including each matrix
};

// MODE 1: x is the raw hidden vector and every block normalises it on the way into LDS (rmsnorm_bf16w with norm_w), so the
// input norm of a decoder layer needs no launch of its own.
// MODE 2: the hidden vector is itself made here, by the layer tail of the previous decoder layer (layer_tail_row with the norm of
// the shared expert's output; k <= 4096, every row and norm weight 16-byte aligned): every block repeats the tail's row
// reductions in its prologue, block 0 writes the result to tail.hidden_out (not a buffer the other blocks still read), and the
// input norm follows as in mode 1.
struct TailFuse {
    const half_t *h2, *h1, *hidden;
    half_t *hidden_out;
    const uint16_t *w_postffn2, *w_postffn, *w_postffn1;
    float eps, layer_scalar;
};
template <int RT, int NP, int SD, int MODE>
__device__ __forceinline__ void qkv_gemv_long_body(const GemvSegments &g, const half_t *x, const uint16_t *norm_w, float eps, int k, const TailFuse &tail,
                                                   u32x4 *xa, float *xsum, float *norm_partial) {
    const int lane = threadIdx.x & 63;
    const long wave = uniform_int((int)(((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6));
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    const long ntiles = g.tile_end[2];
    const size_t tile_bytes = (size_t)RT * (k >> 1);
    const size_t sb_bytes = (size_t)RT * (k >> 6) * 2;

    RowStream<RT, NP> rs;
    typename RowStream<RT, NP>::Tile ta, tb;
    rs.init_map(k, lane);
    // global tile -> (matrix, tile inside it); everything here is wave-uniform
    auto locate = [&](long at, int &seg, long &local) {
        seg = at < (long)g.tile_end[0] ? 0 : (at < (long)g.tile_end[1] ? 1 : 2);
        local = at - (seg == 0 ? 0 : (long)g.tile_end[seg - 1]);
    };
    auto request = [&](typename RowStream<RT, NP>::Tile &t, long at) {
        int seg;
        long local;
        locate(at, seg, local);
        rs.load(t, g.W[seg] + local * tile_bytes, g.S[seg] + local * sb_bytes, g.B[seg] + local * sb_bytes, (long)g.rows[seg] - local * RT);
    };
    long t0 = wave, t1 = wave + nwaves;
    if constexpr (MODE == 2) {
        const RowSlice<true> slice{(uint32_t)k};
        float h2[kPerThread], w2[kPerThread], h1[kPerThread], wp[kPerThread], hid[kPerThread], w1[kPerThread];
        // the rows first: loads return in the order of their requests, and the tail's arithmetic should not wait for the weights
        slice.load_f16(tail.h2, h2);
        slice.load_bf16(tail.w_postffn2, w2);
        slice.load_f16(tail.h1, h1);
        slice.load_bf16(tail.w_postffn, wp);
        slice.load_f16(tail.hidden, hid);
        slice.load_bf16(tail.w_postffn1, w1);
        XNormStage stage;
        stage.request_weight(norm_w, k);
        if (t0 < ntiles) request(ta, t0);
        if (t1 < ntiles) request(tb, t1);
        layer_tail_row<true>((uint32_t)k, h2, w2, h1, wp, hid, w1, tail.eps, tail.layer_scalar, norm_partial + 4);
        if (blockIdx.x == 0) slice.store_f16(tail.hidden_out, hid);
        stage.xr[0] = pack_half8(hid);
        stage.xr[1] = pack_half8(hid + 8);
        stage.xr[2] = stage.xr[3] = u32x4{0u, 0u, 0u, 0u};
        stage.publish(eps, k, xa, xsum, norm_partial);
    } else if constexpr (MODE == 1) {
        XNormStage stage;
        stage.request(x, norm_w, k);
        if (t0 < ntiles) request(ta, t0);
        if (t1 < ntiles) request(tb, t1);
        stage.publish(eps, k, xa, xsum, norm_partial);
    } else {
        XStage stage;
        stage.request(x, k);
        if (t0 < ntiles) request(ta, t0);
        if (t1 < ntiles) request(tb, t1);
        stage.publish(k, xa, xsum);
    }
    if (t0 >= ntiles) return;
    rs.init_x_lds(xa, xsum, k);
    auto emit = [&](const typename RowStream<RT, NP>::Tile &t, long at) {
        int seg;
        long local;
        locate(at, seg, local);
        float out[RT];
        rs.template reduce<SD>(t, out);
        if (lane == 0) {
#pragma unroll
            for (int r = 0; r < RT; ++r)
                if (local * RT + r < (long)g.rows[seg]) g.y[seg][local * RT + r] = (half_t)out[r];
        }
    };
    for (;;) {
        emit(ta, t0);
        t0 += 2 * nwaves;
        if (t0 < ntiles) request(ta, t0);
        if (t1 >= ntiles) break;
        emit(tb, t1);
        t1 += 2 * nwaves;
        if (t1 < ntiles) request(tb, t1);
        if (t0 >= ntiles) break;
    }
}

template <int RT, int NP, int SD, bool FUSE_NORM>
__global__ __launch_bounds__(256, 4) void qkv_gemv_long_kernel(GemvSegments g, const half_t *x, const uint16_t *norm_w, float eps, int k) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ float norm_partial[4];
    qkv_gemv_long_body<RT, NP, SD, FUSE_NORM ? 1 : 0>(g, x, norm_w, eps, k, TailFuse{}, xa, xsum, norm_partial);
}
// the rows of the tail live in registers beside the two weight tiles: two blocks per CU
template <int RT, int NP, int SD>
__global__ __launch_bounds__(256, 2) void qkv_gemv_after_tail_kernel(GemvSegments g, TailFuse tail, const uint16_t *norm_w, float eps, int k) {
    __shared__ __align__(16) u32x4 xa[XStage::kMaxK / 8];
    __shared__ float xsum[XStage::kMaxK / 32];
    __shared__ float norm_partial[16];
    qkv_gemv_long_body<RT, NP, SD, 2>(g, nullptr, norm_w, eps, k, tail, xa, xsum, norm_partial);
}

// K <= 1024: each wave covers 2 * NPASS consecutive rows, one row per half-wave per pass.
template <int NPASS, int SD, typename OutT>
__global__ __launch_bounds__(256) void gemv4_short_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                          const half_t *x, OutT *y, long m, int k) {
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long row0 = wave * (2 * NPASS);
    if (row0 >= m) return;
    ShortRows sr;
    sr.init(x, k, lane);
    ShortRows::Pair t[NPASS];
#pragma unroll
    for (int p = 0; p < NPASS; ++p) sr.load(t[p], W, S, B, row0 + 2 * p, m, k);
#pragma unroll
    for (int p = 0; p < NPASS; ++p) {
        float lo, hi;
        sr.template reduce<SD>(t[p], lo, hi);
        if (lane == 0) {
            if (row0 + 2 * p < m) store_out(y, row0 + 2 * p, lo);
            if (row0 + 2 * p + 1 < m) store_out(y, row0 + 2 * p + 1, hi);
        }
    }
}

template <int BITS, int SD, typename OutT>
__global__ __launch_bounds__(256) void gemv_generic_kernel(const uint8_t *W, const uint8_t *S, const uint8_t *B,
                                                           const half_t *x, OutT *y, long m, int k) {
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    const int groups = k >> 6;
    const size_t row_bytes = BITS == 4 ? (size_t)(k >> 1) : (size_t)k;
    for (long row = wave; row < m; row += nwaves) {
        float v;
        if constexpr (BITS == 4)
            v = generic_row_dot<SD>(W + row * row_bytes, S + (size_t)row * groups * 2, B + (size_t)row * groups * 2, x, k, lane);
        else
            v = generic_row_dot8<SD>(W + row * row_bytes, S + (size_t)row * groups * 2, B + (size_t)row * groups * 2, x, k, lane);
        if (lane == 0) store_out(y, row, v);
    }
}

// int8, 16-byte aligned rows and activations: lanes stride over 16-byte chunks (16 elements, a quarter group).
template <int SD, typename OutT>
__global__ __launch_bounds__(256) void gemv8_aligned_kernel(const uint8_t *W, const uint16_t *S, const uint16_t *B,
                                                            const half_t *x, OutT *y, long m, int k) {
    const int lane = threadIdx.x & 63;
    const long wave = ((long)blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const long nwaves = ((long)gridDim.x * blockDim.x) >> 6;
    const int groups = k >> 6;
    const int chunks = k >> 4;
    for (long row = wave; row < m; row += nwaves) {
        float acc = 0.0f;
        for (int c = lane; c < chunks; c += kWave) {
            const u32x4 w = load16(W + (size_t)row * k + (size_t)c * 16);
            const u32x4 xa = load16(x + c * 16), xb = load16(x + c * 16 + 8);
            const float s = sb_to_f32<SD>(S[(size_t)row * groups + (c >> 2)]);
            const float b = sb_to_f32<SD>(B[(size_t)row * groups + (c >> 2)]);
            float dot = 0.0f, sum = 0.0f;
#pragma unroll
            for (int i = 0; i < 16; ++i) {
                const uint32_t xw = i < 8 ? xa[i >> 1] : xb[(i - 8) >> 1];
                const float xv = (float)__builtin_bit_cast(half_t, (uint16_t)((i & 1) ? (xw >> 16) : (xw & 0xFFFFu)));
                const float q = (float)((w[i >> 2] >> (8 * (i & 3))) & 0xFFu);
                dot = fmaf(q, xv, dot);
                sum += xv;
            }
            acc = fmaf(s, dot, acc);
            acc = fmaf(b, sum, acc);
        }
        const float v = wave_sum(acc);
        if (lane == 0) store_out(y, row, v);
    }
}

// ------------------------------------------------------------------------------------------------ primitives
__global__ __launch_bounds__(256) void gelu_mul_kernel(const half_t *gate, const half_t *up, half_t *out, uint32_t count) {
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= count) return;
    out[i] = (half_t)(gelu_tanh((float)gate[i]) * (float)up[i]);
}

// 16-byte aligned operands, count % 8 == 0: eight elements a thread, the same arithmetic per element
__global__ __launch_bounds__(256) void gelu_mul_vec_kernel(const half_t *gate, const half_t *up, half_t *out, uint32_t count) {
    const uint32_t i = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
    if (i >= count) return;
    const uint4 g_raw = *reinterpret_cast<const uint4 *>(gate + i);
    const uint4 u_raw = *reinterpret_cast<const uint4 *>(up + i);
    const half_t *g = reinterpret_cast<const half_t *>(&g_raw);
    const half_t *u = reinterpret_cast<const half_t *>(&u_raw);
    uint4 packed;
    half_t *o = reinterpret_cast<half_t *>(&packed);
#pragma unroll
    for (uint32_t e = 0; e < 8; ++e) o[e] = (half_t)(gelu_tanh((float)g[e]) * (float)u[e]);
    *reinterpret_cast<uint4 *>(out + i) = packed;
}

// One row of RMSNorm by a 256-thread block: out = half(x * inv [* weight]), weight bf16.  In place is fine.
template <bool WEIGHTED>
__device__ __forceinline__ void rmsnorm_row_scalar(const half_t *x, const uint16_t *weight, half_t *out, uint32_t d, float eps, float *partial) {
    const float inv = block_rms_inv(x, d, eps, partial);
    for (uint32_t i = threadIdx.x; i < d; i += blockDim.x) {
        if constexpr (WEIGHTED) out[i] = (half_t)((float)x[i] * inv * bf16_to_f32(weight[i]));
        else out[i] = (half_t)((float)x[i] * inv);
    }
}

// 16-byte aligned operands, d % 8 == 0, d <= 2048 * PASSES: every thread requests all of its (at most PASSES) 8-element
// chunks of x and of the weight up front, so the row costs one memory round trip instead of one per element.
template <int PASSES, bool WEIGHTED>
__device__ __forceinline__ void rmsnorm_row_vec(const half_t *x, const uint16_t *weight, half_t *out, uint32_t d, float eps, float *partial) {
    u32x4 xr[PASSES], wr[PASSES];
    float acc = 0.0f;
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const uint32_t i = (threadIdx.x + 256u * p) * 8u;
        xr[p] = wr[p] = u32x4{0u, 0u, 0u, 0u};
        if (i < d) {
            xr[p] = load16(x + i);
            if constexpr (WEIGHTED) wr[p] = load16(weight + i);
        }
    }
#pragma unroll
    for (int p = 0; p < PASSES; ++p)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t h = as_half2(xr[p][j]);
            acc = fmaf((float)h[0], (float)h[0], acc);
            acc = fmaf((float)h[1], (float)h[1], acc);
        }
    acc = wave_sum(acc);
    if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
    __syncthreads();
    const float inv = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)d + eps);
#pragma unroll
    for (int p = 0; p < PASSES; ++p) {
        const uint32_t i = (threadIdx.x + 256u * p) * 8u;
        if (i < d) {
            u32x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half2_t h = as_half2(xr[p][j]);
                half2_t n;
                if constexpr (WEIGHTED) {
                    const uint32_t wv = wr[p][j];
                    n[0] = (half_t)((float)h[0] * inv * __uint_as_float(wv << 16));
                    n[1] = (half_t)((float)h[1] * inv * __uint_as_float(wv & 0xFFFF0000u));
                } else {
                    n[0] = (half_t)((float)h[0] * inv);
                    n[1] = (half_t)((float)h[1] * inv);
                }
                o[j] = as_u32(n);
            }
            *reinterpret_cast<u32x4 *>(out + i) = o;
        }
    }
}

// Rows of a block: grid (heads, tokens), row (t, h) = x + t * token_stride + h * d, one shared weight row [d].  PASSES > 0
// says that d and the weight allow the vector path; a row takes it when its own addresses do, exactly as a single-row call
// on that row would, so a block of rows equals the rows done one by one, bit for bit.
template <int PASSES, bool WEIGHTED>
__global__ __launch_bounds__(256) void rmsnorm_rows_kernel(const half_t *x, const uint16_t *weight, half_t *out, uint32_t d, float eps,
                                                           uint32_t token_stride) {
    __shared__ float partial[4];
    const size_t row = (size_t)blockIdx.y * token_stride + (size_t)blockIdx.x * d;
    const half_t *xr = x + row;
    half_t *outr = out + row;
    if constexpr (PASSES > 0) {
        if ((reinterpret_cast<uintptr_t>(xr) | reinterpret_cast<uintptr_t>(outr)) % 16 == 0) {
            rmsnorm_row_vec<PASSES, WEIGHTED>(xr, weight, outr, d, eps, partial);
            return;
        }
    }
    rmsnorm_row_scalar<WEIGHTED>(xr, weight, outr, d, eps, partial);
}

template <int BITS>
int32_t dequantize_entry(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t wo, const void *scales, uint64_t so,
                         const void *biases, uint64_t bo, void *out, uint64_t oo, uint32_t m, uint32_t n, tf_dtype sd) {
    TF_REQUIRE(ctx, ctx && weights && scales && biases && out, TF_ERR_INVALID_ARGUMENT, "dequantize: null argument");
    TF_REQUIRE(ctx, m > 0 && n > 0 && n % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "dequantize: n=%u must be a positive multiple of 64", n);
    TF_REQUIRE(ctx, so % 2 == 0 && bo % 2 == 0 && oo % 4 == 0, TF_ERR_INVALID_ARGUMENT, "dequantize: misaligned offset");
    TF_REQUIRE(ctx, sd == TF_BF16 || sd == TF_FP16, TF_ERR_INVALID_ARGUMENT, "dequantize: scale dtype must be bf16 or fp16");
    const uint8_t *w = at(weights, wo);
    const uint16_t *s = reinterpret_cast<const uint16_t *>(at(scales, so));
    const uint16_t *b = reinterpret_cast<const uint16_t *>(at(biases, bo));
    TF_REQUIRE(ctx, aligned(s, 2) && aligned(b, 2) && aligned(at(out, oo), 4), TF_ERR_INVALID_ARGUMENT, "dequantize: misaligned pointer");
    float *o = reinterpret_cast<float *>(at(out, oo));
    const uint64_t pairs = (uint64_t)m * (n / 2);
    const uint32_t grid = (uint32_t)std::min<uint64_t>((pairs + 255) / 256, (uint64_t)ctx->num_cus * 32);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (sd == TF_BF16) hipLaunchKernelGGL((dequantize_kernel<BITS, 0>), dim3(grid), dim3(256), 0, st, w, s, b, o, m, n);
    else hipLaunchKernelGGL((dequantize_kernel<BITS, 1>), dim3(grid), dim3(256), 0, st, w, s, b, o, m, n);
    return check_launch(ctx, "dequantize");
}

}  // namespace

namespace tfk {

// Shared by tf_dequant_int4_gemv, the shared expert and the logits head.
template <int SD, typename OutT>
static int32_t launch_gemv4_typed(tf_ctx *ctx, hipStream_t st, const uint8_t *w, const uint8_t *s, const uint8_t *b,
                                  const half_t *x, OutT *y, uint32_t m, uint32_t n, const uint16_t *norm_w, float eps) {
    const bool fast = aligned16(w) && aligned16(x);
    if (fast && n <= 1024) {
        constexpr int NPASS = 4;
        const long waves = ((long)m + 2 * NPASS - 1) / (2 * NPASS);
        const uint32_t grid = (uint32_t)((waves + 3) / 4);
        hipLaunchKernelGGL((gemv4_short_kernel<NPASS, SD, OutT>), dim3(grid), dim3(256), 0, st, w, s, b, x, y, (long)m, (int)n);
        return check_launch(ctx, "gemv4_short");
    }
    const LongPlan plan = plan_long_rows((int)n);
    if (fast && plan.rt > 0) {
        const long ntiles = ((long)m + plan.rt - 1) / plan.rt;
        const long max_blocks = (long)ctx->num_cus * ctx->stream_blocks_per_cu;
        const uint32_t grid = (uint32_t)std::max<long>(1, std::min<long>((ntiles + 3) / 4, max_blocks));
#define TF_LONG_CASE(RT_, NP_)                                                                                          \
    if (plan.rt == RT_ && plan.np == NP_) {                                                                             \
        if (norm_w)                                                                                                     \
            hipLaunchKernelGGL((gemv4_long_kernel<RT_, NP_, SD, OutT, true>), dim3(grid), dim3(256), 0, st, w, s,       \
                               b, x, norm_w, eps, y, (long)m, (int)n);                                                  \
        else                                                                                                            \
            hipLaunchKernelGGL((gemv4_long_kernel<RT_, NP_, SD, OutT, false>), dim3(grid), dim3(256), 0, st, w, s,      \
                               b, x, norm_w, eps, y, (long)m, (int)n);                                                  \
        return check_launch(ctx, "gemv4_long");                                                                         \
    }
        TF_LONG_CASE(1, 1) TF_LONG_CASE(1, 2) TF_LONG_CASE(1, 3) TF_LONG_CASE(1, 4)
        TF_LONG_CASE(2, 1) TF_LONG_CASE(2, 2) TF_LONG_CASE(2, 3) TF_LONG_CASE(2, 4)
        TF_LONG_CASE(4, 1) TF_LONG_CASE(4, 2) TF_LONG_CASE(4, 3) TF_LONG_CASE(4, 4)
#undef TF_LONG_CASE
    }
    const uint32_t grid = (uint32_t)std::min<long>(((long)m + 3) / 4, (long)ctx->num_cus * 16);
    hipLaunchKernelGGL((gemv_generic_kernel<4, SD, OutT>), dim3(grid), dim3(256), 0, st, w, s, b, x, y, (long)m, (int)n);
    return check_launch(ctx, "gemv4_generic");
}

bool gemv4_can_fuse_norm(const uint8_t *w, const void *x, const void *norm_w, uint32_t n) {
    return aligned16(w) && aligned16(x) && aligned16(norm_w) && n > 1024 && n <= (uint32_t)kMaxFusedNormD && plan_long_rows((int)n).rt > 0;
}

// norm_w != nullptr: x is the raw hidden vector, normalised inside the kernel; only legal when gemv4_can_fuse_norm().
int32_t launch_gemv4(tf_ctx *ctx, hipStream_t st, const uint8_t *w, const uint8_t *s, const uint8_t *b, const void *x,
                     void *y, uint32_t m, uint32_t n, tf_dtype sd, tf_dtype od, const void *norm_w, float eps) {
    const half_t *xh = static_cast<const half_t *>(x);
    const uint16_t *nw = static_cast<const uint16_t *>(norm_w);
    if (sd == TF_BF16) {
        if (od == TF_FP16) return launch_gemv4_typed<0, half_t>(ctx, st, w, s, b, xh, static_cast<half_t *>(y), m, n, nw, eps);
        return launch_gemv4_typed<0, float>(ctx, st, w, s, b, xh, static_cast<float *>(y), m, n, nw, eps);
    }
    if (od == TF_FP16) return launch_gemv4_typed<1, half_t>(ctx, st, w, s, b, xh, static_cast<half_t *>(y), m, n, nw, eps);
    return launch_gemv4_typed<1, float>(ctx, st, w, s, b, xh, static_cast<float *>(y), m, n, nw, eps);
}

// weight == nullptr: no scale.  heads x tokens rows of d elements, token rows token_stride elements apart.
int32_t launch_rmsnorm_rows(tf_ctx *ctx, hipStream_t st, const void *x, const void *w, void *out, uint32_t d, uint32_t heads, uint32_t tokens,
                            uint32_t token_stride, float eps, const char *who) {
    const half_t *xh = static_cast<const half_t *>(x);
    const uint16_t *wh = static_cast<const uint16_t *>(w);
    half_t *oh = static_cast<half_t *>(out);
    const bool vec = (w == nullptr || aligned16(w)) && d % 8 == 0 && d <= 16384;
    const int passes = !vec ? 0 : d <= 2048 ? 1 : d <= 4096 ? 2 : d <= 8192 ? 4 : 8;
    const dim3 grid(heads, tokens);
#define TF_NORM_ROWS(P_)                                                                                                       \
    case P_:                                                                                                                   \
        if (w) hipLaunchKernelGGL((rmsnorm_rows_kernel<P_, true>), grid, dim3(256), 0, st, xh, wh, oh, d, eps, token_stride);   \
        else hipLaunchKernelGGL((rmsnorm_rows_kernel<P_, false>), grid, dim3(256), 0, st, xh, wh, oh, d, eps, token_stride);    \
        break;
    switch (passes) {
        TF_NORM_ROWS(1) TF_NORM_ROWS(2) TF_NORM_ROWS(4) TF_NORM_ROWS(8)
        default:
            if (w) hipLaunchKernelGGL((rmsnorm_rows_kernel<0, true>), grid, dim3(256), 0, st, xh, wh, oh, d, eps, token_stride);
            else hipLaunchKernelGGL((rmsnorm_rows_kernel<0, false>), grid, dim3(256), 0, st, xh, wh, oh, d, eps, token_stride);
            break;
    }
#undef TF_NORM_ROWS
    return check_launch(ctx, who);
}

int32_t launch_rmsnorm_bf16w(tf_ctx *ctx, hipStream_t st, const void *x, const void *w, void *out, uint32_t d, float eps) {
    return launch_rmsnorm_rows(ctx, st, x, w, out, d, 1, 1, 0, eps, "rmsnorm_bf16w");
}

// argument checks shared by the RMSNorm entry points
int32_t rmsnorm_rows_entry(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight, uint64_t weight_offset, bool weighted,
                           void *out, uint64_t out_offset, uint32_t d, uint32_t heads, uint32_t tokens, uint32_t token_stride, float eps,
                           const char *who) {
    TF_REQUIRE(ctx, ctx && x && out && (!weighted || weight), TF_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    TF_REQUIRE(ctx, tokens > 0, TF_ERR_INVALID_ARGUMENT, "%s: queryCount must be positive", who);
    TF_REQUIRE(ctx, d > 0, TF_ERR_INVALID_ARGUMENT, "%s: headDim must be positive", who);
    TF_REQUIRE(ctx, heads > 0, TF_ERR_INVALID_ARGUMENT, "%s: numHeads must be positive", who);
    TF_REQUIRE(ctx, tokens == 1 || (uint64_t)token_stride >= (uint64_t)d * heads, TF_ERR_INVALID_ARGUMENT, "%s: token stride is too small", who);
    TF_REQUIRE(ctx, heads <= 65535 && tokens <= 65535, TF_ERR_INVALID_ARGUMENT, "%s: more than 65535 heads or tokens", who);
    TF_REQUIRE(ctx, x_offset % 2 == 0 && out_offset % 2 == 0 && (!weighted || weight_offset % 2 == 0), TF_ERR_INVALID_ARGUMENT,
               "%s: offsets must be 2-byte aligned", who);
    return launch_rmsnorm_rows(ctx, static_cast<hipStream_t>(stream), at(x, x_offset), weighted ? at(weight, weight_offset) : nullptr,
                               at(out, out_offset), d, heads, tokens, token_stride, eps, who);
}

int32_t launch_gelu_mul(tf_ctx *ctx, hipStream_t st, const void *gate, const void *up, void *out, uint32_t count) {
    if (count % 8 == 0 && aligned16(gate) && aligned16(up) && aligned16(out))
        hipLaunchKernelGGL(gelu_mul_vec_kernel, dim3((count / 8 + 255) / 256), dim3(256), 0, st, static_cast<const half_t *>(gate),
                           static_cast<const half_t *>(up), static_cast<half_t *>(out), count);
    else
        hipLaunchKernelGGL(gelu_mul_kernel, dim3((count + 255) / 256), dim3(256), 0, st, static_cast<const half_t *>(gate),
                           static_cast<const half_t *>(up), static_cast<half_t *>(out), count);
    return check_launch(ctx, "gelu_mul_fp16");
}

int32_t validate_gemv(tf_ctx *ctx, const char *who, const void *weights, uint64_t wo, const void *scales, uint64_t so,
                      const void *biases, uint64_t bo, const void *x, uint64_t xo, const void *y, uint64_t yo,
                      uint32_t m, uint32_t n, tf_dtype sd, tf_dtype od, unsigned weights_align) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "%s: null context", who);
    TF_REQUIRE(ctx, weights && scales && biases && x && y, TF_ERR_INVALID_ARGUMENT, "%s: null buffer", who);
    TF_REQUIRE(ctx, m > 0, TF_ERR_INVALID_ARGUMENT, "%s: m must be positive", who);
    TF_REQUIRE(ctx, n > 0 && n % TF_GROUP_SIZE == 0, TF_ERR_INVALID_ARGUMENT, "%s: N must be a multiple of 64, got %u", who, n);
    TF_REQUIRE(ctx, aligned(at(weights, wo), weights_align), TF_ERR_INVALID_ARGUMENT, "%s needs a %u-aligned weightsOffset, got %llu", who,
               weights_align, (unsigned long long)wo);
    TF_REQUIRE(ctx, aligned(at(scales, so), 2) && aligned(at(biases, bo), 2) && aligned(at(x, xo), 2), TF_ERR_INVALID_ARGUMENT,
               "%s: scales, biases and x must be 2-byte aligned", who);
    TF_REQUIRE(ctx, sd == TF_BF16 || sd == TF_FP16, TF_ERR_INVALID_ARGUMENT, "%s: scale dtype must be bf16 or fp16", who);
    TF_REQUIRE(ctx, od == TF_FP16 || od == TF_FP32, TF_ERR_INVALID_ARGUMENT, "%s: output dtype must be fp16 or fp32", who);
    TF_REQUIRE(ctx, aligned(at(y, yo), od == TF_FP16 ? 2 : 4), TF_ERR_INVALID_ARGUMENT, "%s: misaligned output", who);
    return TF_OK;
}

}  // namespace tfk

extern "C" {

int32_t tf_dequantize_int4_affine(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset,
                                  const void *scales, uint64_t scales_offset, const void *biases, uint64_t biases_offset,
                                  void *out_f32, uint64_t out_offset, uint32_t m, uint32_t n, tf_dtype scale_dtype) {
    return dequantize_entry<4>(ctx, stream, weights, weights_offset, scales, scales_offset, biases, biases_offset, out_f32,
                               out_offset, m, n, scale_dtype);
}

int32_t tf_dequantize_int8_affine(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset,
                                  const void *scales, uint64_t scales_offset, const void *biases, uint64_t biases_offset,
                                  void *out_f32, uint64_t out_offset, uint32_t m, uint32_t n, tf_dtype scale_dtype) {
    return dequantize_entry<8>(ctx, stream, weights, weights_offset, scales, scales_offset, biases, biases_offset, out_f32,
                               out_offset, m, n, scale_dtype);
}

int32_t tf_dequant_int4_gemv(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                             uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *x,
                             uint64_t x_offset, void *y, uint64_t y_offset, uint32_t m, uint32_t n, tf_dtype scale_dtype,
                             tf_dtype out_dtype) {
    const int32_t rc = validate_gemv(ctx, "dequant_int4_gemv", weights, weights_offset, scales, scales_offset, biases,
                                     biases_offset, x, x_offset, y, y_offset, m, n, scale_dtype, out_dtype, 2);
    if (rc != TF_OK) return rc;
    return launch_gemv4(ctx, static_cast<hipStream_t>(stream), at(weights, weights_offset), at(scales, scales_offset),
                        at(biases, biases_offset), at(x, x_offset), at(y, y_offset), m, n, scale_dtype, out_dtype);
}

int32_t tf_dequant_int8_gemv(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                             uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *x,
                             uint64_t x_offset, void *y, uint64_t y_offset, uint32_t m, uint32_t n, tf_dtype scale_dtype,
                             tf_dtype out_dtype) {
    const int32_t rc = validate_gemv(ctx, "dequant_int8_gemv", weights, weights_offset, scales, scales_offset, biases,
                                     biases_offset, x, x_offset, y, y_offset, m, n, scale_dtype, out_dtype, 1);
    if (rc != TF_OK) return rc;
    const uint8_t *w = at(weights, weights_offset);
    const uint8_t *s = at(scales, scales_offset);
    const uint8_t *b = at(biases, biases_offset);
    const half_t *xh = reinterpret_cast<const half_t *>(at(x, x_offset));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t grid = (uint32_t)std::min<long>(((long)m + 3) / 4, (long)ctx->num_cus * 16);
    const bool fast = aligned16(w) && aligned16(xh);
#define TF_GEMV8(SD_, OUT_)                                                                                             \
    do {                                                                                                                \
        OUT_ *yo = reinterpret_cast<OUT_ *>(at(y, y_offset));                                                           \
        if (fast)                                                                                                       \
            hipLaunchKernelGGL((gemv8_aligned_kernel<SD_, OUT_>), dim3(grid), dim3(256), 0, st, w,                      \
                               reinterpret_cast<const uint16_t *>(s), reinterpret_cast<const uint16_t *>(b), xh, yo,    \
                               (long)m, (int)n);                                                                        \
        else                                                                                                            \
            hipLaunchKernelGGL((gemv_generic_kernel<8, SD_, OUT_>), dim3(grid), dim3(256), 0, st, w, s, b, xh, yo,      \
                               (long)m, (int)n);                                                                        \
    } while (0)
    if (scale_dtype == TF_BF16) {
        if (out_dtype == TF_FP16) TF_GEMV8(0, half_t); else TF_GEMV8(0, float);
    } else {
        if (out_dtype == TF_FP16) TF_GEMV8(1, half_t); else TF_GEMV8(1, float);
    }
#undef TF_GEMV8
    return check_launch(ctx, "gemv8");
}

int32_t tf_gelu_mul_fp16(tf_ctx *ctx, tf_stream stream, const void *gate, uint64_t gate_offset, const void *up,
                         uint64_t up_offset, void *out, uint64_t out_offset, uint32_t count) {
    TF_REQUIRE(ctx, ctx && gate && up && out, TF_ERR_INVALID_ARGUMENT, "gelu_mul_fp16: null argument");
    TF_REQUIRE(ctx, gate_offset % 2 == 0 && up_offset % 2 == 0 && out_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT,
               "gelu_mul_fp16: offsets must be 2-byte aligned");
    if (count == 0) return TF_OK;
    return launch_gelu_mul(ctx, static_cast<hipStream_t>(stream), at(gate, gate_offset), at(up, up_offset), at(out, out_offset), count);
}

int32_t tf_rmsnorm_bf16w(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight,
                         uint64_t weight_offset, void *out, uint64_t out_offset, uint32_t d, float eps) {
    TF_REQUIRE(ctx, ctx && x && weight && out, TF_ERR_INVALID_ARGUMENT, "rmsnorm_bf16w: null argument");
    TF_REQUIRE(ctx, d > 0, TF_ERR_INVALID_ARGUMENT, "rmsnorm_bf16w: d must be positive");
    TF_REQUIRE(ctx, x_offset % 2 == 0 && weight_offset % 2 == 0 && out_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT,
               "rmsnorm_bf16w: offsets must be 2-byte aligned");
    return launch_rmsnorm_bf16w(ctx, static_cast<hipStream_t>(stream), at(x, x_offset), at(weight, weight_offset), at(out, out_offset), d, eps);
}

int32_t tf_rmsnorm_no_scale(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *out, uint64_t out_offset, uint32_t d, float eps) {
    return rmsnorm_rows_entry(ctx, stream, x, x_offset, nullptr, 0, false, out, out_offset, d, 1, 1, 0, eps, "rmsnorm_no_scale");
}

int32_t tf_rmsnorm_bf16w_perhead(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight, uint64_t weight_offset,
                                 void *out, uint64_t out_offset, uint32_t head_dim, uint32_t num_heads, float eps) {
    return rmsnorm_rows_entry(ctx, stream, x, x_offset, weight, weight_offset, true, out, out_offset, head_dim, num_heads, 1, 0, eps,
                              "rmsnorm_bf16w_perhead");
}

int32_t tf_rmsnorm_no_scale_perhead(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *out, uint64_t out_offset,
                                    uint32_t head_dim, uint32_t num_heads, float eps) {
    return rmsnorm_rows_entry(ctx, stream, x, x_offset, nullptr, 0, false, out, out_offset, head_dim, num_heads, 1, 0, eps,
                              "rmsnorm_no_scale_perhead");
}

int32_t tf_prefill_rmsnorm_bf16w_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight, uint64_t weight_offset,
                                       void *out, uint64_t out_offset, uint32_t tokens, uint32_t d, float eps) {
    return rmsnorm_rows_entry(ctx, stream, x, x_offset, weight, weight_offset, true, out, out_offset, d, 1, tokens, d, eps,
                              "prefill_rmsnorm_bf16w_block");
}

int32_t tf_prefill_rmsnorm_bf16w_perhead_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, const void *weight,
                                               uint64_t weight_offset, void *out, uint64_t out_offset, uint32_t query_count, uint32_t head_dim,
                                               uint32_t num_heads, uint32_t token_stride_elements, float eps) {
    return rmsnorm_rows_entry(ctx, stream, x, x_offset, weight, weight_offset, true, out, out_offset, head_dim, num_heads, query_count,
                              token_stride_elements, eps, "prefill_rmsnorm_bf16w_perhead_block");
}

int32_t tf_prefill_rmsnorm_no_scale_perhead_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *out, uint64_t out_offset,
                                                  uint32_t query_count, uint32_t head_dim, uint32_t num_heads, uint32_t token_stride_elements,
                                                  float eps) {
    return rmsnorm_rows_entry(ctx, stream, x, x_offset, nullptr, 0, false, out, out_offset, head_dim, num_heads, query_count,
                              token_stride_elements, eps, "prefill_rmsnorm_no_scale_perhead_block");
}

// The layer tail that makes the hidden vector of a tf_fused_layer_tail_norm_qkv_gemv call
struct TailCall {
    const void *h2, *shared_out, *hidden;
    void *hidden_out;
    const void *w_postffn1, *w_postffn2, *w_postffn;
    uint64_t w_postffn1_offset, w_postffn2_offset, w_postffn_offset;
    float eps, layer_scalar;
};

static int32_t qkv_gemv_entry(tf_ctx *ctx, tf_stream stream, const char *who, const void *norm_weight, uint64_t norm_weight_offset, float eps, const void *q_weights, uint64_t q_weights_offset, const void *q_scales,
                          uint64_t q_scales_offset, const void *q_biases, uint64_t q_biases_offset, const void *k_weights,
                          uint64_t k_weights_offset, const void *k_scales, uint64_t k_scales_offset, const void *k_biases,
                          uint64_t k_biases_offset, const void *v_weights, uint64_t v_weights_offset, const void *v_scales,
                          uint64_t v_scales_offset, const void *v_biases, uint64_t v_biases_offset, const void *x, void *q_out,
                          uint64_t q_out_offset, void *k_out, uint64_t k_out_offset, void *v_out, uint64_t v_out_offset, uint32_t q_rows,
                          uint32_t kv_rows, uint32_t n, tf_dtype scale_dtype, const TailCall *tail = nullptr) {
    const uint16_t *nw = norm_weight ? reinterpret_cast<const uint16_t *>(at(norm_weight, norm_weight_offset)) : nullptr;
    const void *w[3] = {q_weights, k_weights, v_weights};
    const void *s[3] = {q_scales, k_scales, v_scales};
    const void *b[3] = {q_biases, k_biases, v_biases};
    void *y[3] = {q_out, k_out, v_out};
    const uint64_t wo[3] = {q_weights_offset, k_weights_offset, v_weights_offset};
    const uint64_t so[3] = {q_scales_offset, k_scales_offset, v_scales_offset};
    const uint64_t bo[3] = {q_biases_offset, k_biases_offset, v_biases_offset};
    const uint64_t yo[3] = {q_out_offset, k_out_offset, v_out_offset};
    const uint32_t rows[3] = {q_rows, kv_rows, kv_rows};
    for (int i = 0; i < 3; ++i) {
        const int32_t rc = validate_gemv(ctx, who, w[i], wo[i], s[i], so[i], b[i], bo[i], x, 0, y[i], yo[i], rows[i], n,
                                         scale_dtype, TF_FP16, 2);
        if (rc != TF_OK) return rc;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const LongPlan plan = plan_long_rows((int)n);
    bool fast = aligned16(x) && n > 1024 && n <= (uint32_t)XStage::kMaxK && plan.rt > 0 && (!nw || aligned16(nw));
    for (int i = 0; i < 3; ++i) fast = fast && aligned16(at(w[i], wo[i]));
    // the one refusal left after the operand checks, ahead of the tail's launch: a refused call has launched nothing
    TF_REQUIRE(ctx, fast || !nw || n <= kMaxHeadD, TF_ERR_SCRATCH_TOO_SMALL, "%s: rows of %u values exceed the context's one-row buffer (%u)", who, n,
               kMaxHeadD);
    TailFuse tf = {};
    bool tail_fused = false;
    if (tail) {
        // x is tail->hidden_out, which the tail makes.  Inside the projection launch when that is the row streamer, every row and
        // norm weight moves in 16-byte pieces and the output is not a row the other blocks still read; a launch of its own otherwise.
        tf = {static_cast<const half_t *>(tail->h2), static_cast<const half_t *>(tail->shared_out), static_cast<const half_t *>(tail->hidden),
              static_cast<half_t *>(tail->hidden_out), reinterpret_cast<const uint16_t *>(at(tail->w_postffn2, tail->w_postffn2_offset)),
              reinterpret_cast<const uint16_t *>(at(tail->w_postffn, tail->w_postffn_offset)),
              reinterpret_cast<const uint16_t *>(at(tail->w_postffn1, tail->w_postffn1_offset)), tail->eps, tail->layer_scalar};
        // the output row (n halves) must not overlap any of the three input rows
        const void *ins[3] = {tf.h2, tf.h1, tf.hidden};
        const uintptr_t row_bytes = (uintptr_t)n * 2, out_at = (uintptr_t)tf.hidden_out;
        bool distinct = true;
        for (int i = 0; i < 3; ++i) distinct = distinct && ((uintptr_t)ins[i] + row_bytes <= out_at || out_at + row_bytes <= (uintptr_t)ins[i]);
        tail_fused = fast && nw && distinct && n <= kGlueMaxD && n % 8 == 0 && aligned16(tf.h2) && aligned16(tf.h1) && aligned16(tf.hidden) &&
                     aligned16(tf.hidden_out) && aligned16(tf.w_postffn2) && aligned16(tf.w_postffn) && aligned16(tf.w_postffn1);
        if (!tail_fused) {
            const int32_t rc = layer_tail_shared_norm_to(ctx, stream, tail->h2, tail->shared_out, tail->hidden, tail->hidden_out, tail->w_postffn1,
                                                         tail->w_postffn1_offset, tail->w_postffn2, tail->w_postffn2_offset, tail->w_postffn,
                                                         tail->w_postffn_offset, n, tail->eps, tail->layer_scalar);
            if (rc != TF_OK) return rc;
        }
    }
    if (fast) {
        GemvSegments g;
        uint32_t total = 0;
        for (int i = 0; i < 3; ++i) {
            g.W[i] = at(w[i], wo[i]);
            g.S[i] = at(s[i], so[i]);
            g.B[i] = at(b[i], bo[i]);
            g.y[i] = reinterpret_cast<half_t *>(at(y[i], yo[i]));
            g.rows[i] = rows[i];
            total += (rows[i] + plan.rt - 1) / plan.rt;
            g.tile_end[i] = total;
        }
        const long max_blocks = (long)ctx->num_cus * ctx->stream_blocks_per_cu;
        const uint32_t grid = (uint32_t)std::max<long>(1, std::min<long>(((long)total + 3) / 4, max_blocks));
        const half_t *xh = static_cast<const half_t *>(x);
#define TF_QKV_CASE(RT_, NP_)                                                                                             \
    if (plan.rt == RT_ && plan.np == NP_) {                                                                               \
        if (tail_fused) {                                                                                                 \
            if (scale_dtype == TF_BF16) hipLaunchKernelGGL((qkv_gemv_after_tail_kernel<RT_, NP_, 0>), dim3(grid), dim3(256), 0, st, g, tf, nw, eps, (int)n); \
            else hipLaunchKernelGGL((qkv_gemv_after_tail_kernel<RT_, NP_, 1>), dim3(grid), dim3(256), 0, st, g, tf, nw, eps, (int)n); \
        } else if (nw) {                                                                                                  \
            if (scale_dtype == TF_BF16) hipLaunchKernelGGL((qkv_gemv_long_kernel<RT_, NP_, 0, true>), dim3(grid), dim3(256), 0, st, g, xh, nw, eps, (int)n); \
            else hipLaunchKernelGGL((qkv_gemv_long_kernel<RT_, NP_, 1, true>), dim3(grid), dim3(256), 0, st, g, xh, nw, eps, (int)n); \
        } else {                                                                                                          \
            if (scale_dtype == TF_BF16) hipLaunchKernelGGL((qkv_gemv_long_kernel<RT_, NP_, 0, false>), dim3(grid), dim3(256), 0, st, g, xh, nw, eps, (int)n); \
            else hipLaunchKernelGGL((qkv_gemv_long_kernel<RT_, NP_, 1, false>), dim3(grid), dim3(256), 0, st, g, xh, nw, eps, (int)n); \
        }                                                                                                                 \
        return check_launch(ctx, who);                                                                                    \
    }
        TF_QKV_CASE(1, 1) TF_QKV_CASE(1, 2) TF_QKV_CASE(1, 3) TF_QKV_CASE(1, 4)
        TF_QKV_CASE(2, 1) TF_QKV_CASE(2, 2) TF_QKV_CASE(2, 3) TF_QKV_CASE(2, 4)
        TF_QKV_CASE(4, 1) TF_QKV_CASE(4, 2) TF_QKV_CASE(4, 3) TF_QKV_CASE(4, 4)
#undef TF_QKV_CASE
    }
    // any other shape or alignment: the three projections one after the other (same arithmetic per row), after the norm as
    // a launch of its own into the context's one-row buffer
    if (nw) {
        const int32_t rc = launch_rmsnorm_bf16w(ctx, st, x, nw, ctx->head_x_normed, n, eps);
        if (rc != TF_OK) return rc;
        x = ctx->head_x_normed;
    }
    for (int i = 0; i < 3; ++i) {
        const int32_t rc = launch_gemv4(ctx, st, at(w[i], wo[i]), at(s[i], so[i]), at(b[i], bo[i]), x, at(y[i], yo[i]), rows[i], n, scale_dtype, TF_FP16);
        if (rc != TF_OK) return rc;
    }
    return TF_OK;
}


int32_t tf_fused_qkv_gemv(tf_ctx *ctx, tf_stream stream, const void *q_weights, uint64_t q_weights_offset, const void *q_scales,
                          uint64_t q_scales_offset, const void *q_biases, uint64_t q_biases_offset, const void *k_weights,
                          uint64_t k_weights_offset, const void *k_scales, uint64_t k_scales_offset, const void *k_biases,
                          uint64_t k_biases_offset, const void *v_weights, uint64_t v_weights_offset, const void *v_scales,
                          uint64_t v_scales_offset, const void *v_biases, uint64_t v_biases_offset, const void *x, void *q_out,
                          uint64_t q_out_offset, void *k_out, uint64_t k_out_offset, void *v_out, uint64_t v_out_offset, uint32_t q_rows,
                          uint32_t kv_rows, uint32_t n, tf_dtype scale_dtype) {
    return qkv_gemv_entry(ctx, stream, "fused_qkv_gemv", nullptr, 0, 0.0f, q_weights, q_weights_offset, q_scales, q_scales_offset, q_biases,
                          q_biases_offset, k_weights, k_weights_offset, k_scales, k_scales_offset, k_biases, k_biases_offset, v_weights,
                          v_weights_offset, v_scales, v_scales_offset, v_biases, v_biases_offset, x, q_out, q_out_offset, k_out, k_out_offset,
                          v_out, v_out_offset, q_rows, kv_rows, n, scale_dtype);
}

int32_t tf_fused_norm_qkv_gemv(tf_ctx *ctx, tf_stream stream, const void *norm_weight, uint64_t norm_weight_offset, float eps,
                               const void *q_weights, uint64_t q_weights_offset, const void *q_scales, uint64_t q_scales_offset,
                               const void *q_biases, uint64_t q_biases_offset, const void *k_weights, uint64_t k_weights_offset,
                               const void *k_scales, uint64_t k_scales_offset, const void *k_biases, uint64_t k_biases_offset,
                               const void *v_weights, uint64_t v_weights_offset, const void *v_scales, uint64_t v_scales_offset,
                               const void *v_biases, uint64_t v_biases_offset, const void *hidden, void *q_out, uint64_t q_out_offset,
                               void *k_out, uint64_t k_out_offset, void *v_out, uint64_t v_out_offset, uint32_t q_rows, uint32_t kv_rows,
                               uint32_t n, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx && norm_weight, TF_ERR_INVALID_ARGUMENT, "fused_norm_qkv_gemv: null argument");
    TF_REQUIRE(ctx, norm_weight_offset % 2 == 0 && aligned(norm_weight, 2), TF_ERR_INVALID_ARGUMENT, "fused_norm_qkv_gemv: misaligned norm weight");
    return qkv_gemv_entry(ctx, stream, "fused_norm_qkv_gemv", norm_weight, norm_weight_offset, eps, q_weights, q_weights_offset, q_scales,
                          q_scales_offset, q_biases, q_biases_offset, k_weights, k_weights_offset, k_scales, k_scales_offset, k_biases,
                          k_biases_offset, v_weights, v_weights_offset, v_scales, v_scales_offset, v_biases, v_biases_offset, hidden, q_out,
                          q_out_offset, k_out, k_out_offset, v_out, v_out_offset, q_rows, kv_rows, n, scale_dtype);
}

int32_t tf_fused_layer_tail_norm_qkv_gemv(tf_ctx *ctx, tf_stream stream, const void *h2, const void *shared_out, const void *hidden,
                                          void *hidden_out, const void *post_ffn1_weight, uint64_t post_ffn1_weight_offset,
                                          const void *post_ffn2_weight, uint64_t post_ffn2_weight_offset, const void *post_ffn_weight,
                                          uint64_t post_ffn_weight_offset, float tail_eps, float layer_scalar, const void *norm_weight,
                                          uint64_t norm_weight_offset, float eps, const void *q_weights, uint64_t q_weights_offset,
                                          const void *q_scales, uint64_t q_scales_offset, const void *q_biases, uint64_t q_biases_offset,
                                          const void *k_weights, uint64_t k_weights_offset, const void *k_scales, uint64_t k_scales_offset,
                                          const void *k_biases, uint64_t k_biases_offset, const void *v_weights, uint64_t v_weights_offset,
                                          const void *v_scales, uint64_t v_scales_offset, const void *v_biases, uint64_t v_biases_offset,
                                          void *q_out, uint64_t q_out_offset, void *k_out, uint64_t k_out_offset, void *v_out,
                                          uint64_t v_out_offset, uint32_t q_rows, uint32_t kv_rows, uint32_t n, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx && norm_weight && h2 && shared_out && hidden && hidden_out && post_ffn1_weight && post_ffn2_weight && post_ffn_weight,
               TF_ERR_INVALID_ARGUMENT, "fused_layer_tail_norm_qkv_gemv: null argument");
    TF_REQUIRE(ctx, norm_weight_offset % 2 == 0 && aligned(norm_weight, 2), TF_ERR_INVALID_ARGUMENT, "fused_layer_tail_norm_qkv_gemv: misaligned norm weight");
    TF_REQUIRE(ctx, n > 0 && n <= kGlueMaxD, TF_ERR_INVALID_ARGUMENT, "fused_layer_tail_norm_qkv_gemv: D must be in 1...4096, got %u", n);
    const TailCall tail = {h2, shared_out, hidden, hidden_out, post_ffn1_weight, post_ffn2_weight, post_ffn_weight, post_ffn1_weight_offset,
                           post_ffn2_weight_offset, post_ffn_weight_offset, tail_eps, layer_scalar};
    return qkv_gemv_entry(ctx, stream, "fused_layer_tail_norm_qkv_gemv", norm_weight, norm_weight_offset, eps, q_weights, q_weights_offset, q_scales,
                          q_scales_offset, q_biases, q_biases_offset, k_weights, k_weights_offset, k_scales, k_scales_offset, k_biases,
                          k_biases_offset, v_weights, v_weights_offset, v_scales, v_scales_offset, v_biases, v_biases_offset, hidden_out, q_out,
                          q_out_offset, k_out, k_out_offset, v_out, v_out_offset, q_rows, kv_rows, n, scale_dtype, &tail);
}

}  // extern "C"

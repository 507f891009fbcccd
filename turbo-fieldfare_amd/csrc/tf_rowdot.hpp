// Row-streaming int4 dot products for one wavefront.
//
// Three shapes of the same arithmetic  y = sum_g [ s_g * sum_k q_k x_k + b_g * sum_k x_k ]:
//
//   RowStream<RT, NP> a wave owns RT consecutive rows (RT * K/2 contiguous bytes) and reads them as one flat
//                     stream of 16-byte chunks: pass p, lane l reads chunk 64p + l, so every load instruction
//                     of the wave covers 1024 contiguous bytes.  The chunk -> (row, column) map is the same for
//                     every tile, so each lane keeps the activations of its <= NP column positions in registers
//                     for the lifetime of the wave.  Used for K > 1024 (2816, 2112, 4096, 8192 ...).
//   ShortRows         K <= 1024: a row is at most 32 chunks; each half-wave owns one row per pass, two rows per
//                     load instruction, one activation chunk per lane.
//   generic_row_dot   any K % 64 == 0 at any 2-byte alignment: 16-bit loads, fp32 FMAs (the slow, always-legal path).
//
// Scales/biases are read with 16-bit loads straight from their [rows, K/64] arrays (rows of the routed layout are
// only 2-byte aligned).
#pragma once

#include "tf_common.hpp"

namespace tfk {

// ------------------------------------------------------------------------------------------------ row stream
// A value that is the same in every lane, told to the compiler: arithmetic on it runs on the scalar unit.
template <typename T>
__device__ __forceinline__ T *uniform_ptr(T *p) {
    const uint64_t v = (uint64_t)p;
    const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v);
    const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
    return (T *)(((uint64_t)hi << 32) | lo);
}
__device__ __forceinline__ int uniform_int(int v) { return __builtin_amdgcn_readfirstlane(v); }
__device__ __forceinline__ uint32_t uniform_u32(uint32_t v) { return (uint32_t)__builtin_amdgcn_readfirstlane((int)v); }

// Every load is a bounds-checked buffer load: the tile base is wave-uniform and lives in a buffer descriptor (scalar
// registers), each lane keeps constant byte offsets, so a tile costs no address arithmetic on the vector unit and no
// branches.  The descriptor ends where the tile (or the matrix) ends: lanes without a chunk in the last pass and rows
// past the end of the matrix read zeros and contribute nothing.
typedef __amdgpu_buffer_rsrc_t rsrc_t;
// Cache policy of the packed-weight loads: non-temporal.  A launch reads every weight byte once, so keeping the lines in L2
// only evicts what is reused (activations, scales); a plain streaming read measures 7.0-7.2 TB/s with this hint against
// 6.5 TB/s without it, and the vocabulary-sized head 64 us against 69 us.
constexpr int kStreamOnce = 2;
__device__ __forceinline__ rsrc_t make_rsrc(const void *base, uint32_t bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)bytes, 0x00020000);
}

template <int RT, int NP>
struct RowStream {
    uint32_t woff[NP];   // byte offset of this lane's chunk inside the tile's weights
    uint32_t sboff[NP];  // byte offset of its (scale, bias) inside the tile's scale / bias block
    int row[NP];         // tile row served in pass p, -1 when idle
    int col[NP];         // chunk column inside that row
    half2_t xq[NP][16];
    float xs[NP];
    uint32_t row_bytes, sb_row_bytes;   // wave-uniform

    // chunk -> (row, column) map of this lane; independent of the data.
    // RT == 2 places the second row as the first row's mirror image: chunk c of row 0 sits in lane c % 64 of pass c / 64,
    // chunk c of row 1 in lane (c + 32) % 64 of pass NP - 1 - c / 64.  Each lane of row 1 then accumulates the same chunks
    // as the lane 32 places away does for row 0, and the wave sum is symmetric under that swap of half-waves (its last
    // step adds the two half-wave sums), so a row's dot product does not depend on its position in the tile: two rows
    // with identical bytes give identical sums, and an argmax over rows breaks ties exactly by index.  plan_long_rows
    // only offers RT == 2 where the two images do not overlap.  Other RT use the flat order (chunk 64 p + lane).
    __device__ __forceinline__ void init_map(int k, int lane) {
        const int nch = k >> 5;  // 16-byte chunks per row
        const int groups = k >> 6;
        row_bytes = (uint32_t)k >> 1;
        sb_row_bytes = (uint32_t)groups * 2u;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            int r, cc;
            bool valid;
            if constexpr (RT == 2) {
                const int c0 = lane + 64 * p;
                const int c1 = ((lane + 32) & 63) + 64 * (NP - 1 - p);
                const bool v0 = c0 < nch;
                valid = v0 || c1 < nch;
                r = v0 ? 0 : 1;
                cc = v0 ? c0 : c1;
            } else {
                const int c = lane + 64 * p;
                valid = c < RT * nch;
                r = c / nch;
                cc = c - r * nch;
            }
            col[p] = valid ? cc : 0;
            row[p] = valid ? r : -1;
            woff[p] = valid ? (uint32_t)r * row_bytes + (uint32_t)cc * 16u : 0xFFFFFFF0u;   // past the tile when !valid: reads zeros
            sboff[p] = valid ? (uint32_t)(r * groups + (cc >> 1)) * 2u : 0xFFFFFFF0u;
        }
    }

    // The activations of this lane's column positions, requested (load_x) and later arranged into registers
    // (arrange): a caller can put other loads between the two.  x must be 16-byte aligned.
    struct XRaw {
        u32x4 r[NP][4];
    };
    __device__ __forceinline__ void load_x(XRaw &raw, const half_t *x) const {
#pragma unroll
        for (int p = 0; p < NP; ++p)
#pragma unroll
            for (int d = 0; d < 4; ++d) raw.r[p][d] = load16(x + col[p] * 32 + d * 8);
    }
    __device__ __forceinline__ void arrange(const XRaw &raw) {
#pragma unroll
        for (int p = 0; p < NP; ++p) xs[p] = arrange_x(raw.r[p], xq[p]);
    }
    __device__ __forceinline__ void init_x(const half_t *x) {
        XRaw raw;
        load_x(raw, x);
        arrange(raw);
    }

    // The same from a block-wide LDS image written by XStage (below): xa[d * nch + c] holds word d of chunk column c
    // already in chunk_dot order, xsum[c] the column's sum.
    __device__ __forceinline__ void init_x_lds(const u32x4 *xa, const float *xsum, int k) {
        const int nch = k >> 5;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const u32x4 v = xa[d * nch + col[p]];
#pragma unroll
                for (int j = 0; j < 4; ++j) xq[p][4 * d + j] = as_half2(v[j]);
            }
            xs[p] = xsum[col[p]];
        }
    }

    struct Tile {
        u32x4 w[NP];
        uint16_t s[NP], b[NP];
    };

    // w_tile / s_tile / b_tile: wave-uniform bases of the tile; rows: rows of the matrix from the tile's first row on
    // (wave-uniform, >= 1).
    __device__ __forceinline__ void load(Tile &t, const uint8_t *w_tile, const uint8_t *s_tile, const uint8_t *b_tile,
                                         long rows) const {
        const uint32_t nr = rows < RT ? (uint32_t)rows : (uint32_t)RT;
        const rsrc_t rw = make_rsrc(w_tile, nr * row_bytes);
        const rsrc_t rs = make_rsrc(s_tile, nr * sb_row_bytes);
        const rsrc_t rb = make_rsrc(b_tile, nr * sb_row_bytes);
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            t.w[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rw, woff[p], 0, kStreamOnce));
            t.s[p] = __builtin_amdgcn_raw_buffer_load_b16(rs, sboff[p], 0, 0);
            t.b[p] = __builtin_amdgcn_raw_buffer_load_b16(rb, sboff[p], 0, 0);
        }
    }

    // out[r]: the dot product of tile row r, wave-uniform.  Wave-uniform control flow only (see chunk_dot).
    template <int SD>
    __device__ __forceinline__ void reduce(const Tile &t, float *out) const {
        float part[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p)
            part[p] = fmaf(sb_to_f32<SD>(t.s[p]), chunk_dot(t.w[p], xq[p]), sb_to_f32<SD>(t.b[p]) * xs[p]);
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float v = 0.0f;
#pragma unroll
            for (int p = 0; p < NP; ++p) v += (row[p] == r) ? part[p] : 0.0f;
            out[r] = wave_sum(v);
        }
    }
};

// Block-wide staging of an activation vector into LDS in chunk_dot order, shared by all waves of a 256-thread block:
// request() issues the global loads (k <= 8192, x 16-byte aligned), publish() arranges them, writes the image and
// ends with a barrier; a caller puts its weight loads between the two.  Every thread of the block must call both.
// With a norm weight (request_norm / publish_norm) the vector is first normalised as rmsnorm_bf16w does:
// half(x * rsqrt(mean(x^2) + eps) * w).
struct XStage {
    static constexpr int kMaxK = 8192;
    u32x4 r[4];

    __device__ __forceinline__ void request(const half_t *x, int k) {
        const int pieces = k >> 3;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int piece = threadIdx.x + 256 * i;
            r[i] = u32x4{0u, 0u, 0u, 0u};
            if (piece < pieces) r[i] = load16(x + piece * 8);
        }
    }

    // piece = 8 consecutive activations = word (piece & 3) of chunk column (piece >> 2)
    // xsum_stride: distance between the sums of neighbouring columns (1: one vector's sums side by side; a caller that keeps
    // several vectors' sums interleaved per column passes their count)
    static __device__ __forceinline__ void publish_piece(const u32x4 raw, int piece, int pieces, int nch, u32x4 *xa, float *xsum,
                                                         int xsum_stride = 1) {
        const half2_t sixteenth = {(half_t)0.0625f, (half_t)0.0625f};
        const uint32_t p01 = raw[0], p23 = raw[1], p45 = raw[2], p67 = raw[3];
        u32x4 o;
        o[0] = (p01 & 0xFFFFu) | (p45 << 16);
        o[1] = as_u32(as_half2((p01 >> 16) | (p45 & 0xFFFF0000u)) * sixteenth);
        o[2] = (p23 & 0xFFFFu) | (p67 << 16);
        o[3] = as_u32(as_half2((p23 >> 16) | (p67 & 0xFFFF0000u)) * sixteenth);
        float sum = 0.0f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const half2_t h = as_half2(raw[j]);
            sum += (float)h[0];
            sum += (float)h[1];
        }
        sum += dpp_f32<0xB1>(sum);   // the four pieces of a column sit in one aligned quad of lanes
        sum += dpp_f32<0x4E>(sum);
        if (piece < pieces) {
            xa[(piece & 3) * nch + (piece >> 2)] = o;
            if ((piece & 3) == 0) xsum[(piece >> 2) * xsum_stride] = sum;
        }
    }

    __device__ __forceinline__ void publish(int k, u32x4 *xa, float *xsum) const {
#pragma unroll
        for (int i = 0; i < 4; ++i) publish_piece(r[i], threadIdx.x + 256 * i, k >> 3, k >> 5, xa, xsum);
        __syncthreads();
    }
};

struct XNormStage {
    u32x4 xr[4], wr[4];

    __device__ __forceinline__ void request(const half_t *x, const uint16_t *w_bf16, int k) {
        const int pieces = k >> 3;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int piece = threadIdx.x + 256 * i;
            xr[i] = wr[i] = u32x4{0u, 0u, 0u, 0u};
            if (piece < pieces) {
                xr[i] = load16(x + piece * 8);
                wr[i] = load16(w_bf16 + piece * 8);
            }
        }
    }

    // the norm weight only: the caller fills xr itself
    __device__ __forceinline__ void request_weight(const uint16_t *w_bf16, int k) {
        const int pieces = k >> 3;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int piece = threadIdx.x + 256 * i;
            wr[i] = u32x4{0u, 0u, 0u, 0u};
            if (piece < pieces) wr[i] = load16(w_bf16 + piece * 8);
        }
    }

    // partial: 4 floats of LDS
    __device__ __forceinline__ void publish(float eps, int k, u32x4 *xa, float *xsum, float *partial) const {
        float acc = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half2_t h = as_half2(xr[i][j]);
                acc = fmaf((float)h[0], (float)h[0], acc);
                acc = fmaf((float)h[1], (float)h[1], acc);
            }
        acc = wave_sum(acc);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = acc;
        __syncthreads();
        const float inv = 1.0f / sqrtf((partial[0] + partial[1] + partial[2] + partial[3]) / (float)k + eps);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            u32x4 o;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const half2_t h = as_half2(xr[i][j]);
                half2_t n;
                n[0] = (half_t)((float)h[0] * inv * __uint_as_float(wr[i][j] << 16));
                n[1] = (half_t)((float)h[1] * inv * __uint_as_float(wr[i][j] & 0xFFFF0000u));
                o[j] = as_u32(n);
            }
            XStage::publish_piece(o, threadIdx.x + 256 * i, k >> 3, k >> 5, xa, xsum);
        }
        __syncthreads();
    }
};

// ------------------------------------------------------------------------------------------------ short rows
struct ShortRows {
    int col;       // chunk column of this lane (lane & 31), -1 if beyond the row
    int half;      // 0: lanes 0..31, 1: lanes 32..63
    half2_t xq[16];
    float xs;

    __device__ __forceinline__ void init_map(int k, int lane) {
        const int nch = k >> 5;
        const int c = lane & 31;
        half = lane >> 5;
        col = c < nch ? c : -1;
    }

    __device__ __forceinline__ void init_x(const half_t *x) {
        u32x4 xr[4];
#pragma unroll
        for (int d = 0; d < 4; ++d) xr[d] = load16(x + (col < 0 ? 0 : col) * 32 + d * 8);
        xs = arrange_x(xr, xq);
    }

    __device__ __forceinline__ void init(const half_t *x, int k, int lane) {
        init_map(k, lane);
        init_x(x);
    }

    struct Pair {
        u32x4 w;
        uint16_t s, b;
    };

    // Loads this lane's chunk of row (row0 + half) if that row exists.
    __device__ __forceinline__ void load(Pair &t, const uint8_t *w, const uint8_t *s, const uint8_t *b, long row0,
                                         long rows, int k) const {
        t.w = u32x4{0u, 0u, 0u, 0u};
        t.s = 0;
        t.b = 0;
        const long r = row0 + half;
        if (col >= 0 && r < rows) {
            const int groups = k >> 6;
            t.w = __builtin_nontemporal_load(reinterpret_cast<const u32x4 *>(w + (size_t)r * (k >> 1) + (size_t)col * 16));
            t.s = *reinterpret_cast<const uint16_t *>(s + ((size_t)r * groups + (col >> 1)) * 2);
            t.b = *reinterpret_cast<const uint16_t *>(b + ((size_t)r * groups + (col >> 1)) * 2);
        }
    }

    template <int SD>
    __device__ __forceinline__ void reduce(const Pair &t, float &lo, float &hi) const {
        const float part = fmaf(sb_to_f32<SD>(t.s), chunk_dot(t.w, xq), sb_to_f32<SD>(t.b) * xs);
        half_wave_sums(part, lo, hi);
    }
};

// ------------------------------------------------------------------------------------------------ generic
// One wave, one row, any even alignment: lanes stride over 32-bit words (8 nibbles) assembled from two 16-bit loads,
// exactly the access pattern the reference's kernels use for 2-byte-aligned tensors (dequant_int4.metal:127-134).
// Returns the wave-uniform dot product.
template <int SD>
__device__ __forceinline__ float generic_row_dot(const uint8_t *w_row, const uint8_t *s_row, const uint8_t *b_row,
                                                 const half_t *x, int k, int lane) {
    float acc = 0.0f;
    const int words = k >> 3;
    for (int wi = lane; wi < words; wi += kWave) {
        const uint16_t *wp = reinterpret_cast<const uint16_t *>(w_row + wi * 4);
        const uint32_t w4 = (uint32_t)wp[0] | ((uint32_t)wp[1] << 16);
        const int g = wi >> 3;
        const float s = sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(s_row + g * 2));
        const float b = sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(b_row + g * 2));
        float dot = 0.0f, sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const float xv = (float)x[wi * 8 + i];
            dot = fmaf((float)((w4 >> (4 * i)) & 0xFu), xv, dot);
            sum += xv;
        }
        acc = fmaf(s, dot, acc);
        acc = fmaf(b, sum, acc);
    }
    return wave_sum(acc);
}

// int8 analogue (one byte per element): lanes stride over 4-byte words assembled from bytes' 16-bit halves.
template <int SD>
__device__ __forceinline__ float generic_row_dot8(const uint8_t *w_row, const uint8_t *s_row, const uint8_t *b_row,
                                                  const half_t *x, int k, int lane) {
    float acc = 0.0f;
    const int words = k >> 2;
    for (int wi = lane; wi < words; wi += kWave) {
        const int g = wi >> 4;
        const float s = sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(s_row + g * 2));
        const float b = sb_to_f32<SD>(*reinterpret_cast<const uint16_t *>(b_row + g * 2));
        float dot = 0.0f, sum = 0.0f;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const float xv = (float)x[wi * 4 + i];
            dot = fmaf((float)w_row[wi * 4 + i], xv, dot);
            sum += xv;
        }
        acc = fmaf(s, dot, acc);
        acc = fmaf(b, sum, acc);
    }
    return wave_sum(acc);
}

// Picks the rows-per-tile and pass count of RowStream for a given K: best lane utilisation with NP <= 4 and RT <= max_rt.
// RT == 2 needs the two mirrored row images of RowStream::init_map to be disjoint: either each row has passes of its own
// (2 * passes per row == NP) or the shared middle pass holds at most 32 chunks of each row.
struct LongPlan {
    int rt, np;
};
inline LongPlan plan_long_rows(int k, int max_rt = 4) {
    const int nch = k / 32;
    LongPlan best{0, 0};
    double best_util = 0.0;
    const int rts[3] = {1, 2, 4};
    for (int i = 0; i < 3; ++i) {
        const int rt = rts[i];
        if (rt > max_rt) continue;
        const int np = (rt * nch + 63) / 64;
        if (np > 4) continue;
        if (rt == 2) {
            const int per_row = (nch + 63) / 64, tail = nch % 64;
            if (2 * per_row != np && !(tail != 0 && tail <= 32)) continue;
        }
        const double util = (double)(rt * nch) / (64.0 * np);
        if (util > best_util + 1e-9) {
            best_util = util;
            best = LongPlan{rt, np};
        }
    }
    return best;
}

}  // namespace tfk

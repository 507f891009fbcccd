// Row-streaming int4 dot products for one wavefront.
//
// Three shapes of the same arithmetic  y = sum_g [ s_g * sum_k q_k x_k + b_g * sum_k x_k ]:
//
//   LongRows<RT, NP>  a wave owns RT consecutive rows (RT * K/2 contiguous bytes) and reads them as one flat
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

// ------------------------------------------------------------------------------------------------ long rows
template <int RT, int NP>
struct LongRows {
    // per-lane constants
    int row[NP];    // row within the tile served by this lane in pass p (-1: lane idle in that pass)
    int col[NP];    // chunk column inside that row
    int sb[NP];     // row * groups + group: index of the (scale, bias) pair inside the tile's scale block
    half2_t xq[NP][16];
    float xs[NP];

    // chunk -> (row, column) map of this lane; independent of the data
    __device__ __forceinline__ void init_map(int k, int lane) {
        const int nch = k >> 5;  // 16-byte chunks per row
        const int groups = k >> 6;
        const int tot = RT * nch;
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const int c = lane + 64 * p;
            const bool valid = c < tot;
            const int cc = valid ? c : 0;
            const int r = cc / nch;
            col[p] = cc - r * nch;
            row[p] = valid ? r : -1;
            sb[p] = r * groups + (col[p] >> 1);
        }
    }

    // activations of this lane's column positions, kept in registers; x must be 16-byte aligned
    __device__ __forceinline__ void init_x(const half_t *x, int /*lane*/) {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            u32x4 xr[4];
#pragma unroll
            for (int d = 0; d < 4; ++d) xr[d] = load16(x + col[p] * 32 + d * 8);
            xs[p] = arrange_x(xr, xq[p]);
        }
    }

    __device__ __forceinline__ void init(const half_t *x, int k, int lane) {
        init_map(k, lane);
        init_x(x, lane);
    }

    struct Tile {
        u32x4 w[NP];
        uint16_t s[NP], b[NP];
    };

    // rows_left: rows of the matrix from the tile's first row on (>= 1); rows beyond it are not touched.
    __device__ __forceinline__ void load(Tile &t, const uint8_t *w_tile, const uint16_t *s_tile, const uint16_t *b_tile,
                                         int rows_left, int lane) const {
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            t.w[p] = u32x4{0u, 0u, 0u, 0u};
            t.s[p] = 0;
            t.b[p] = 0;
            if (row[p] >= 0 && row[p] < rows_left) {
                t.w[p] = load16(w_tile + (size_t)(lane + 64 * p) * 16);
                t.s[p] = s_tile[sb[p]];
                t.b[p] = b_tile[sb[p]];
            }
        }
    }

    // out[r]: the dot product of tile row r, wave-uniform
    template <int SD>
    __device__ __forceinline__ void reduce(const Tile &t, float *out) const {
        float part[NP];
#pragma unroll
        for (int p = 0; p < NP; ++p) {
            const float s = sb_to_f32<SD>(t.s[p]);
            const float b = sb_to_f32<SD>(t.b[p]);
            part[p] = fmaf(s, chunk_dot(t.w[p], xq[p]), b * xs[p]);   // idle lanes loaded zeros: contributes 0
        }
#pragma unroll
        for (int r = 0; r < RT; ++r) {
            float v = 0.0f;
#pragma unroll
            for (int p = 0; p < NP; ++p) v += (row[p] == r) ? part[p] : 0.0f;
            out[r] = wave_sum(v);
        }
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
            t.w = load16(w + (size_t)r * (k >> 1) + (size_t)col * 16);
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

// Picks the rows-per-tile and pass count of LongRows for a given K: best lane utilisation with NP <= 4.
struct LongPlan {
    int rt, np;
};
inline LongPlan plan_long_rows(int k) {
    const int nch = k / 32;
    LongPlan best{0, 0};
    double best_util = 0.0;
    const int rts[3] = {1, 2, 4};
    for (int i = 0; i < 3; ++i) {
        const int rt = rts[i];
        const int np = (rt * nch + 63) / 64;
        if (np > 4) continue;
        const double util = (double)(rt * nch) / (64.0 * np);
        if (util > best_util + 1e-9) {
            best_util = util;
            best = LongPlan{rt, np};
        }
    }
    return best;
}

}  // namespace tfk

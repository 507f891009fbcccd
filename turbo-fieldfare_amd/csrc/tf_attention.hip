// Single-token decode attention over an fp16 KV cache: split-KV online softmax (partial states per chunk, then a merge),
// sliding-window and full-causal, grouped-query, optional ring addressing of the window's rows.
//
// One block serves ALL query heads of one KV head for one chunk of positions, so every K and V row is read once however
// many query heads share it.  A wave takes 16 positions at a time:
//   scores  S[16 positions, heads] = K_tile . Q^T on the matrix cores (v_mfma_f32_16x16x32_f16: lane (i, kb) supplies
//           8 consecutive elements of K row i, the query fragments stay in registers), which also does the cross-lane
//           reduction that a vector-ALU dot product would need per position and head;
//   softmax the online recurrence per head, once per tile (m, d and the rescale factor alpha);
//   values  O[head, :] = alpha O[head, :] + sum_p P[p, head] V[p, :] on the vector ALU with V rows read fully coalesced
//           (a lane owns 8 consecutive output elements), probabilities passed through a per-wave LDS tile.
// The four waves of a block, and then the chunks, are merged with the usual rescale by exp(m - m_max).
//
// Causal attention of a block of query tokens (prefill) follows further down: both products on the matrix cores, K and V
// tiles shared by a block's waves through LDS.
#include <algorithm>

#include "tf_common.hpp"
#include "tf_context.hpp"

using namespace tfk;

namespace {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));

constexpr int kAttnThreads = 256;
constexpr int kAttnWaves = kAttnThreads / 64;
constexpr int kTilePositions = 16;
constexpr int kTileHeads = 16;        // columns of the score tile; heads beyond the group are zero
constexpr uint32_t kMaxHeadDim = 512; // Attention.maxHeadDim
constexpr uint32_t kMaxQHeads = 16;   // Attention.maxQHeads
constexpr uint32_t kMaxDeviceChunks = 512;

struct AttnShape {
    uint32_t num_q_heads, num_kv_heads;
    uint32_t seq_len, kv_start, chunk_len, num_chunks, ring_capacity;
    float scale;
};

__device__ __forceinline__ uint32_t physical_row(const AttnShape &s, uint32_t p) { return s.ring_capacity ? p % s.ring_capacity : p; }

__device__ __forceinline__ float exp_weight(float m, float m_max) { return m == -INFINITY ? 0.0f : __expf(m - m_max); }

// ---- matrix-core path: HD in {64, 128, 256, 512}, G = query heads per KV head in {1, 2, 4, 8}, 16-byte aligned rows
template <int HD, int G>
__global__ __launch_bounds__(kAttnThreads, 1) void attention_partial_kernel(const half_t *Q, const half_t *K, const half_t *V, float *m_out,
                                                                            float *d_out, float *o_out, AttnShape s) {
    constexpr int KS = HD / 32;                 // MFMA steps over the head dimension
    constexpr int LPR = HD / 8;                 // lanes that cover one V row
    constexpr int R = 64 / LPR;                 // V rows per load instruction
    constexpr int VLOADS = kTilePositions / R;  // V load instructions per tile
    __shared__ __align__(16) half_t p_tile[kAttnWaves][kTilePositions][kTileHeads];   // probabilities, rounded to fp16 for the packed dot
    __shared__ float alpha_tile[kAttnWaves][kTileHeads];
    __shared__ float m_wave[kAttnWaves][kTileHeads], d_wave[kAttnWaves][kTileHeads];
    __shared__ float o_wave[kAttnWaves][G][HD];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t kv_head = blockIdx.x / s.num_chunks, chunk = blockIdx.x % s.num_chunks;
    const uint32_t p_start = s.kv_start + chunk * s.chunk_len;
    const uint32_t p_end = min(p_start + s.chunk_len, s.seq_len);
    const int col = lane & 15, quad = lane >> 4;   // score tile: head `col`, positions 4 quad .. 4 quad + 3
    const size_t row_halves = (size_t)s.num_kv_heads * HD;

    // query fragments: lane (n, kb) holds Q[head n][32 d + 8 kb ..] for every step d; heads beyond the group are zero
    half8_t qf[KS];
#pragma unroll
    for (int d = 0; d < KS; ++d) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (col < G) raw = load16(Q + (size_t)(kv_head * G + (uint32_t)col) * HD + 32 * d + 8 * quad);
        qf[d] = __builtin_bit_cast(half8_t, raw);
    }
    float o[G][8];
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) o[g][e] = 0.0f;
    float m_run = -INFINITY, d_run = 0.0f;   // of head `col`
    const int vrow = lane / LPR, ve = lane % LPR;

    // two tiles of K and V rows in flight: the next tile is requested before the current one is reduced
    auto request = [&](u32x4 *kf, u32x4 *vf, uint32_t t0) {
        // rows past the chunk repeat its last row; their scores are masked and their probabilities are zero
        const uint32_t pk = min(t0 + (uint32_t)col, p_end - 1);
        const half_t *k_row = K + (size_t)physical_row(s, pk) * row_halves + (size_t)kv_head * HD + 8 * quad;
#pragma unroll
        for (int d = 0; d < KS; ++d) kf[d] = load16(k_row + 32 * d);
#pragma unroll
        for (int j = 0; j < VLOADS; ++j) {
            const uint32_t pv = min(t0 + (uint32_t)(j * R + vrow), p_end - 1);
            vf[j] = load16(V + (size_t)physical_row(s, pv) * row_halves + (size_t)kv_head * HD + 8 * ve);
        }
    };
    auto consume = [&](const u32x4 *kf, const u32x4 *vf, uint32_t t0) {
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int d = 0; d < KS; ++d) acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, kf[d]), qf[d], acc, 0, 0, 0);
        float sc[4], tile_max = -INFINITY;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            sc[r] = t0 + (uint32_t)(4 * quad + r) < p_end ? acc[r] * s.scale : -INFINITY;
            tile_max = fmaxf(tile_max, sc[r]);
        }
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16));
        tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32));
        const float m_new = fmaxf(m_run, tile_max);          // finite: the tile holds at least one position
        const float alpha = exp_weight(m_run, m_new);
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float pe = exp_weight(sc[r], m_new);
            p_tile[wave][4 * quad + r][col] = (half_t)pe;
            sum += pe;
        }
        sum += __shfl_xor(sum, 16);
        sum += __shfl_xor(sum, 32);
        d_run = d_run * alpha + sum;
        m_run = m_new;
        if (quad == 0) alpha_tile[wave][col] = alpha;
        // the wave reads back what its own lanes wrote: LDS operations of one wave complete in order
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int g = 0; g < G; ++g) {
            const float a = alpha_tile[wave][g];
#pragma unroll
            for (int e = 0; e < 8; ++e) o[g][e] *= a;
        }
        // two positions per instruction: v_dot2_f32_f16 adds p_a v_a + p_b v_b to the fp32 sum.  Loads j and j + 1 of a
        // lane hold rows a = j R + vrow and b = a + R; their elements are interleaved into (v_a[e], v_b[e]) pairs and the
        // two probability rows into (p_a[g], p_b[g]) pairs.
#pragma unroll
        for (int j = 0; j < VLOADS; j += 2) {
            const u32x4 ra = vf[j], rb = vf[j + 1];
            uint32_t vv[8];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                vv[2 * w] = __builtin_amdgcn_perm(rb[w], ra[w], 0x05040100u);       // (a.lo, b.lo)
                vv[2 * w + 1] = __builtin_amdgcn_perm(rb[w], ra[w], 0x07060302u);   // (a.hi, b.hi)
            }
            const u32x4 pa = *reinterpret_cast<const u32x4 *>(&p_tile[wave][j * R + vrow][0]);
            const u32x4 pb = *reinterpret_cast<const u32x4 *>(&p_tile[wave][(j + 1) * R + vrow][0]);
#pragma unroll
            for (int g = 0; g < G; ++g) {
                const uint32_t sel = (g & 1) ? 0x07060302u : 0x05040100u;
                const half2_t pg = as_half2(__builtin_amdgcn_perm(pb[g >> 1], pa[g >> 1], sel));
#pragma unroll
                for (int e = 0; e < 8; ++e) o[g][e] = __builtin_amdgcn_fdot2(pg, as_half2(vv[e]), o[g][e], false);
            }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // the tile is rewritten by the next one
    };
    constexpr uint32_t kStride = kAttnWaves * kTilePositions;
    u32x4 ka[KS], va[VLOADS], kb[KS], vb[VLOADS];
    uint32_t ta = p_start + (uint32_t)wave * kTilePositions, tb = ta + kStride;
    if (ta < p_end) {
        request(ka, va, ta);
        for (;;) {
            if (tb < p_end) request(kb, vb, tb);
            consume(ka, va, ta);
            ta += 2 * kStride;
            if (tb >= p_end) break;
            if (ta < p_end) request(ka, va, ta);
            consume(kb, vb, tb);
            tb += 2 * kStride;
            if (ta >= p_end) break;
        }
    }

    // lanes that served different rows of a load hold different parts of the same sums
#pragma unroll
    for (int g = 0; g < G; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            float v = o[g][e];
            if constexpr (R >= 2) v += __shfl_xor(v, 32);
            if constexpr (R >= 4) v += __shfl_xor(v, 16);
            if constexpr (R >= 8) v += __shfl_xor(v, 8);
            o[g][e] = v;
        }
    if (quad == 0) {
        m_wave[wave][col] = m_run;
        d_wave[wave][col] = d_run;
    }
    if (vrow == 0) {
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
            for (int e = 0; e < 8; ++e) o_wave[wave][g][8 * ve + e] = o[g][e];
    }
    __syncthreads();
    // merge of the four waves -> the chunk's un-normalized partial state per query head
    for (int idx = threadIdx.x; idx < G * HD; idx += kAttnThreads) {
        const int g = idx / HD, i = idx - g * HD;
        float m_max = -INFINITY;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) m_max = fmaxf(m_max, m_wave[w][g]);
        float acc = 0.0f, den = 0.0f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) {
            const float wt = exp_weight(m_wave[w][g], m_max);
            acc += o_wave[w][g][i] * wt;
            den += d_wave[w][g] * wt;
        }
        const size_t base = (size_t)(kv_head * G + (uint32_t)g) * s.num_chunks + chunk;
        o_out[base * HD + i] = acc;
        if (i == 0) {
            m_out[base] = m_max;
            d_out[base] = den;
        }
    }
}

// ---- any head dimension, group size and alignment: one block per (query head, chunk), position by position, the
// reference kernel's own shape (attention.metal:135-222)
__global__ __launch_bounds__(kAttnThreads) void attention_partial_generic_kernel(const half_t *Q, const half_t *K, const half_t *V,
                                                                                 float *m_out, float *d_out, float *o_out, uint32_t head_dim,
                                                                                 AttnShape s) {
    __shared__ float q_s[kMaxHeadDim];
    __shared__ float part[kAttnWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t q_head = blockIdx.x / s.num_chunks, chunk = blockIdx.x % s.num_chunks;
    const uint32_t kv_head = q_head / (s.num_q_heads / s.num_kv_heads);
    const uint32_t p_start = s.kv_start + chunk * s.chunk_len, p_end = min(p_start + s.chunk_len, s.seq_len);
    for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads) q_s[i] = (float)Q[(size_t)q_head * head_dim + i];
    __syncthreads();
    float o_local[(kMaxHeadDim + kAttnThreads - 1) / kAttnThreads] = {};
    float m_run = -INFINITY, d_run = 0.0f;
    for (uint32_t p = p_start; p < p_end; ++p) {
        const size_t row = ((size_t)physical_row(s, p) * s.num_kv_heads + kv_head) * head_dim;
        float partial = 0.0f;
        for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads) partial = fmaf(q_s[i], (float)K[row + i], partial);
        partial = wave_sum(partial);
        __syncthreads();   // the previous position's sums have been read
        if (lane == 0) part[wave] = partial;
        __syncthreads();
        float sc = 0.0f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) sc += part[w];
        sc *= s.scale;
        const float m_new = fmaxf(m_run, sc);
        const float alpha = exp_weight(m_run, m_new), pe = __expf(sc - m_new);
        d_run = d_run * alpha + pe;
        int slot = 0;
        for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads, ++slot) o_local[slot] = o_local[slot] * alpha + pe * (float)V[row + i];
        m_run = m_new;
    }
    const size_t base = (size_t)q_head * s.num_chunks + chunk;
    if (threadIdx.x == 0) {
        m_out[base] = m_run;
        d_out[base] = d_run;
    }
    int slot = 0;
    for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads, ++slot) o_out[base * head_dim + i] = o_local[slot];
}

// attention_decode_combine (attention.metal:339-377): out = sum_c o_c e^{m_c - m} / sum_c d_c e^{m_c - m}.
// Block = one query head x 64 output elements; the chunk weights e^{m_c - m} are formed once per block in LDS, and the
// four waves each add every fourth chunk (in ascending order) before the four sums are added in wave order.
constexpr uint32_t kCombineElems = 64;
__global__ __launch_bounds__(kAttnThreads) void attention_combine_kernel(const float *m_in, const float *d_in, const float *o_in, half_t *out,
                                                                         uint32_t head_dim, uint32_t num_chunks) {
    __shared__ float weight[kMaxDeviceChunks];
    __shared__ float red[kAttnWaves], sums[kAttnWaves][kCombineElems];
    const uint32_t q_head = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *m_row = m_in + (size_t)q_head * num_chunks, *d_row = d_in + (size_t)q_head * num_chunks;
    float m_max = -INFINITY;
    for (uint32_t c = threadIdx.x; c < num_chunks; c += kAttnThreads) m_max = fmaxf(m_max, m_row[c]);
    m_max = wave_max(m_max);
    if (lane == 0) red[wave] = m_max;
    __syncthreads();
    m_max = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float den = 0.0f;
    for (uint32_t c = threadIdx.x; c < num_chunks; c += kAttnThreads) {
        const float w = exp_weight(m_row[c], m_max);
        weight[c] = w;
        den += d_row[c] * w;
    }
    den = wave_sum(den);
    if (lane == 0) red[wave] = den;
    __syncthreads();
    den = (red[0] + red[1]) + (red[2] + red[3]);
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    const uint32_t i = blockIdx.y * kCombineElems + lane;
    float acc = 0.0f;
    if (i < head_dim) {
        const float *o_base = o_in + (size_t)q_head * num_chunks * head_dim + i;
        // eight loads in flight per lane; the additions stay in ascending chunk order
        for (uint32_t c0 = wave; c0 < num_chunks; c0 += 8 * kAttnWaves) {
            float part[8];
#pragma unroll
            for (uint32_t j = 0; j < 8; ++j) {
                const uint32_t c = c0 + j * kAttnWaves;
                part[j] = c < num_chunks ? o_base[(size_t)c * head_dim] : 0.0f;
            }
#pragma unroll
            for (uint32_t j = 0; j < 8; ++j) {
                const uint32_t c = c0 + j * kAttnWaves;
                if (c < num_chunks) acc = fmaf(part[j], weight[c], acc);
            }
        }
    }
    sums[wave][lane] = acc;
    __syncthreads();
    if (wave == 0 && i < head_dim) out[(size_t)q_head * head_dim + i] = (half_t)(((sums[0][lane] + sums[1][lane]) + (sums[2][lane] + sums[3][lane])) * inv);
}

// ---- causal attention of a block of query tokens (prefill) ---------------------------------------------------------
struct PrefillShape {
    uint32_t start, count, num_q_heads, num_kv_heads, kv_valid, window, kv_stride, q_stride, o_stride, ring_capacity;
    float scale;
};

__device__ __forceinline__ uint32_t prefill_row(const PrefillShape &s, uint32_t p) { return s.ring_capacity ? p % s.ring_capacity : p; }
// keys query t sees: [first, last)
__device__ __forceinline__ void visible_keys(const PrefillShape &s, uint32_t t, uint32_t &first, uint32_t &last) {
    const uint32_t abs_q = s.start + t;
    first = (s.window != 0u && abs_q + 1u > s.window) ? abs_q + 1u - s.window : 0u;
    last = min(s.kv_valid, abs_q + 1u);
}

// Matrix-core path.  A block owns 64 (query, head) columns that share one kv head - with G query heads per kv head that
// is 64 / G consecutive queries - and one chunk of the keys any of them sees; each of its four waves owns 16 of the columns.
// The block walks its keys 32 at a time: the K and V rows of a tile go through LDS once for all four waves.
//   scores  S^T[32 keys, 16 columns] = K_tile . Q^T (v_mfma_f32_16x16x32_f16, A = K rows out of LDS, B = the wave's query
//           fragments, which stay in registers); a lane ends up with 8 keys of ONE column, so the online softmax state
//           (m, d) and the rescale factor are per-lane scalars, and a key outside the column's causal range or window is
//           masked for that column only;
//   values  O^T[HD, 16 columns] += V_tile^T . P^T: the lane's 8 probabilities are already laid out as the B operand; the A
//           operand (8 keys of one element of V) is put together from 8 row pieces of 16 bytes with byte permutes - the
//           lane's pieces hold 8 neighbouring elements, which feed 8 matrix instructions - so V needs no transposed copy.
// With several chunks the block leaves an unnormalised partial state (m, d, o) per column for the merge kernel; with one
// it writes the rows itself.  HD in {64, 128, 256, 512}, G in {1, 2, 4, 8, 16}, rows 16-byte aligned.
constexpr int kPrefillKeys = 32, kPrefillCols = 64;
constexpr uint32_t kMaxPrefillChunks = 16, kMinChunkKeys = 256;
constexpr uint32_t kXcds = 8;

typedef __amdgpu_buffer_rsrc_t attn_rsrc_t;
// 16 bytes per lane from a buffer straight into LDS: lane l's bytes land at dst + 16 l (dst wave-uniform)
__device__ __forceinline__ void attn_lds_copy16(attn_rsrc_t rsrc, uint32_t dst, uint32_t lane_offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)(uintptr_t)dst, 16, lane_offset, 0, 0, 0);
}
// LDS reads the compiler does not see as memory accesses: it would make each of them wait for every copy still on its way
// into LDS, the prefetched tiles included.  The result registers are only valid after attn_lds_wait on them.
template <int OFFSET>
__device__ __forceinline__ u32x4 attn_lds_read16(uint32_t addr) {
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
__device__ __forceinline__ void attn_lds_wait(u32x4 (&r)[8]) {
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(r[0]), "+v"(r[1]), "+v"(r[2]), "+v"(r[3]), "+v"(r[4]), "+v"(r[5]), "+v"(r[6]), "+v"(r[7]));
}

// lane l and the lanes l ^ 16, l ^ 32, l ^ 48 (the four row groups of a score tile's column) combined, through the row
// swaps of the vector ALU instead of four trips through the LDS crossbar: after a swap of a value with itself the two
// results hold the lane's own row group and its partner's
template <typename Op>
__device__ __forceinline__ float column_reduce(float v, Op op) {
    const uint32_t u = __builtin_bit_cast(uint32_t, v);
    const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
    const float a = op(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
    const uint32_t ua = __builtin_bit_cast(uint32_t, a);
    const auto q = __builtin_amdgcn_permlane32_swap(ua, ua, false, false);
    return op(__builtin_bit_cast(float, (uint32_t)q[0]), __builtin_bit_cast(float, (uint32_t)q[1]));
}

template <int HD>
__global__ __launch_bounds__(kAttnThreads, HD > 256 ? 1 : 2) void attention_prefill_kernel(const half_t *Q, const half_t *K, const half_t *V, half_t *O,
                                                                                           float *m_part, float *d_part, float *o_part, PrefillShape s,
                                                                                           uint32_t group_shift, uint32_t col_blocks, uint32_t num_chunks) {
    constexpr int KS = HD / 32;                         // matrix steps over the head dimension for the scores
    constexpr int NG = HD >= 128 ? HD / 128 : 1;        // groups of 128 output elements (16 lanes x 8)
    constexpr int CPR = HD / 8;                         // 16-byte pieces per row
    // A tile in LDS: one copy instruction moves 64 pieces = RPI rows; copy n of a tile carries rows n, n + NI, n + 2 NI, ...
    // into the 1024 contiguous bytes of block n, and blocks are 1040 bytes apart: the 16 rows (or row groups) a score
    // operand touches then start 4 banks apart.  Row r, piece c: block r % NI, byte (r / NI) * RB + 16 c.
    constexpr int RPI = CPR >= 64 ? 1 : 64 / CPR, NI = kPrefillKeys / RPI, RB = CPR * 16, BLK = 1040, TILEB = NI * BLK;
    constexpr int JOFF = NI >= 32 ? 16 * BLK : (16 / NI) * RB;   // from row r to row r + 16
    constexpr int CPW = NI >= kAttnWaves ? NI / kAttnWaves : 1;  // copies per wave, tile and matrix
    constexpr int DB = KS < 4 ? KS : 4, NB = KS / DB;            // score steps per batch of LDS reads, batches
    __shared__ __align__(16) uint8_t k_lds[2][TILEB];
    __shared__ __align__(16) uint8_t v_lds[2][TILEB];
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int col = lane & 15, quad = lane >> 4;

    // which (kv head, chunk, column block): blocks are dealt round-robin to the 8 XCDs, so when the number of
    // (kv head, chunk) groups allows it every group's column blocks - which read the same K and V rows - share one XCD's L2
    const uint32_t groups = s.num_kv_heads * num_chunks;
    uint32_t grp, col_block;
    if (groups % kXcds == 0u) {
        const uint32_t xcd = blockIdx.x % kXcds, slot = blockIdx.x / kXcds;
        grp = xcd + kXcds * (slot / col_blocks);
        col_block = slot % col_blocks;
    } else {
        grp = blockIdx.x / col_blocks;
        col_block = blockIdx.x % col_blocks;
    }
    const uint32_t kv_head = grp / num_chunks, chunk = grp % num_chunks;
    const uint32_t group = 1u << group_shift, pairs = s.count << group_shift;

    // the keys any live column of the block sees (columns ascend by query), cut into num_chunks runs of whole tiles
    const uint32_t col0 = col_block * kPrefillCols;
    const uint32_t t_lo = min(col0 >> group_shift, s.count - 1u), t_hi = min((col0 + kPrefillCols - 1u) >> group_shift, s.count - 1u);
    uint32_t p_lo, p_hi, unused;
    visible_keys(s, t_lo, p_lo, unused);
    visible_keys(s, t_hi, unused, p_hi);
    const uint32_t span = p_hi > p_lo ? p_hi - p_lo : 0u;
    const uint32_t chunk_len = ((span + num_chunks - 1u) / num_chunks + kPrefillKeys - 1u) / kPrefillKeys * kPrefillKeys;
    const uint32_t c_lo = p_lo + chunk * chunk_len, c_hi = min(p_hi, c_lo + chunk_len);

    // this lane's column: pair index -> (query, head of the group)
    const uint32_t pair = col0 + (uint32_t)(wave * kTileHeads + col);
    const bool col_live = pair < pairs;
    const uint32_t t_col = col_live ? pair >> group_shift : 0u, q_head = kv_head * group + (pair & (group - 1u));
    uint32_t first_col = 0u, last_col = 0u;
    if (col_live) visible_keys(s, t_col, first_col, last_col);

    half8_t qf[KS];
#pragma unroll
    for (int d = 0; d < KS; ++d) {
        u32x4 raw = {0u, 0u, 0u, 0u};
        if (col_live) raw = load16(Q + (size_t)t_col * s.q_stride + (size_t)q_head * HD + 32 * d + 8 * quad);
        qf[d] = __builtin_bit_cast(half8_t, raw);
    }
    float4_t o[NG][8];   // o[g][t][r]: element 128 g + 8 (4 quad + r) + t of column `col`
#pragma unroll
    for (int g = 0; g < NG; ++g)
#pragma unroll
        for (int t = 0; t < 8; ++t) o[g][t] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    float m_run = -INFINITY, d_run = 0.0f;

    // Copies: descriptors over this kv head's part of the caches (32-bit byte offsets; the host checks that the rows fit).
    // Rows past the chunk repeat its last row: their scores are masked, their probabilities zero.
    const attn_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(K + (size_t)kv_head * HD), 0, (int)0xFFFFFFFFu, 0x00020000);
    const attn_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(V + (size_t)kv_head * HD), 0, (int)0xFFFFFFFFu, 0x00020000);
    const uint32_t lane_rows = RPI > 1 ? (uint32_t)(lane / CPR) * NI : 0u, lane_piece = (uint32_t)(lane % CPR) * 16u;
    const uint32_t row_bytes = s.kv_stride * 2u;
    auto copy_tile = [&](attn_rsrc_t rsrc, uint32_t tile, uint32_t t0) {
        if (wave >= NI) return;               // fewer copies than waves (head_dim 64)
#pragma unroll
        for (int q = 0; q < CPW; ++q) {
            const uint32_t n = (uint32_t)wave + (uint32_t)(kAttnWaves * q);
            const uint32_t p = min(t0 + n + lane_rows, c_hi - 1u);
            attn_lds_copy16(rsrc, tile + n * BLK, prefill_row(s, p) * row_bytes + lane_piece);
        }
    };
    const uint32_t k_tile[2] = {(uint32_t)(uintptr_t)k_lds[0], (uint32_t)(uintptr_t)k_lds[1]};
    const uint32_t v_tile[2] = {(uint32_t)(uintptr_t)v_lds[0], (uint32_t)(uintptr_t)v_lds[1]};
    // this lane's operand pieces inside a tile: K row `col`, piece `quad` of every step; V rows 4 quad .., piece `col`
    const uint32_t k_lane = (uint32_t)((col % NI) * BLK + (col / NI) * RB + quad * 16);
    const uint32_t v_lane = (uint32_t)(((4 * quad) % NI) * BLK + ((4 * quad) / NI) * RB + (HD >= 128 ? col : (col & 7)) * 16);

    // scores of keys 16 j + 4 quad + r of a K tile for column `col`; the reads of a batch of steps are in flight while the
    // previous batch is multiplied
    auto scores = [&](uint32_t tile, float4_t &acc0, float4_t &acc1) {
        const uint32_t at = tile + k_lane;
        acc0 = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        acc1 = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        u32x4 kf[2][8];
        auto issue = [&](u32x4 (&f)[8], int b) {   // b is a compile-time constant after unrolling
#pragma unroll
            for (int d = 0; d < DB; ++d) {
                switch (b) {
                    case 0: f[2 * d] = attn_lds_read16<0 * DB * 64>(at + d * 64); f[2 * d + 1] = attn_lds_read16<0 * DB * 64 + JOFF>(at + d * 64); break;
                    case 1: f[2 * d] = attn_lds_read16<1 * DB * 64>(at + d * 64); f[2 * d + 1] = attn_lds_read16<1 * DB * 64 + JOFF>(at + d * 64); break;
                    case 2: f[2 * d] = attn_lds_read16<2 * DB * 64>(at + d * 64); f[2 * d + 1] = attn_lds_read16<2 * DB * 64 + JOFF>(at + d * 64); break;
                    default: f[2 * d] = attn_lds_read16<3 * DB * 64>(at + d * 64); f[2 * d + 1] = attn_lds_read16<3 * DB * 64 + JOFF>(at + d * 64); break;
                }
            }
#pragma unroll
            for (int d = 2 * DB; d < 8; ++d) f[d] = u32x4{0u, 0u, 0u, 0u};
        };
        issue(kf[0], 0);
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            attn_lds_wait(kf[b & 1]);
            if (b + 1 < NB) issue(kf[(b + 1) & 1], b + 1);
#pragma unroll
            for (int d = 0; d < DB; ++d) {
                acc0 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, kf[b & 1][2 * d]), qf[b * DB + d], acc0, 0, 0, 0);
                acc1 = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, kf[b & 1][2 * d + 1]), qf[b * DB + d], acc1, 0, 0, 0);
            }
        }
    };
    auto issue_values = [&](u32x4 (&in)[8], uint32_t tile, int g) {
        const uint32_t at = tile + v_lane + (uint32_t)(g * 256);
        in[0] = attn_lds_read16<0 * BLK>(at);
        in[1] = attn_lds_read16<1 * BLK>(at);
        in[2] = attn_lds_read16<2 * BLK>(at);
        in[3] = attn_lds_read16<3 * BLK>(at);
        in[4] = attn_lds_read16<JOFF + 0 * BLK>(at);
        in[5] = attn_lds_read16<JOFF + 1 * BLK>(at);
        in[6] = attn_lds_read16<JOFF + 2 * BLK>(at);
        in[7] = attn_lds_read16<JOFF + 3 * BLK>(at);
    };

    if (c_lo < c_hi) {
        const uint32_t n_tiles = (c_hi - c_lo + kPrefillKeys - 1u) / kPrefillKeys;
        copy_tile(k_rsrc, k_tile[0], c_lo);
        copy_tile(k_rsrc, k_tile[1], c_lo + kPrefillKeys);
        copy_tile(v_rsrc, v_tile[0], c_lo);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        float4_t acc0, acc1;
        scores(k_tile[0], acc0, acc1);
        __syncthreads();
        // Step i, first half: start the copies of the tiles two (K) and one (V) ahead, take the scores of tile i + 1, and
        // turn the scores of tile i into probabilities.  Here K tiles i (its scores are in acc0/acc1) and i + 1 and V tile
        // i are in LDS and nobody reads the other two buffers any more.
        // The reference maximum of a column only moves when a score exceeds it by more than kMaxSlack (probabilities then
        // reach at most e^kMaxSlack, far inside fp16): after the first tiles the accumulators are hardly ever rescaled.
        constexpr float kMaxSlack = 8.0f;
        auto first_half = [&](uint32_t i, float &alpha, half8_t &p8, float4_t &next0, float4_t &next1) {
            const uint32_t t0 = c_lo + i * kPrefillKeys, cur = i & 1u;
            copy_tile(k_rsrc, k_tile[cur], t0 + 2 * kPrefillKeys);
            copy_tile(v_rsrc, v_tile[cur ^ 1u], t0 + kPrefillKeys);
            scores(k_tile[cur ^ 1u], next0, next1);   // of tile i + 1 (past the chunk: repeated rows, never used)
            float sc[8], tile_max = -INFINITY;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const uint32_t p = t0 + (uint32_t)(16 * (e >> 2) + 4 * quad + (e & 3));
                const float raw = e < 4 ? acc0[e & 3] : acc1[e & 3];
                sc[e] = (p >= first_col && p < last_col) ? raw * s.scale : -INFINITY;
                tile_max = fmaxf(tile_max, sc[e]);
            }
            tile_max = column_reduce(tile_max, [](float a, float b) { return fmaxf(a, b); });
            // stays -inf while the column has seen no key; the first finite maximum costs no rescale (o and d are zero)
            const bool fresh = m_run == -INFINITY;
            const float m_new = (fresh || tile_max > m_run + kMaxSlack) ? fmaxf(m_run, tile_max) : m_run;
            alpha = fresh ? 1.0f : __expf(m_run - m_new);
            float sum = 0.0f;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float pe = exp_weight(sc[e], m_new);
                p8[e] = (half_t)pe;
                sum += pe;
            }
            sum = column_reduce(sum, [](float a, float b) { return a + b; });
            d_run = d_run * alpha + sum;
            m_run = m_new;
        };
        // Step i, second half: values.  Slot e of the lane's 8 keys is row 16 (e / 4) + 4 quad + e % 4 of the tile.
        auto second_half = [&](uint32_t i, const half8_t &p8, const float4_t &next0, const float4_t &next1) {
            const uint32_t cur = i & 1u;
            u32x4 in[2][8];
            issue_values(in[0], v_tile[cur], 0);
#pragma unroll
            for (int g = 0; g < NG; ++g) {
                attn_lds_wait(in[g & 1]);
                if (g + 1 < NG) issue_values(in[(g + 1) & 1], v_tile[cur], g + 1);
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const uint32_t sel = (t & 1) ? 0x07060302u : 0x05040100u;
                    u32x4 a;
#pragma unroll
                    for (int kp = 0; kp < 4; ++kp) a[kp] = __builtin_amdgcn_perm(in[g & 1][2 * kp + 1][t >> 1], in[g & 1][2 * kp][t >> 1], sel);
                    o[g][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8_t, a), p8, o[g][t], 0, 0, 0);
                }
            }
            acc0 = next0;
            acc1 = next1;
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this wave's copies have landed
            __syncthreads();
        };
        for (uint32_t i = 0; i < n_tiles; ++i) {
            float alpha;
            half8_t p8;
            float4_t next0, next1;
            first_half(i, alpha, p8, next0, next1);
            if (__builtin_expect(__any(alpha != 1.0f), 0)) {
                // The accumulators live in the accumulation registers, where the matrix instructions update them in
                // place.  Written as plain multiplications, this rare path makes the register allocator move all of them
                // to vector registers and back in EVERY step; so it does the move itself.  The matrix instructions that
                // last wrote them finished long ago (the scores came after them and have been read), and the next ones to
                // read them follow LDS reads and a wait.
#pragma unroll
                for (int g = 0; g < NG; ++g)
#pragma unroll
                    for (int t = 0; t < 8; ++t) o[g][t] *= alpha;
            }
            second_half(i, p8, next0, next1);
        }
    }

    if (!col_live || (HD < 128 && quad >= 2)) return;      // no barrier follows
    if (num_chunks == 1u) {
        // out[t, head, :] = o / d, zero where the column saw no key
        const float inv = d_run > 0.0f ? 1.0f / d_run : 0.0f;
        half_t *dst = O + (size_t)t_col * s.o_stride + (size_t)q_head * HD + 32 * quad;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                u32x4 packed;
#pragma unroll
                for (int t = 0; t < 8; t += 2) {
                    const half2_t h = {(half_t)(o[g][t][r] * inv), (half_t)(o[g][t + 1][r] * inv)};
                    packed[t >> 1] = as_u32(h);
                }
                *reinterpret_cast<u32x4 *>(dst + 128 * g + 8 * r) = packed;
            }
    } else {
        const size_t state = ((size_t)t_col * s.num_q_heads + q_head) * num_chunks + chunk;
        if (quad == 0) {
            m_part[state] = m_run;
            d_part[state] = d_run;
        }
        float *dst = o_part + state * HD + 32 * quad;
#pragma unroll
        for (int g = 0; g < NG; ++g)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                *reinterpret_cast<float4_t *>(dst + 128 * g + 8 * r) = float4_t{o[g][0][r], o[g][1][r], o[g][2][r], o[g][3][r]};
                *reinterpret_cast<float4_t *>(dst + 128 * g + 8 * r + 4) = float4_t{o[g][4][r], o[g][5][r], o[g][6][r], o[g][7][r]};
            }
    }
}

// merge of the chunks' partial states of one (query, head) column: out = sum_c w_c o_c / sum_c w_c d_c, w_c = exp(m_c - max m);
// chunks are added in ascending order; a chunk that saw no key has weight zero and its o is not read
__global__ __launch_bounds__(128) void attention_prefill_combine_kernel(const float *m_part, const float *d_part, const float *o_part, half_t *O,
                                                                        uint32_t head_dim, uint32_t num_chunks, uint32_t num_q_heads,
                                                                        uint32_t o_stride) {
    const uint32_t column = blockIdx.x, t = column / num_q_heads, q_head = column % num_q_heads;
    const float *m_row = m_part + (size_t)column * num_chunks, *d_row = d_part + (size_t)column * num_chunks;
    float w[kMaxPrefillChunks], m_max = -INFINITY, den = 0.0f;
    for (uint32_t c = 0; c < num_chunks; ++c) m_max = fmaxf(m_max, m_row[c]);
#pragma unroll
    for (uint32_t c = 0; c < kMaxPrefillChunks; ++c) {
        w[c] = c < num_chunks ? exp_weight(m_row[c], m_max) : 0.0f;
        if (c < num_chunks) den += d_row[c] * w[c];
    }
    const float inv = den > 0.0f ? 1.0f / den : 0.0f;
    for (uint32_t e = threadIdx.x * 4u; e < head_dim; e += 128u * 4u) {
        float4_t acc = {0.0f, 0.0f, 0.0f, 0.0f};
        const float *src = o_part + (size_t)column * num_chunks * head_dim + e;
#pragma unroll
        for (uint32_t c = 0; c < kMaxPrefillChunks; ++c)
            if (c < num_chunks && w[c] != 0.0f) acc += *reinterpret_cast<const float4_t *>(src + (size_t)c * head_dim) * w[c];
        const half2_t lo = {(half_t)(acc[0] * inv), (half_t)(acc[1] * inv)}, hi = {(half_t)(acc[2] * inv), (half_t)(acc[3] * inv)};
        uint32_t *dst = reinterpret_cast<uint32_t *>(O + (size_t)t * o_stride + (size_t)q_head * head_dim + e);
        dst[0] = as_u32(lo);
        dst[1] = as_u32(hi);
    }
}

// any shape and alignment: one block per (query, head), key by key (attention_prefill_causal_tiled, prefill.metal:835-902)
__global__ __launch_bounds__(kAttnThreads) void attention_prefill_generic_kernel(const half_t *Q, const half_t *K, const half_t *V, half_t *O,
                                                                                 uint32_t head_dim, PrefillShape s) {
    __shared__ float part[kAttnWaves];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t t = blockIdx.x, qh = blockIdx.y;
    const uint32_t kvh = qh / (s.num_q_heads / s.num_kv_heads);
    uint32_t first, last;
    visible_keys(s, t, first, last);
    const half_t *q_row = Q + (size_t)t * s.q_stride + (size_t)qh * head_dim;
    float qv[(kMaxHeadDim + kAttnThreads - 1) / kAttnThreads], acc[(kMaxHeadDim + kAttnThreads - 1) / kAttnThreads] = {};
    int slot = 0;
    for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads, ++slot) qv[slot] = (float)q_row[i];
    float row_max = -INFINITY, row_sum = 0.0f;
    for (uint32_t key = first; key < last; ++key) {
        const size_t row = (size_t)prefill_row(s, key) * s.kv_stride + (size_t)kvh * head_dim;
        float partial = 0.0f;
        slot = 0;
        for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads, ++slot) partial = fmaf(qv[slot], (float)K[row + i], partial);
        partial = wave_sum(partial);
        __syncthreads();
        if (lane == 0) part[wave] = partial;
        __syncthreads();
        float sc = 0.0f;
#pragma unroll
        for (int w = 0; w < kAttnWaves; ++w) sc += part[w];
        sc *= s.scale;
        const float new_max = fmaxf(row_max, sc);
        const float old_scale = row_sum > 0.0f ? __expf(row_max - new_max) : 0.0f, new_scale = __expf(sc - new_max);
        slot = 0;
        for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads, ++slot) acc[slot] = fmaf(new_scale, (float)V[row + i], acc[slot] * old_scale);
        row_sum = row_sum * old_scale + new_scale;
        row_max = new_max;
    }
    half_t *out_row = O + (size_t)t * s.o_stride + (size_t)qh * head_dim;
    slot = 0;
    for (uint32_t i = threadIdx.x; i < head_dim; i += kAttnThreads, ++slot) out_row[i] = (half_t)(row_sum > 0.0f ? acc[slot] / row_sum : 0.0f);
}

// the context's partial-state scratch: m and d [heads x chunks], o [heads x chunks x head_dim]
int32_t attention_scratch(tf_ctx *ctx, size_t floats, float *&out) {
    const size_t need = floats * sizeof(float);
    if (ctx->attn_scratch_bytes < need) return scratch_too_small(ctx, "attention", need, ctx->attn_scratch_bytes);
    out = static_cast<float *>(ctx->attn_scratch);
    return TF_OK;
}

template <int HD>
bool launch_partial_hd(uint32_t group, dim3 grid, hipStream_t st, const half_t *q, const half_t *k, const half_t *v, float *m, float *d, float *o,
                       const AttnShape &s) {
    switch (group) {
        case 1: hipLaunchKernelGGL((attention_partial_kernel<HD, 1>), grid, dim3(kAttnThreads), 0, st, q, k, v, m, d, o, s); return true;
        case 2: hipLaunchKernelGGL((attention_partial_kernel<HD, 2>), grid, dim3(kAttnThreads), 0, st, q, k, v, m, d, o, s); return true;
        case 4: hipLaunchKernelGGL((attention_partial_kernel<HD, 4>), grid, dim3(kAttnThreads), 0, st, q, k, v, m, d, o, s); return true;
        case 8: hipLaunchKernelGGL((attention_partial_kernel<HD, 8>), grid, dim3(kAttnThreads), 0, st, q, k, v, m, d, o, s); return true;
        default: return false;
    }
}

int32_t attention_split(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k, uint64_t k_offset, const void *v,
                        uint64_t v_offset, void *out, uint64_t out_offset, uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                        uint32_t seq_len, uint32_t kv_start, float scale, uint32_t ring_capacity, const char *who) {
    TF_REQUIRE(ctx, q && k && v && out, TF_ERR_INVALID_ARGUMENT, "%s: null argument", who);
    TF_REQUIRE(ctx, num_kv_heads > 0 && num_q_heads > 0 && num_q_heads % num_kv_heads == 0, TF_ERR_INVALID_ARGUMENT,
               "%s: numQHeads must be a multiple of numKVHeads for GQA", who);
    TF_REQUIRE(ctx, head_dim > 0 && head_dim <= kMaxHeadDim, TF_ERR_INVALID_ARGUMENT, "%s: head_dim must be <= 512", who);
    TF_REQUIRE(ctx, num_q_heads <= kMaxQHeads, TF_ERR_INVALID_ARGUMENT, "%s: numQHeads %u exceeds split-KV scratch (max %u)", who, num_q_heads,
               kMaxQHeads);
    TF_REQUIRE(ctx, q_offset % 2 == 0 && k_offset % 2 == 0 && v_offset % 2 == 0 && out_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT,
               "%s: offsets must be 2-byte aligned", who);
    const half_t *qp = reinterpret_cast<const half_t *>(at(q, q_offset));
    const half_t *kp = reinterpret_cast<const half_t *>(at(k, k_offset));
    const half_t *vp = reinterpret_cast<const half_t *>(at(v, v_offset));
    half_t *op = reinterpret_cast<half_t *>(at(out, out_offset));
    hipStream_t st = static_cast<hipStream_t>(stream);
    const uint32_t group = num_q_heads / num_kv_heads;
    const uint32_t effective = seq_len > kv_start ? seq_len - kv_start : 0;
    const bool mfma = (head_dim == 64 || head_dim == 128 || head_dim == 256 || head_dim == 512) && (group == 1 || group == 2 || group == 4 || group == 8) &&
                      aligned16(qp) && aligned16(kp) && aligned16(vp);
    // chunks: enough blocks for every compute unit, whole 64-position rounds of a block's four waves
    AttnShape s;
    s.num_q_heads = num_q_heads;
    s.num_kv_heads = num_kv_heads;
    s.seq_len = seq_len;
    s.kv_start = kv_start;
    s.ring_capacity = ring_capacity;
    s.scale = scale;
    const uint32_t blocks_per_chunk = mfma ? num_kv_heads : num_q_heads;
    const uint32_t round = mfma ? kAttnWaves * kTilePositions : 16;
    uint32_t want = ((uint32_t)ctx->num_cus * (mfma ? 1u : 4u) + blocks_per_chunk - 1) / blocks_per_chunk;
    want = want < kMaxDeviceChunks ? want : kMaxDeviceChunks;
    const uint32_t eff = effective ? effective : 1;
    uint32_t chunk_len = (eff + want - 1) / want;
    chunk_len = (chunk_len + round - 1) / round * round;
    s.chunk_len = chunk_len;
    s.num_chunks = (eff + chunk_len - 1) / chunk_len;
    float *scratch = nullptr;
    const size_t states = (size_t)num_q_heads * s.num_chunks;
    const int32_t rc = attention_scratch(ctx, states * (2 + (size_t)head_dim), scratch);
    if (rc != TF_OK) return rc;
    float *m = scratch, *d = scratch + states, *o = scratch + 2 * states;
    const dim3 grid(blocks_per_chunk * s.num_chunks);
    bool launched = false;
    if (mfma) {
        switch (head_dim) {
            case 64: launched = launch_partial_hd<64>(group, grid, st, qp, kp, vp, m, d, o, s); break;
            case 128: launched = launch_partial_hd<128>(group, grid, st, qp, kp, vp, m, d, o, s); break;
            case 256: launched = launch_partial_hd<256>(group, grid, st, qp, kp, vp, m, d, o, s); break;
            default: launched = launch_partial_hd<512>(group, grid, st, qp, kp, vp, m, d, o, s); break;
        }
    }
    if (!launched) hipLaunchKernelGGL(attention_partial_generic_kernel, grid, dim3(kAttnThreads), 0, st, qp, kp, vp, m, d, o, head_dim, s);
    hipLaunchKernelGGL(attention_combine_kernel, dim3(num_q_heads, (head_dim + kCombineElems - 1) / kCombineElems), dim3(kAttnThreads), 0, st, m, d, o, op,
                       head_dim, s.num_chunks);
    return check_launch(ctx, who);
}

float default_scale(uint32_t head_dim) { return 1.0f / sqrtf((float)head_dim); }

}  // namespace

namespace tfk {

// Upper bound of the partial states (m, d and head_dim values of o each) any call within the limits asks for.
// Decode: q_heads x chunks with at most kMaxDeviceChunks chunks.  Block attention: n = queries x q_heads columns make at
// least ceil(n / 64) blocks per chunk, and chunks stop at two blocks per compute unit or kMaxPrefillChunks.
size_t attention_scratch_floats_for(int num_cus, uint32_t q_heads, uint32_t head_dim, uint32_t block_tokens) {
    size_t states = (size_t)q_heads * kMaxDeviceChunks;
    const size_t target = (size_t)(num_cus > 0 ? num_cus : 256) * 2;
    const size_t max_n = (size_t)block_tokens * q_heads;
    for (size_t n = 1; n <= max_n; ++n) {
        const size_t base = (n + kPrefillCols - 1) / kPrefillCols;
        const size_t chunks = std::min<size_t>(kMaxPrefillChunks, (target + base - 1) / base);
        states = std::max(states, n * chunks);
    }
    return states * (2 + (size_t)head_dim);
}

}  // namespace tfk

extern "C" {

int32_t tf_attention_swa(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k, uint64_t k_offset, const void *v,
                         uint64_t v_offset, void *out, uint64_t out_offset, uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                         uint32_t seq_len, uint32_t window, float scale, uint32_t ring_capacity) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "attention_swa: null context");
    const uint32_t kv_start = seq_len > window ? seq_len - window : 0;
    // every position of the window must still be in the ring
    TF_REQUIRE(ctx, ring_capacity == 0 || seq_len - kv_start <= ring_capacity, TF_ERR_INVALID_ARGUMENT,
               "attention_swa: the window (%u positions) does not fit the ring (%u rows)", seq_len - kv_start, ring_capacity);
    return attention_split(ctx, stream, q, q_offset, k, k_offset, v, v_offset, out, out_offset, head_dim, num_q_heads, num_kv_heads, seq_len,
                           kv_start, scale > 0.0f ? scale : default_scale(head_dim ? head_dim : 1), ring_capacity, "attention_swa");
}

int32_t tf_attention_full(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k, uint64_t k_offset, const void *v,
                          uint64_t v_offset, void *out, uint64_t out_offset, uint32_t head_dim, uint32_t num_q_heads, uint32_t num_kv_heads,
                          uint32_t seq_len, float scale) {
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "attention_full: null context");
    TF_REQUIRE(ctx, seq_len > 0, TF_ERR_INVALID_ARGUMENT, "attention_full: full attention requires at least one KV position");
    return attention_split(ctx, stream, q, q_offset, k, k_offset, v, v_offset, out, out_offset, head_dim, num_q_heads, num_kv_heads, seq_len, 0,
                           scale > 0.0f ? scale : default_scale(head_dim ? head_dim : 1), 0, "attention_full");
}

int32_t tf_prefill_attention_causal(tf_ctx *ctx, tf_stream stream, const void *q, uint64_t q_offset, const void *k, uint64_t k_offset,
                                    const void *v, uint64_t v_offset, void *out, uint64_t out_offset, const tf_prefill_attention_params *p,
                                    uint32_t kv_ring_capacity) {
    TF_REQUIRE(ctx, ctx && q && k && v && out && p, TF_ERR_INVALID_ARGUMENT, "prefill_attention: null argument");
    // PrefillAttention.validate (PrefillAttention.swift:120-136)
    TF_REQUIRE(ctx, p->head_dim > 0, TF_ERR_INVALID_ARGUMENT, "headDim must be positive");
    TF_REQUIRE(ctx, p->query_count > 0, TF_ERR_INVALID_ARGUMENT, "queryCount must be positive");
    TF_REQUIRE(ctx, p->num_q_heads > 0, TF_ERR_INVALID_ARGUMENT, "numQHeads must be positive");
    TF_REQUIRE(ctx, p->num_kv_heads > 0, TF_ERR_INVALID_ARGUMENT, "numKVHeads must be positive");
    TF_REQUIRE(ctx, p->num_q_heads % p->num_kv_heads == 0, TF_ERR_INVALID_ARGUMENT, "numQHeads must be divisible by numKVHeads");
    TF_REQUIRE(ctx, (uint64_t)p->q_token_stride_elements >= (uint64_t)p->num_q_heads * p->head_dim, TF_ERR_INVALID_ARGUMENT, "qTokenStrideElements too small");
    TF_REQUIRE(ctx, (uint64_t)p->o_token_stride_elements >= (uint64_t)p->num_q_heads * p->head_dim, TF_ERR_INVALID_ARGUMENT, "oTokenStrideElements too small");
    TF_REQUIRE(ctx, (uint64_t)p->kv_token_stride_elements >= (uint64_t)p->num_kv_heads * p->head_dim, TF_ERR_INVALID_ARGUMENT, "kvTokenStrideElements too small");
    TF_REQUIRE(ctx, (uint64_t)p->start_position + p->query_count <= p->kv_valid_count, TF_ERR_INVALID_ARGUMENT,
               "query block exceeds kvValidCount");
    TF_REQUIRE(ctx, p->head_dim <= kMaxHeadDim, TF_ERR_INVALID_ARGUMENT, "prefill_attention: head_dim must be <= 512");
    TF_REQUIRE(ctx, p->query_count <= 65535 && p->num_q_heads <= 65535, TF_ERR_INVALID_ARGUMENT, "prefill_attention: more than 65535 queries or heads");
    TF_REQUIRE(ctx, q_offset % 2 == 0 && k_offset % 2 == 0 && v_offset % 2 == 0 && out_offset % 2 == 0, TF_ERR_INVALID_ARGUMENT,
               "prefill_attention: offsets must be 2-byte aligned");
    const half_t *qp = reinterpret_cast<const half_t *>(at(q, q_offset));
    const half_t *kp = reinterpret_cast<const half_t *>(at(k, k_offset));
    const half_t *vp = reinterpret_cast<const half_t *>(at(v, v_offset));
    half_t *op = reinterpret_cast<half_t *>(at(out, out_offset));
    hipStream_t st = static_cast<hipStream_t>(stream);
    PrefillShape s;
    s.start = p->start_position;
    s.count = p->query_count;
    s.num_q_heads = p->num_q_heads;
    s.num_kv_heads = p->num_kv_heads;
    s.kv_valid = p->kv_valid_count;
    s.window = p->sliding_window;
    s.kv_stride = p->kv_token_stride_elements;
    s.q_stride = p->q_token_stride_elements;
    s.o_stride = p->o_token_stride_elements;
    s.ring_capacity = kv_ring_capacity;
    s.scale = p->scale;
    const uint32_t group = p->num_q_heads / p->num_kv_heads, hd = p->head_dim;
    uint32_t shift = 0;
    while ((1u << shift) < group) ++shift;
    const uint64_t cache_bytes = (uint64_t)(kv_ring_capacity ? kv_ring_capacity : p->kv_valid_count) * p->kv_token_stride_elements * 2u;
    const bool mfma = (hd == 64 || hd == 128 || hd == 256 || hd == 512) && (1u << shift) == group && group <= (uint32_t)kTileHeads && aligned16(qp) &&
                      aligned16(kp) && aligned16(vp) && aligned16(op) && s.q_stride % 8 == 0 && s.kv_stride % 8 == 0 && s.o_stride % 8 == 0 &&
                      cache_bytes < (1ull << 32);   // the copies address cache rows with 32-bit byte offsets
    if (mfma) {
        const uint32_t col_blocks = (s.count * group + kPrefillCols - 1) / kPrefillCols, base = col_blocks * s.num_kv_heads;
        // enough chunks to give every CU a block (two where two fit), none shorter than kMinChunkKeys
        const uint32_t abs_first = s.start, abs_last = s.start + s.count - 1u;
        const uint32_t lo_first = (s.window != 0u && abs_first + 1u > s.window) ? abs_first + 1u - s.window : 0u;
        const uint32_t hi_last = std::min(s.kv_valid, abs_last + 1u);
        const uint32_t span = hi_last > lo_first ? hi_last - lo_first : 0u;
        const uint32_t target = (uint32_t)ctx->num_cus * (hd > 256 ? 1u : 2u);
        uint32_t chunks = std::max(1u, std::min({(target + base - 1) / base, span / kMinChunkKeys, kMaxPrefillChunks}));
        float *m = nullptr, *d = nullptr, *o = nullptr;
        if (chunks > 1) {
            const size_t states = (size_t)s.count * s.num_q_heads * chunks;
            float *scratch = nullptr;
            const int32_t rc = attention_scratch(ctx, states * (2 + (size_t)hd), scratch);
            if (rc != TF_OK) return rc;
            m = scratch;
            d = scratch + states;
            o = scratch + 2 * states;
        }
        const dim3 grid(base * chunks);
        switch (hd) {
            case 64: hipLaunchKernelGGL(attention_prefill_kernel<64>, grid, dim3(kAttnThreads), 0, st, qp, kp, vp, op, m, d, o, s, shift, col_blocks, chunks); break;
            case 128: hipLaunchKernelGGL(attention_prefill_kernel<128>, grid, dim3(kAttnThreads), 0, st, qp, kp, vp, op, m, d, o, s, shift, col_blocks, chunks); break;
            case 256: hipLaunchKernelGGL(attention_prefill_kernel<256>, grid, dim3(kAttnThreads), 0, st, qp, kp, vp, op, m, d, o, s, shift, col_blocks, chunks); break;
            default: hipLaunchKernelGGL(attention_prefill_kernel<512>, grid, dim3(kAttnThreads), 0, st, qp, kp, vp, op, m, d, o, s, shift, col_blocks, chunks); break;
        }
        if (chunks > 1)
            hipLaunchKernelGGL(attention_prefill_combine_kernel, dim3(s.count * s.num_q_heads), dim3(128), 0, st, m, d, o, op, hd, chunks, s.num_q_heads,
                               s.o_stride);
    } else {
        hipLaunchKernelGGL(attention_prefill_generic_kernel, dim3(s.count, s.num_q_heads), dim3(kAttnThreads), 0, st, qp, kp, vp, op, hd, s);
    }
    return check_launch(ctx, "prefill_attention");
}

void tf_attention_split_geometry(uint32_t num_q_heads, uint32_t num_kv_heads, uint32_t seq_len, uint32_t kv_start, int32_t prefer_gqa_swa,
                                 tf_attention_split_geometry_t *out) {
    if (!out || num_kv_heads == 0) return;
    const int q_per_kv = (int)(num_q_heads / num_kv_heads);
    const bool grouped = prefer_gqa_swa != 0 && q_per_kv <= 2;
    const int effective = (int)seq_len - (int)kv_start;
    const int eff = effective > 1 ? effective : 1;
    const int default_chunks = grouped ? 8 : 16;
    int base = default_chunks < 64 ? default_chunks : 64;
    base = base < eff ? base : eff;
    base = base > 1 ? base : 1;
    int scaled = base * q_per_kv;
    scaled = scaled < 64 ? scaled : 64;
    const int chunks = grouped ? (base > scaled ? base : scaled) : base;
    out->effective_length = effective;
    out->num_chunks = chunks;
    out->chunk_length = (eff + chunks - 1) / chunks;
    out->partial_threadgroups = (grouped ? (int)num_kv_heads : (int)num_q_heads) * chunks;
    out->use_swa_grouped_partial = grouped ? 1 : 0;
}

}  // extern "C"

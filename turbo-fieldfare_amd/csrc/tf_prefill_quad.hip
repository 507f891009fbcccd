// Grouped expert stages for chunks of a few pairs (multi-token verification, small prefill chunks): the quad kernels.
#include <algorithm>

#include "tf_prefill_kernels.hpp"

using namespace tfk;

namespace {

// ------------------------------------------------------------------------------------------------ grouped, few pairs a chunk
// Chunks of a few pairs (a handful of tokens per expert: speculative verification, short prefill blocks) are bound by the
// experts' bytes, not by arithmetic: every touched expert has to stream through once, at the rate of a plain read.
//
// v_mfma_f32_4x4x4_16b_f16 multiplies, in each group of four lanes, the lanes' four A rows with the lanes' four B columns.
// Here the four lanes of a quad hold the SAME 32-element piece of FOUR DIFFERENT weight rows (B: nibbles isolated as fp16
// subnormals, exact) and the activations of that piece for FOUR DIFFERENT pairs (A, from an LDS image of the chunk's
// activation rows): all sixteen products of the instruction are wanted, a 4-row x 4-pair x 32-element product costs eight
// instructions, and the nibbles of a piece are isolated once however many pairs meet it.  Result register i of lane j of a
// quad = pair i x row j, over the quad's piece: a lane collects ITS OWN row against four pairs, so the row's scale and bias
// are the ones the lane loaded itself (with the operands the other way round every pass paid eight cross-lane moves for them).
// A wave's 16 quads take QC consecutive pieces of 16 / QC groups of four rows; pieces of a row are summed across quads at
// the end of a tile.  A block takes one slice of one chunk's rows; the next tile's loads follow the current tile's use
// pass by pass, so one tile buffer keeps the memory pipe full.
constexpr uint32_t kQuadMaxPairs = 8;    // most pairs whose activations a block holds in LDS: 2 MFMA pair groups (the gate / up kernel's MAXP is 8 or 4)
// A pair's row in the LDS image is followed by 64 bytes of padding: the four lanes of a quad read the same pieces of four
// different pairs at once, and rows a multiple of 256 bytes apart would put them on the same banks.
constexpr int kQuadRowPad = 4;   // in 16-byte pieces
constexpr size_t quad_row_bytes(int k) { return (size_t)k * 2 + kQuadRowPad * 16; }
constexpr size_t quad_lds_bytes(int k, uint32_t max_pairs = kQuadMaxPairs) { return (size_t)max_pairs * (quad_row_bytes(k) + (size_t)(k >> 5) * 4 + 16); }
// Behind the image: per wave, the scales and the biases of the tile it is working on (512 bytes each at most: 4 rows of 48
// groups or 8 rows of 16).  A tile's scales are consecutive bytes of the matrix, so the wave fetches them with ONE load per
// array (4 or 8 bytes a lane), puts them down here and every pass picks its 16-bit value with an LDS read: two memory
// instructions a tile instead of two per pass, which had been two thirds of these kernels' memory instructions (without them
// the down kernel ran 16 % faster, the gate / up kernel 7 %).
constexpr size_t kQuadSBArrayBytes = 512;
constexpr size_t kQuadSBWaveBytes = 2 * kQuadSBArrayBytes;
constexpr size_t quad_lds_total(int k, uint32_t max_pairs = kQuadMaxPairs) { return (quad_lds_bytes(k, max_pairs) + 15) / 16 * 16 + 4 * kQuadSBWaveBytes; }
// The sums of a column's 32 activations sit side by side for the kQuadMaxPairs pairs of the image (xsum[column][pair]): a lane
// needs the sums of four pairs at once and takes them in one 16-byte read.

template <int CTRL>
__device__ __forceinline__ float quad_bcast(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}

// QC: quads along the row per pass (16: one group of four rows a wave; 8: two groups).  NPASS * QC pieces cover a row.
template <int QC, int NPASS>
struct QuadMap {
    static constexpr int RG = 16 / QC;            // groups of four rows a wave takes at once
    static constexpr int kRows = 4 * RG;          // rows per tile
    // Pass p takes piece QC p + kq of the lane's row: every pass but the last has a piece for every lane, and its offsets
    // are the first pass's plus a constant that fits the load instruction's immediate field.
    uint32_t woff0, sboff0, woff_last, sboff_last;   // byte offsets from the tile's start; the last pass's are 0 for a lane without a piece
    int kq;                                       // the lane's piece within a pass
    bool last_valid;                              // whether the lane has a piece in the last pass
    int m, rg;                                    // lane within the quad; row group
    __device__ __forceinline__ void init(int k, int lane) {
        const int nch = k >> 5, groups = k >> 6;
        m = lane & 3;
        const int quad = lane >> 2;
        kq = quad % QC;
        rg = quad / QC;
        const uint32_t r = (uint32_t)(rg * 4 + m);
        woff0 = r * ((uint32_t)k >> 1) + (uint32_t)kq * 16u;
        sboff0 = (r * (uint32_t)groups + (uint32_t)(kq >> 1)) * 2u;
        last_valid = QC * (NPASS - 1) + kq < nch;
        woff_last = last_valid ? woff0 + (uint32_t)(QC * (NPASS - 1)) * 16u : 0u;
        sboff_last = last_valid ? sboff0 + (uint32_t)(QC * (NPASS - 1) / 2) * 2u : 0u;
    }
    __device__ __forceinline__ bool has(int p) const { return p < NPASS - 1 || last_valid; }
    __device__ __forceinline__ int col(int p) const { return p < NPASS - 1 ? QC * p + kq : (last_valid ? QC * p + kq : 0); }   // 0: a piece that exists, for a lane whose result is not used
    __device__ __forceinline__ uint32_t woff(int p) const { return p < NPASS - 1 ? woff0 + (uint32_t)(QC * p) * 16u : woff_last; }
    __device__ __forceinline__ uint32_t sboff(int p) const { return p < NPASS - 1 ? sboff0 + (uint32_t)(QC * p / 2) * 2u : sboff_last; }
};

// chunks of the call, as every thread of a launch sees it
__device__ __forceinline__ uint32_t quad_chunk_count(const ChunkList &cl, uint32_t n_chunks_upper) {
    return uniform_u32(min(cl.dev ? *cl.dev_n : cl.n, n_chunks_upper));
}

// The tiles of all chunks, in chunk order, are shared out over the blocks of a launch, which has as many blocks as the
// compute units hold at once.  Few chunks: every chunk gets the same number of blocks, and the few blocks left over idle.
// Many chunks: the tiles are split evenly, and a block's span may end in one chunk and go on in the next (it then sets up
// twice, which only pays when whole blocks per chunk would leave many blocks idle).
constexpr uint32_t kQuadMinBlocksPerChunk = 8;
__device__ __forceinline__ void quad_span(uint32_t n_chunks, uint32_t tiles_per_chunk, uint32_t &lo, uint32_t &hi) {
    const uint32_t per_chunk = n_chunks ? gridDim.x / n_chunks : 0u;
    if (per_chunk >= kQuadMinBlocksPerChunk) {
        const uint32_t chunk = blockIdx.x / per_chunk, part = blockIdx.x - chunk * per_chunk;
        const bool idle = chunk >= n_chunks;
        lo = idle ? 0u : chunk * tiles_per_chunk + tiles_per_chunk * part / per_chunk;
        hi = idle ? 0u : chunk * tiles_per_chunk + tiles_per_chunk * (part + 1) / per_chunk;
    } else {
        const uint64_t total = (uint64_t)n_chunks * tiles_per_chunk;
        lo = (uint32_t)(total * blockIdx.x / gridDim.x);
        hi = (uint32_t)(total * (blockIdx.x + 1) / gridDim.x);
    }
}

struct QuadPass {
    u32x4 w;
};

// One buffer descriptor covers the whole expert blob for the life of the block; a tile's place inside it is a scalar offset
// per load, so a block keeps four scalar registers of descriptors instead of a fresh descriptor per matrix, array and tile.
// Whole tiles only: the callers require the row counts to be multiples of the tile height.
__device__ __forceinline__ rsrc_t quad_blob_rsrc(const uint8_t *blob) { return make_rsrc(blob, 0xFFFFFFFFu); }

template <int QC, int NPASS>
__device__ __forceinline__ void quad_request(QuadPass &t, const QuadMap<QC, NPASS> &qm, int p, rsrc_t blob, uint32_t w_at) {
    t.w = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(blob, qm.woff(p), (int)w_at, kStreamOnce));
}

// The scales and biases of one tile (kRows consecutive rows: kRows * groups * 2 consecutive bytes of each array), W bytes a
// lane (4 or 8): lane l fetches bytes W l .. W l + W - 1 of each array, lanes beyond the tile byte 0 again (the descriptor
// covers the whole blob and checks nothing: no lane may reach past the tile).  put(): the wave's copy in LDS; at(): a value.
template <int W>
struct QuadTileSB {
    uint32_t s[W / 4], b[W / 4];
    uint32_t lane_off;
    __device__ __forceinline__ void init(int lane, uint32_t tile_bytes) { lane_off = (uint32_t)lane * W < tile_bytes ? (uint32_t)lane * W : 0u; }
    __device__ __forceinline__ void request(rsrc_t blob, uint32_t s_at, uint32_t b_at) {
        if constexpr (W == 4) {
            s[0] = __builtin_amdgcn_raw_buffer_load_b32(blob, lane_off, (int)s_at, 0);
            b[0] = __builtin_amdgcn_raw_buffer_load_b32(blob, lane_off, (int)b_at, 0);
        } else {
            const u32x2 sv = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(blob, lane_off, (int)s_at, 0));
            const u32x2 bv = __builtin_bit_cast(u32x2, __builtin_amdgcn_raw_buffer_load_b64(blob, lane_off, (int)b_at, 0));
            s[0] = sv[0]; s[1] = sv[1]; b[0] = bv[0]; b[1] = bv[1];
        }
    }
    // area: the wave's kQuadSBWaveBytes of LDS.  Same-wave LDS accesses execute in program order; the wave barriers keep the
    // compiler from moving a pass's reads ahead of the tile's writes or the next tile's writes ahead of this tile's reads.
    __device__ __forceinline__ void put(uint8_t *area, int lane) const {
        __builtin_amdgcn_wave_barrier();
        if constexpr (W == 4) {
            reinterpret_cast<uint32_t *>(area)[lane] = s[0];
            reinterpret_cast<uint32_t *>(area + kQuadSBArrayBytes)[lane] = b[0];
        } else {
            reinterpret_cast<u32x2 *>(area)[lane] = u32x2{s[0], s[1]};
            reinterpret_cast<u32x2 *>(area + kQuadSBArrayBytes)[lane] = u32x2{b[0], b[1]};
        }
        __builtin_amdgcn_wave_barrier();
    }
    static __device__ __forceinline__ uint16_t scale_at(const uint8_t *area, uint32_t byte) { return *reinterpret_cast<const uint16_t *>(area + byte); }
    static __device__ __forceinline__ uint16_t bias_at(const uint8_t *area, uint32_t byte) { return *reinterpret_cast<const uint16_t *>(area + kQuadSBArrayBytes + byte); }
};

// acc[i] += (pair i of the group) . (this lane's row), over one piece: eight matrix instructions, then the row's scale and
// bias.  o: this lane's row piece; xq: the piece's activations of the lane's pair (lane % 4 of the group); xs4: the sums of the
// four pairs' activations over the piece.  The matrix pipe's subnormal units (2^-24) are folded into the scale: s * 2^24 is
// exact, so fma(s 2^24, c, .) rounds exactly as fma(s, c 2^24, .) would.
template <int SD>
__device__ __forceinline__ void quad_piece(const ChunkOperands &o, uint16_t s_bits, uint16_t b_bits, const half2_t *xq, const f32x4 xs4, float acc[4]) {
    f32x4 c = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        const half4_t a0 = __builtin_shufflevector(xq[4 * d + 0], xq[4 * d + 1], 0, 1, 2, 3);
        const half4_t a1 = __builtin_shufflevector(xq[4 * d + 2], xq[4 * d + 3], 0, 1, 2, 3);
        c = __builtin_amdgcn_mfma_f32_4x4x4f16(a0, __builtin_bit_cast(half4_t, o.a[2 * d]), c, 0, 0, 0);
        c = __builtin_amdgcn_mfma_f32_4x4x4f16(a1, __builtin_bit_cast(half4_t, o.a[2 * d + 1]), c, 0, 0, 0);
    }
    const float s24 = sb_to_f32<SD>(s_bits) * 16777216.0f, bf = sb_to_f32<SD>(b_bits);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(s24, c[i], fmaf(bf, xs4[i], acc[i]));
}

// sum over the QC quads that hold pieces of the same rows: lanes that agree in (lane & 3) and in the row group
template <int QC>
__device__ __forceinline__ float quad_sum(float v) {
    v += dpp_f32<0x124>(v);   // row_ror:4
    v += dpp_f32<0x128>(v);   // row_ror:8: the four quads of a 16-lane row
    v += __builtin_bit_cast(float, __builtin_amdgcn_ds_swizzle(__builtin_bit_cast(int, v), 0x401F));   // lane ^ 16 (within 32 lanes)
    if constexpr (QC == 16) v += __shfl_xor(v, 32, kWave);
    return v;
}

// activation rows -> LDS image in dot-product order; `row_of(j)` gives the row of batch pair j; all threads call
template <typename RowOf>
__device__ __forceinline__ void quad_stage_rows(uint32_t nb, int k, u32x4 *xa, float *xsum, RowOf row_of, int max_pairs = (int)kQuadMaxPairs) {
    const int nch = k >> 5, pieces = k >> 3, total = (int)nb * pieces;
    for (int q0 = 0; q0 < total; q0 += 1024) {
        u32x4 raw[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q = q0 + 256 * i + (int)threadIdx.x;
            raw[i] = u32x4{0u, 0u, 0u, 0u};
            if (q < total) {
                const int j = q / pieces, piece = q - j * pieces;
                raw[i] = load16(row_of((uint32_t)j) + piece * 8);
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int q = q0 + 256 * i + (int)threadIdx.x;
            const int j = q < total ? q / pieces : 0, piece = q < total ? q - j * pieces : pieces;   // piece == pieces: nothing is written
            XStage::publish_piece(raw[i], piece, pieces, nch, xa + (size_t)j * (pieces + kQuadRowPad), xsum + j, max_pairs);
        }
    }
}

// pieces of one pass x the LDS image of the batch's pairs -> acc[g][i] (pair 4 g + i x the lane's row).  A group's pairs beyond
// the batch repeat its last pair (their sums are not stored); the sums of their activations are whatever the image holds.
template <int QC, int NPASS, int SD, int G>
__device__ __forceinline__ void quad_pass(const ChunkOperands &o, uint16_t s_bits, uint16_t b_bits, int colp, const QuadMap<QC, NPASS> &qm, const u32x4 *xa,
                                          const float *xsum, int nch, int pieces, uint32_t nb, int groups_of_pairs, float (&acc)[G][4]) {
#pragma unroll
    for (int g = 0; g < G; ++g) {
        if (g < groups_of_pairs) {
            uint32_t j = min((uint32_t)(4 * g + qm.m), nb - 1);
            asm volatile("" : "+v"(j));   // the LDS addresses are made here, pass by pass: kept across the tile loop they would crowd out the tile buffers
            const u32x4 *xj = xa + (size_t)j * (pieces + kQuadRowPad);
            half2_t xq[16];
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const u32x4 v = xj[dd * nch + colp];
#pragma unroll
                for (int q = 0; q < 4; ++q) xq[4 * dd + q] = as_half2(v[q]);
            }
            quad_piece<SD>(o, s_bits, b_bits, xq, *reinterpret_cast<const f32x4 *>(xsum + (size_t)colp * (4 * G) + 4 * g), acc[g]);
        }
    }
}

// Three blocks a CU is what this kernel is built around: with two, a SIMD's two waves wait for memory at the same time too often
// (gate / up at 16 tokens: 45.8 us with two blocks, 40.4 us with three).  Registers: 165 a lane with the 8-pair image (this file is
// compiled with the register-pressure trackers of the scheduler switched on: without them the allocator ends at 168 and one spill,
// and a kernel that touches scratch memory dispatches several times slower).  LDS: the image is sized for the rows in use, 52.6 KB at
// 2816 columns; wider rows (up to kQuadMaxD) leave room for two blocks.
// MAXP: pairs in the LDS image, 8 or 4.  With four the kernel needs 143 registers and 30 KB; chunks of more than four pairs then
// go through in two batches, which pays as long as they are rare (calls of up to 96 pairs: 8 / 12 tokens 55.4 / 59.8 -> 54.4 / 58.9 us).
template <int NPASS, int SD, int MAXP>
__global__ __launch_bounds__(256, 3) void grouped_phase1_quad_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl, uint32_t n_chunks_upper,
                                                                     const tf_prefill_pair *pairs, const half_t *hidden, long hidden_stride,
                                                                     half_t *acts, uint32_t acts_pair_base, int d, int f) {
    constexpr int QC = 16, G = MAXP / 4;
    typedef QuadMap<QC, NPASS> Map;
    extern __shared__ __align__(16) uint8_t quad_lds[];      // quad_lds_total(d, MAXP) bytes: sized for the rows in use, so that three blocks fit a CU at 2816 columns
    const int lane = threadIdx.x & 63, wave = uniform_int((int)(threadIdx.x >> 6));
    const int nch = d >> 5, pieces = d >> 3;
    u32x4 *xa = reinterpret_cast<u32x4 *>(quad_lds);
    float *xsum = reinterpret_cast<float *>(quad_lds + (size_t)MAXP * quad_row_bytes(d));
    uint8_t *sb_area = quad_lds + (quad_lds_bytes(d, MAXP) + 15) / 16 * 16 + (size_t)wave * kQuadSBWaveBytes;
    Map qm;
    qm.init(d, lane);
    QuadTileSB<8> tsb;                                    // 4 rows of up to 48 groups: 8 bytes a lane
    tsb.init(lane, (uint32_t)Map::kRows * ((uint32_t)d >> 6) * 2u);
    // One tile buffer, used for a tile's gate rows, then its up rows, then the next tile's gate rows ...: while a matrix's
    // pass p is being used, the same pass of the matrix after it is already on its way into the registers that pass freed.
    QuadPass t[NPASS];
    // the block's share of the tiles of all chunks, in chunk order
    const uint32_t tpe = (uint32_t)f / Map::kRows;
    uint32_t span_lo, span_hi;
    quad_span(quad_chunk_count(cl, n_chunks_upper), tpe, span_lo, span_hi);
    for (uint32_t pos = span_lo; pos < span_hi;) {
    const uint32_t chunk = pos / tpe;
    const int t_lo = (int)(pos - chunk * tpe), t_hi = (int)min(tpe, (uint32_t)t_lo + (span_hi - pos));
    pos += (uint32_t)(t_hi - t_lo);
    tf_prefill_group ch;
    if (!get_chunk(cl, chunk, ch)) continue;
    ch.expert = uniform_u32(ch.expert);
    ch.pair_start = uniform_u32(ch.pair_start);
    ch.pair_count = uniform_u32(ch.pair_count);
    const uint8_t *base = uniform_ptr(expert_base(tab, ch.expert));
    if (!base) continue;
    const rsrc_t blob = quad_blob_rsrc(base);
    // `from`: the blob's descriptor, or one of no records when there is no such tile (the loads then return zeros without
    // touching memory, and the loop needs no branch around them)
    // pass 0 of a matrix's tile is preceded by the tile's scales and biases (their registers are free: the tile before has put
    // its own into LDS)
    auto request = [&](rsrc_t from, bool up, int tile, int p) {
        const uint32_t row0 = (uint32_t)tile * Map::kRows;
        const uint32_t w_byte = row0 * ((uint32_t)d >> 1), sb_byte = row0 * ((uint32_t)d >> 6) * 2u;
        if (p == 0) tsb.request(from, (up ? off.up_s_off : off.gate_s_off) + sb_byte, (up ? off.up_b_off : off.gate_b_off) + sb_byte);
        quad_request(t[p], qm, p, from, (up ? off.up_W_off : off.gate_W_off) + w_byte);
    };
    // a chunk longer than the LDS image goes through in batches, its weights once a batch
    for (uint32_t p0 = 0; p0 < ch.pair_count; p0 += (uint32_t)MAXP) {
        const uint32_t nb = min((uint32_t)MAXP, ch.pair_count - p0), first = ch.pair_start + p0;
        const int groups_of_pairs = (int)((nb + 3) >> 2);
        int tile = t_lo + wave;
        if (tile < t_hi) {
#pragma unroll
            for (int p = 0; p < NPASS; ++p) request(blob, false, tile, p);   // the weights do not wait for the activations
        }
        quad_stage_rows(nb, d, xa, xsum, [&](uint32_t j) { return hidden + (size_t)pairs[first + j].token * hidden_stride; }, MAXP);
        __syncthreads();
        for (; tile < t_hi; tile += 4) {
            float ag[G][4], au[G][4];
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int k = 0; k < 4; ++k) ag[g][k] = au[g][k] = 0.0f;
            const bool more = tile + 4 < t_hi;
            tsb.put(sb_area, lane);                          // the gate rows' scales and biases
#pragma unroll
            for (int p = 0; p < NPASS; ++p) {
                const bool has = qm.has(p);
                const ChunkOperands og = chunk_operands(has ? t[p].w : u32x4{0u, 0u, 0u, 0u});
                const uint16_t gs = QuadTileSB<8>::scale_at(sb_area, qm.sboff(p)), gb = has ? QuadTileSB<8>::bias_at(sb_area, qm.sboff(p)) : (uint16_t)0;
                request(blob, true, tile, p);
                quad_pass<QC, NPASS, SD, G>(og, gs, gb, qm.col(p), qm, xa, xsum, nch, pieces, nb, groups_of_pairs, ag);
            }
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int k = 0; k < 4; ++k) ag[g][k] = gelu_tanh_fast(quad_sum<QC>(ag[g][k]));
            tsb.put(sb_area, lane);                          // the up rows'
#pragma unroll
            for (int p = 0; p < NPASS; ++p) {
                const bool has = qm.has(p);
                const ChunkOperands ou = chunk_operands(has ? t[p].w : u32x4{0u, 0u, 0u, 0u});
                const uint16_t us = QuadTileSB<8>::scale_at(sb_area, qm.sboff(p)), ub = has ? QuadTileSB<8>::bias_at(sb_area, qm.sboff(p)) : (uint16_t)0;
                if (more) request(blob, false, tile + 4, p);
                quad_pass<QC, NPASS, SD, G>(ou, us, ub, qm.col(p), qm, xa, xsum, nch, pieces, nb, groups_of_pairs, au);
            }
            const int row0 = tile * Map::kRows;
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (g < groups_of_pairs) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const half_t h = (half_t)(ag[g][i] * quad_sum<QC>(au[g][i]));
                        const uint32_t j = 4 * g + i;
                        if (lane < 4 && j < nb) acts[(size_t)(first + j - acts_pair_base) * f + row0 + lane] = h;   // lanes 0..3: the tile's four rows
                    }
                }
            }
        }
        __syncthreads();   // everyone is done with the LDS image before the next batch overwrites it
    }
    }
}

// down rows for such chunks: rows of 22 pieces (f = 704): eight quads along the row, two groups of four rows a wave.  95 registers
// and 22 KB: five blocks a CU (48 / 64 tokens 116.6 / 150.6 -> 114.4 / 148.6 us against four).
template <int NPASS, int SD>
__global__ __launch_bounds__(256, 5) void grouped_down_quad_kernel(ExpertTable tab, tf_expert_offsets off, ChunkList cl, uint32_t n_chunks_upper,
                                                                   const tf_prefill_pair *pairs, const half_t *acts, uint32_t acts_pair_base,
                                                                   half_t *route_partials, int d, int f, int top_k) {
    constexpr int QC = 8, G = (int)kQuadMaxPairs / 4;
    typedef QuadMap<QC, NPASS> Map;
    __shared__ __align__(16) uint8_t quad_lds[quad_lds_total(kQuadMaxF)];
    const int lane = threadIdx.x & 63, wave = uniform_int((int)(threadIdx.x >> 6));
    const int nch = f >> 5, pieces = f >> 3;
    uint8_t *sb_area = quad_lds + (quad_lds_bytes(kQuadMaxF) + 15) / 16 * 16 + (size_t)wave * kQuadSBWaveBytes;
    u32x4 *xa = reinterpret_cast<u32x4 *>(quad_lds);
    float *xsum = reinterpret_cast<float *>(quad_lds + (size_t)kQuadMaxPairs * quad_row_bytes(f));
    uint32_t *out_row = reinterpret_cast<uint32_t *>(quad_lds + (size_t)kQuadMaxPairs * (quad_row_bytes(f) + (size_t)nch * 4));   // token * top_k + rank
    Map qm;
    qm.init(f, lane);
    QuadPass t[NPASS];
    QuadTileSB<4> tsb;                                    // 8 rows of up to 16 groups: 4 bytes a lane
    tsb.init(lane, (uint32_t)Map::kRows * ((uint32_t)f >> 6) * 2u);
    // the tiles of all chunks, split evenly over the blocks (see the gate / up kernel)
    const uint32_t tiles = (uint32_t)d / Map::kRows;
    uint32_t span_lo, span_hi;
    quad_span(quad_chunk_count(cl, n_chunks_upper), tiles, span_lo, span_hi);
    for (uint32_t pos = span_lo; pos < span_hi;) {
    const uint32_t chunk = pos / tiles;
    const int t_lo = (int)(pos - chunk * tiles), t_hi = (int)min(tiles, (uint32_t)t_lo + (span_hi - pos));
    pos += (uint32_t)(t_hi - t_lo);
    tf_prefill_group ch;
    if (!get_chunk(cl, chunk, ch)) continue;
    ch.expert = uniform_u32(ch.expert);
    ch.pair_start = uniform_u32(ch.pair_start);
    ch.pair_count = uniform_u32(ch.pair_count);
    const uint8_t *base = uniform_ptr(expert_base(tab, ch.expert));
    if (!base) continue;
    const rsrc_t blob = quad_blob_rsrc(base);
    auto request = [&](rsrc_t from, int tile, int p) {
        const uint32_t row0 = (uint32_t)tile * Map::kRows;
        if (p == 0) tsb.request(from, off.down_s_off + row0 * ((uint32_t)f >> 6) * 2u, off.down_b_off + row0 * ((uint32_t)f >> 6) * 2u);
        quad_request(t[p], qm, p, from, off.down_W_off + row0 * ((uint32_t)f >> 1));
    };
    for (uint32_t p0 = 0; p0 < ch.pair_count; p0 += kQuadMaxPairs) {
        const uint32_t nb = min(kQuadMaxPairs, ch.pair_count - p0), first = ch.pair_start + p0;
        const int groups_of_pairs = (int)((nb + 3) >> 2);
        int tile = t_lo + wave;
        if (tile < t_hi) {
#pragma unroll
            for (int p = 0; p < NPASS; ++p) request(blob, tile, p);
        }
        quad_stage_rows(nb, f, xa, xsum, [&](uint32_t j) { return acts + (size_t)(first + j - acts_pair_base) * f; });
        if (threadIdx.x < nb) {
            const tf_prefill_pair pr = pairs[first + threadIdx.x];
            out_row[threadIdx.x] = pr.token * (uint32_t)top_k + pr.rank;
        }
        __syncthreads();
        for (; tile < t_hi; tile += 4) {
            float acc[G][4];
#pragma unroll
            for (int g = 0; g < G; ++g)
#pragma unroll
                for (int k = 0; k < 4; ++k) acc[g][k] = 0.0f;
            const rsrc_t next = make_rsrc(base, uniform_u32(tile + 4 < t_hi ? 0xFFFFFFFFu : 0u));
            tsb.put(sb_area, lane);
#pragma unroll
            for (int p = 0; p < NPASS; ++p) {
                const bool has = qm.has(p);
                const ChunkOperands ow = chunk_operands(has ? t[p].w : u32x4{0u, 0u, 0u, 0u});
                const uint16_t ws = QuadTileSB<4>::scale_at(sb_area, qm.sboff(p)), wb = has ? QuadTileSB<4>::bias_at(sb_area, qm.sboff(p)) : (uint16_t)0;
                request(next, tile + 4, p);
                quad_pass<QC, NPASS, SD, G>(ow, ws, wb, qm.col(p), qm, xa, xsum, nch, pieces, nb, groups_of_pairs, acc);
            }
            const uint32_t row0 = (uint32_t)tile * Map::kRows + (uint32_t)(qm.rg * 4 + qm.m);   // this lane's row
#pragma unroll
            for (int g = 0; g < G; ++g) {
                if (g < groups_of_pairs) {
#pragma unroll
                    for (int i = 0; i < 4; ++i) {
                        const half_t h = (half_t)quad_sum<QC>(acc[g][i]);
                        const uint32_t j = 4 * g + i;
                        if ((lane & 31) < 4 && j < nb)   // lanes 0..3: rows of group 0; lanes 32..35: rows of group 1
                            route_partials[(size_t)out_row[j] * d + row0] = h;
                    }
                }
            }
        }
        __syncthreads();
    }
    }
}

}  // namespace

namespace tfk {

int32_t launch_grouped_quad(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off, const ChunkList &cl,
                            uint32_t n_chunks_upper, const GroupedGeom &g, tf_dtype sd, uint32_t stream_pairs) {
    const int p1_passes = ((g.d >> 5) + 15) / 16, dn_passes = ((g.f >> 5) + 7) / 8;
    int32_t rc;
    {
        // as many blocks as the compute units hold at once: three of the gate / up kernel where its LDS image leaves room (rows of up
        // to 2816 columns; the 4-pair image for calls of up to 96 pairs), five of the down kernel
        const bool few_pairs = stream_pairs != 0 && stream_pairs <= 96;
        const size_t lds1 = quad_lds_total(g.d, few_pairs ? 4u : 8u);
        const uint32_t per_cu = (uint32_t)std::min<size_t>(3, std::max<size_t>(1, (size_t)160 * 1024 / (lds1 + 256)));
        const dim3 grid(per_cu * (uint32_t)ctx->num_cus), grid_down(5u * (uint32_t)ctx->num_cus);
#define TF_GP1Q_LAUNCH(NP_, SD_, MAXP_)                                                                                   \
    hipLaunchKernelGGL((grouped_phase1_quad_kernel<NP_, SD_, MAXP_>), grid, dim3(256), lds1, st, tab, off, cl, n_chunks_upper, g.pairs, g.hidden, \
                       g.hidden_stride, g.acts, g.acts_pair_base, g.d, g.f)
#define TF_GP1Q(NP_)                                                                                                       \
    if (p1_passes == NP_) {                                                                                                \
        if (sd == TF_BF16) {                                                                                               \
            if (few_pairs) TF_GP1Q_LAUNCH(NP_, 0, 4); else TF_GP1Q_LAUNCH(NP_, 0, 8);                                       \
        } else {                                                                                                           \
            if (few_pairs) TF_GP1Q_LAUNCH(NP_, 1, 4); else TF_GP1Q_LAUNCH(NP_, 1, 8);                                       \
        }                                                                                                                  \
    }
        TF_GP1Q(1) TF_GP1Q(2) TF_GP1Q(3) TF_GP1Q(4) TF_GP1Q(5) TF_GP1Q(6)
#undef TF_GP1Q
#undef TF_GP1Q_LAUNCH
        rc = check_launch(ctx, "grouped phase 1 quad");
        if (rc != TF_OK) return rc;
#define TF_GDQ(NP_)                                                                                                        \
    if (dn_passes == NP_) {                                                                                                \
        if (sd == TF_BF16)                                                                                                 \
            hipLaunchKernelGGL((grouped_down_quad_kernel<NP_, 0>), grid_down, dim3(256), 0, st, tab, off, cl, n_chunks_upper, g.pairs, g.acts,            \
                               g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k);                                     \
        else                                                                                                               \
            hipLaunchKernelGGL((grouped_down_quad_kernel<NP_, 1>), grid_down, dim3(256), 0, st, tab, off, cl, n_chunks_upper, g.pairs, g.acts,            \
                               g.acts_pair_base, g.route_partials, g.d, g.f, g.top_k);                                     \
    }
        TF_GDQ(1) TF_GDQ(2) TF_GDQ(3) TF_GDQ(4)
#undef TF_GDQ
        return check_launch(ctx, "grouped down quad");
    }
}

}  // namespace tfk

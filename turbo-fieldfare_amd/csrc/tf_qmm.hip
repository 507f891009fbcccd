// Matrix-core (MFMA) kernels: dense int4 QMM, and the grouped expert GEMMs of batched prefill
// (gate/up + GeGLU, then down) driven by a work list of (expert, pair range) chunks.
#include "tf_prefill_kernels.hpp"
#include "tf_rowdot.hpp"

using namespace tfk;

namespace {

// The wave's weight rows: column tile j covers rows row0[j] .. row0[j] + 31 of a matrix of `limit[j]` rows that starts
// at w / s / b.  s[0] and s[1] (and b[0], b[1]) lie within 2 GiB of each other: the same array, or arrays of one expert.
template <int SD>
__device__ __forceinline__ QmmBRows make_b_rows(const uint8_t *const w[2], const uint8_t *const s[2], const uint8_t *const b[2],
                                                const int row0[2], const int limit[2], int row_bytes, int groups, int lane) {
    QmmBRows rows;
#pragma unroll
    for (int j = 0; j < 2; ++j) rows.w[j] = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(w[j]), 0, limit[j] * row_bytes, 0x00020000);
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        const int r = 16 * (t & 1) + (lane >> 2);                    // row inside the column tile
        const int piece = (lane & 3) ^ ((r >> 2) & 3);
        rows.copy_off[t] = (uint32_t)(row0[t >> 1] + r) * (uint32_t)row_bytes + (uint32_t)piece * 16u;
    }
    // scales and biases: one descriptor per kind over the arrays of both tiles, from the lower of the two
    const uint32_t sb_row_bytes = (uint32_t)groups * 2u;
    const uint8_t *const sbase = s[0] <= s[1] ? s[0] : s[1], *const bbase = b[0] <= b[1] ? b[0] : b[1];
    uint32_t srel[2], brel[2], send = 0, bend = 0;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        srel[j] = (uint32_t)(s[j] - sbase);
        brel[j] = (uint32_t)(b[j] - bbase);
        send = max(send, srel[j] + (uint32_t)limit[j] * sb_row_bytes);
        bend = max(bend, brel[j] + (uint32_t)limit[j] * sb_row_bytes);
    }
    rows.sd = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(sbase), 0, (int)send, 0x00020000);
    rows.bd = __builtin_amdgcn_make_buffer_rsrc(const_cast<uint8_t *>(bbase), 0, (int)bend, 0x00020000);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t row = (uint32_t)min(row0[j] + (lane & 31), limit[j] - 1);   // a column past the matrix: its last row (never stored)
        rows.scan_s[j] = srel[j] + row * sb_row_bytes;
        rows.scan_b[j] = brel[j] + row * sb_row_bytes;
        rows.pre[j] = 0u;
        rows.post[j] = 1.0f;
    }
    // as a copier the lane serves row lane & 31 of tile lane >> 5: its own row of one of the tiles
    rows.sb_copy_off[0] = lane < 32 ? rows.scan_s[0] : rows.scan_s[1];
    rows.sb_copy_off[1] = lane < 32 ? rows.scan_b[0] : rows.scan_b[1];
    rows.s_end = send;
    rows.b_end = bend;
    rows.groups = groups;
    return rows;
}

__device__ __forceinline__ void zero_acc(float16_t acc[4][2]) {
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[mt][j][r] = 0.0f;
}

// ---- output tiles
// The accumulator layout gives a lane one column of 16 scattered rows: written straight to memory that is a 2-byte store
// per value, 64-byte runs per wave.  Instead the block's tile goes through LDS (free once the K loop has drained) as fp16
// and leaves as 16-byte pieces of whole rows: 512-byte (256-column tiles) or 256-byte runs per row.
constexpr int kOutPadBytes = 16;   // keeps the rows of a wave's two half-waves on different LDS banks

template <int COLS>
__device__ __forceinline__ uint32_t out_tile_offset(int row, int col) {
    return (uint32_t)row * (uint32_t)(COLS * 2 + kOutPadBytes) + (uint32_t)col * 2u;
}
template <int COLS>
__device__ __forceinline__ void out_tile_put(uint8_t *lds, int row, int col, float v) {
    *reinterpret_cast<half_t *>(lds + out_tile_offset<COLS>(row, col)) = (half_t)v;
}
// row_base(row): where column 0 of the block's tile of that row lives (16-byte aligned); rows_valid / cols_valid bound
// the part of the tile that exists (cols_valid a multiple of 8).  Ends with every thread past the barrier it needs.
template <int COLS, typename RowBase>
__device__ __forceinline__ void out_tile_store(const uint8_t *lds, int rows_valid, int cols_valid, RowBase row_base) {
    constexpr int kPieces = COLS / 8;
    __syncthreads();
    for (int idx = threadIdx.x; idx < kQmmBM * kPieces; idx += (int)blockDim.x) {
        const int row = idx / kPieces, piece = idx - row * kPieces;
        if (row < rows_valid && piece * 8 < cols_valid) {
            const u32x4 v = *reinterpret_cast<const u32x4 *>(lds + out_tile_offset<COLS>(row, piece * 8));
            *reinterpret_cast<u32x4 *>(row_base(row) + piece * 8) = v;
        }
    }
}
// bytes of LDS a block needs: the K loop's buffers, or the staged output tile of COLS columns with a row table behind it
template <int NW, int COLS>
constexpr int block_lds_bytes() {
    constexpr int out_bytes = kQmmBM * (COLS * 2 + kOutPadBytes) + kQmmBM * 4;
    return out_bytes > QmmGeom<NW>::kLoopLdsBytes ? out_bytes : QmmGeom<NW>::kLoopLdsBytes;
}

// ------------------------------------------------------------------------------------------------ dense
// Block number -> (row tile, column tile) of a dense product.  Workgroups go to the 8 XCDs round-robin by linear id and
// each XCD has its own L2: row tile r belongs to XCD r % 8, which computes all of its column tiles, so the activation rows
// of a tile are fetched into one L2 only and every XCD streams the (much smaller) weight matrix once.  With fewer row
// tiles than XCDs the plain numbering is used.  The grid is dense_grid() blocks; surplus ones return false.
constexpr uint32_t kDenseXcds = 8;
__host__ __device__ inline uint32_t dense_grid(uint32_t row_tiles, uint32_t col_tiles) {
    if (row_tiles < kDenseXcds) return row_tiles * col_tiles;
    return kDenseXcds * ((row_tiles + kDenseXcds - 1) / kDenseXcds) * col_tiles;
}
__device__ __forceinline__ bool dense_tile(uint32_t id, uint32_t row_tiles, uint32_t col_tiles, uint32_t &row_tile, uint32_t &col_tile) {
    if (row_tiles < kDenseXcds) {
        row_tile = id / col_tiles;
        col_tile = id - row_tile * col_tiles;
        return row_tile < row_tiles;
    }
    const uint32_t xcd = id % kDenseXcds, j = id / kDenseXcds;
    row_tile = (j / col_tiles) * kDenseXcds + xcd;
    col_tile = j % col_tiles;
    return row_tile < row_tiles;
}

// The four tile kernels are shells around `..._body` functions, so that a dense product can ride along in the launch of a
// grouped one (a block takes one role or the other by its index).  `id`: the block's number within its own kind; `lds`: the
// block's block_lds_bytes<4, columns>() of LDS, 128-byte aligned.
struct DenseArgs {
    const uint8_t *W, *S, *B;
    const half_t *X;
    long ldx;
    half_t *Y;
    long ldy;
    int M, N, K;
    bool rows_vectorizable;   // Y 16-byte aligned, N % 8 == 0, ldy % 8 == 0: whole 16-byte pieces of output rows
};
// VEC: a.rows_vectorizable holds and the tile leaves through LDS as row pieces
template <int SD, bool VEC>
__device__ __forceinline__ void qmm_dense_body(const DenseArgs &a, uint32_t id, uint8_t *lds) {
    const uint8_t *W = a.W, *S = a.S, *B = a.B;
    const half_t *X = a.X;
    half_t *Y = a.Y;
    const long ldx = a.ldx, ldy = a.ldy;
    const int M = a.M, N = a.N, K = a.K;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t row_tile, col_tile;
    if (!dense_tile(id, (uint32_t)(M + kQmmBM - 1) / kQmmBM, (uint32_t)(N + kQmmBN - 1) / kQmmBN, row_tile, col_tile)) return;
    const int n0 = (int)col_tile * kQmmBN + wave * kQmmWaveN, m0 = (int)row_tile * kQmmBM;
    QmmARows<4> arow;
    arow.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(X), 0, (int)0xFFFFFFFFu, 0x00020000);
#pragma unroll
    for (int q = 0; q < QmmGeom<4>::kAChunks; ++q) qmm_a_rows_set(arow, q, (uint64_t)min(m0 + qmm_a_row_of<4>(q), M - 1) * (uint64_t)ldx * 2u);
    const uint8_t *w[2] = {W, W}, *s[2] = {S, S}, *b[2] = {B, B};
    const int row0[2] = {n0, n0 + 32}, limit[2] = {N, N};
    QmmBRows rows = make_b_rows<SD>(w, s, b, row0, limit, K >> 1, K >> 6, lane);
    const int row_tiles = min(4, (M - m0 + 31) >> 5);
    float16_t acc[4][2];
    zero_acc(acc);
    qmm_k_loop<SD, 4>(K >> 6, arow, rows, (uint32_t)(uintptr_t)lds, lane, row_tiles, acc);
    if constexpr (VEC) {
        __syncthreads();   // every wave has left the K loop and nothing it requested is still on its way into LDS
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int mt = 0; mt < 4; ++mt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    out_tile_put<kQmmBN>(lds, mt * 32 + acc_row(r, lane), wave * kQmmWaveN + j * 32 + acc_col(lane), acc[mt][j][r] * rows.post[j]);
        const int nb = (int)col_tile * kQmmBN;
        out_tile_store<kQmmBN>(lds, min(kQmmBM, M - m0), min(kQmmBN, N - nb), [&](int row) { return Y + (size_t)(m0 + row) * ldy + nb; });
        return;
    }
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const int n = n0 + j * 32 + acc_col(lane);
#pragma unroll
        for (int mt = 0; mt < 4; ++mt)
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + mt * 32 + acc_row(r, lane);
                if (m < M && n < N) Y[(size_t)m * ldy + n] = (half_t)(acc[mt][j][r] * rows.post[j]);
            }
    }
}

template <int SD, bool VEC>
__global__ __launch_bounds__(256, 2) void qmm_dense_kernel(DenseArgs a) {
    __shared__ __align__(128) uint8_t lds[block_lds_bytes<4, kQmmBN>()];
    qmm_dense_body<SD, VEC>(a, blockIdx.x, lds);
}

// Shared-expert gate and up projections of a block of rows in one pass: a wave's first column tile is 32 rows of the gate
// matrix, its second the same 32 rows of the up matrix.  Both sums are rounded to fp16 before GeGLU, the stage boundary of
// the reference's chain (two GEMVs writing fp16, then gelu_mul_fp16: SharedExpertInt4.swift:60-84).
constexpr int kGegluBN = 32 * 4;
struct DenseGegluArgs {
    const uint8_t *gW, *gS, *gB, *uW, *uS, *uB;
    const half_t *X;
    long ldx;
    half_t *A;
    long lda;
    int M, F, K;
};
template <int SD>
__device__ __forceinline__ void qmm_dense_geglu_body(const DenseGegluArgs &a, uint32_t id, uint8_t *lds) {
    const uint8_t *gW = a.gW, *gS = a.gS, *gB = a.gB, *uW = a.uW, *uS = a.uS, *uB = a.uB;
    const half_t *X = a.X;
    half_t *A = a.A;
    const long ldx = a.ldx, lda = a.lda;
    const int M = a.M, F = a.F, K = a.K;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    uint32_t row_tile, col_tile;
    if (!dense_tile(id, (uint32_t)(M + kQmmBM - 1) / kQmmBM, (uint32_t)(F + kGegluBN - 1) / kGegluBN, row_tile, col_tile)) return;
    const int n0 = (int)col_tile * kGegluBN + wave * 32, m0 = (int)row_tile * kQmmBM;
    QmmARows<4> arow;
    arow.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(X), 0, (int)0xFFFFFFFFu, 0x00020000);
#pragma unroll
    for (int q = 0; q < QmmGeom<4>::kAChunks; ++q) qmm_a_rows_set(arow, q, (uint64_t)min(m0 + qmm_a_row_of<4>(q), M - 1) * (uint64_t)ldx * 2u);
    const uint8_t *w[2] = {gW, uW}, *s[2] = {gS, uS}, *b[2] = {gB, uB};
    const int row0[2] = {n0, n0}, limit[2] = {F, F};
    QmmBRows rows = make_b_rows<SD>(w, s, b, row0, limit, K >> 1, K >> 6, lane);
    const int row_tiles = min(4, (M - m0 + 31) >> 5);
    float16_t acc[4][2];
    zero_acc(acc);
    qmm_k_loop<SD, 4>(K >> 6, arow, rows, (uint32_t)(uintptr_t)lds, lane, row_tiles, acc);
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        if (mt >= row_tiles) break;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const float gate = (float)(half_t)(acc[mt][0][r] * rows.post[0]), up = (float)(half_t)(acc[mt][1][r] * rows.post[1]);
            out_tile_put<kGegluBN>(lds, mt * 32 + acc_row(r, lane), wave * 32 + acc_col(lane), gelu_tanh_fast(gate) * up);
        }
    }
    const int nb = (int)col_tile * kGegluBN;
    out_tile_store<kGegluBN>(lds, min(kQmmBM, M - m0), min(kGegluBN, F - nb), [&](int row) { return A + (size_t)(m0 + row) * lda + nb; });
}

template <int SD>
__global__ __launch_bounds__(256, 2) void qmm_dense_geglu_kernel(DenseGegluArgs a) {
    __shared__ __align__(128) uint8_t lds[block_lds_bytes<4, kGegluBN>()];
    qmm_dense_geglu_body<SD>(a, blockIdx.x, lds);
}

// Block number -> (chunk, column tile) for the grouped kernels.  Workgroups go to the 8 XCDs round-robin by linear id and
// each XCD has its own L2; the column tiles of one chunk all read the same activation rows, so they are given ids that
// are congruent modulo 8: a run of 16 * tiles consecutive ids serves 16 chunks, two consecutive ones per XCD, and a chunk's
// activations are fetched into one L2 once instead of into all eight.  Two consecutive chunks on one XCD, because the chunks
// of a popular expert follow each other in the work list and read the same weights: side by side in one L2 the second finds
// what the first fetched (2048 tokens, Zipf routing: 0.362 -> 0.355 ms on one box, 0.361 -> 0.347 on another; four a run
// measured slower again, 0.361).
constexpr uint32_t kXcds = 8;
constexpr uint32_t kChunksPerXcdRun = 2;
__device__ __forceinline__ void chunk_and_tile(uint32_t id, uint32_t tiles, uint32_t &chunk, uint32_t &tile) {
    const uint32_t run = kXcds * kChunksPerXcdRun * tiles;
    const uint32_t within = id % run, xcd = within % kXcds, local = within / kXcds;   // local: 0 .. kChunksPerXcdRun * tiles - 1
    chunk = (id / run) * (kXcds * kChunksPerXcdRun) + xcd * kChunksPerXcdRun + local / tiles;
    tile = local % tiles;
}
constexpr uint32_t kChunkRun = kXcds * kChunksPerXcdRun;

// ------------------------------------------------------------------------------------------------ grouped phase 1
// Block = one chunk (<= 128 sorted pairs of one expert) x 32 NW intermediate columns.  A wave's first column tile is 32
// rows of the gate matrix, its second the same 32 rows of the up matrix, so GeGLU is applied to the fp32 accumulators
// in registers.
// Eight-wave blocks (one per CU, the same activation rows serving twice the columns) halve the activation fetches but
// measured slower (gate/up 265 us against 227 us, down 144 us against 118 us at 2048 tokens): four waves, two blocks per CU.
constexpr int kGroupedWaves = 4;
constexpr int kP1BN = 32 * kGroupedWaves;
constexpr int kDownBN = QmmGeom<kGroupedWaves>::kBN;

struct GroupedP1Args {
    ExpertTable tab;
    tf_expert_offsets off;
    ChunkList cl;
    const tf_prefill_pair *pairs;
    const half_t *hidden;
    long hidden_stride;
    half_t *acts;
    uint32_t acts_pair_base;
    int D, F;
};
template <int SD>
__device__ __forceinline__ void grouped_phase1_body(const GroupedP1Args &a, uint32_t id, uint8_t *lds) {
    const ExpertTable &tab = a.tab;
    const tf_expert_offsets &off = a.off;
    const ChunkList &cl = a.cl;
    const tf_prefill_pair *pairs = a.pairs;
    const half_t *hidden = a.hidden;
    const long hidden_stride = a.hidden_stride;
    half_t *acts = a.acts;
    const uint32_t acts_pair_base = a.acts_pair_base;
    const int D = a.D, F = a.F;
    tf_prefill_group ch;
    uint32_t chunk_index, col_tile;
    chunk_and_tile(id, (uint32_t)(F + kP1BN - 1) / kP1BN, chunk_index, col_tile);
    if (!get_chunk(cl, chunk_index, ch)) return;
    // everything taken from the work list is the same in all lanes: say so, the descriptors built from it live in
    // scalar registers
    ch.expert = uniform_u32(ch.expert);
    ch.pair_start = uniform_u32(ch.pair_start);
    ch.pair_count = uniform_u32(ch.pair_count);
    const uint8_t *base = uniform_ptr(expert_base(tab, ch.expert));
    if (!base) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (int)col_tile * kP1BN + wave * 32;
    // the pairs of a chunk ascend by token: offsets are taken from the first pair's row
    const uint32_t token0 = uniform_u32(pairs[ch.pair_start].token);
    QmmARows<kGroupedWaves> arow;
    arow.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(hidden + (size_t)token0 * hidden_stride), 0, (int)0xFFFFFFFFu, 0x00020000);
#pragma unroll
    for (int q = 0; q < QmmGeom<kGroupedWaves>::kAChunks; ++q) {
        const uint32_t r = min((uint32_t)qmm_a_row_of<kGroupedWaves>(q), ch.pair_count - 1);
        qmm_a_rows_set(arow, q, (uint64_t)(pairs[ch.pair_start + r].token - token0) * (uint64_t)hidden_stride * 2u);
    }
    const uint8_t *w[2] = {base + off.gate_W_off, base + off.up_W_off};
    const uint8_t *s[2] = {base + off.gate_s_off, base + off.up_s_off};
    const uint8_t *b[2] = {base + off.gate_b_off, base + off.up_b_off};
    const int row0[2] = {n0, n0}, limit[2] = {F, F};
    QmmBRows rows = make_b_rows<SD>(w, s, b, row0, limit, D >> 1, D >> 6, lane);
    const int row_tiles = (int)((ch.pair_count + 31) >> 5);
    float16_t acc[4][2];
    zero_acc(acc);
    qmm_k_loop<SD, kGroupedWaves>(D >> 6, arow, rows, (uint32_t)(uintptr_t)lds, lane, row_tiles, acc);
    // acts rows of a chunk are consecutive; F % 64 == 0 and a 16-byte aligned acts keep every row piece aligned
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
        if (mt >= row_tiles) break;   // tiles without rows were not multiplied and are not stored
#pragma unroll
        for (int r = 0; r < 16; ++r)
            out_tile_put<kP1BN>(lds, mt * 32 + acc_row(r, lane), wave * 32 + acc_col(lane),
                                gelu_tanh_fast(acc[mt][0][r] * rows.post[0]) * (acc[mt][1][r] * rows.post[1]));
    }
    const int nb = (int)col_tile * kP1BN;
    half_t *tile = acts + (size_t)(ch.pair_start - acts_pair_base) * F + nb;
    out_tile_store<kP1BN>(lds, (int)ch.pair_count, min(kP1BN, F - nb), [&](int row) { return tile + (size_t)row * F; });
}

template <int SD>
__global__ __launch_bounds__(64 * kGroupedWaves, 8 / kGroupedWaves) void grouped_phase1_mfma_kernel(GroupedP1Args a) {
    __shared__ __align__(128) uint8_t lds[block_lds_bytes<kGroupedWaves, kP1BN>()];
    grouped_phase1_body<SD>(a, blockIdx.x, lds);
}
// the same launch with the dense gate / up / GeGLU tiles of a shared expert ahead of the grouped tiles: the blocks that start
// first are the full-height ones, the grouped tiles of every height fill in behind them (0.461 -> 0.428 ms for the 2048-token
// block against the dense tiles last)
template <int SD>
__global__ __launch_bounds__(64 * kGroupedWaves, 8 / kGroupedWaves) void grouped_phase1_and_dense_geglu_kernel(GroupedP1Args a, uint32_t dense_blocks,
                                                                                                             DenseGegluArgs dense) {
    static_assert(kP1BN == kGegluBN && kGroupedWaves == 4, "the two roles share one LDS layout");
    __shared__ __align__(128) uint8_t lds[block_lds_bytes<kGroupedWaves, kP1BN>()];
    if (blockIdx.x < dense_blocks) qmm_dense_geglu_body<SD>(dense, blockIdx.x, lds);
    else grouped_phase1_body<SD>(a, blockIdx.x - dense_blocks, lds);
}

// ------------------------------------------------------------------------------------------------ grouped down
// Block = one chunk x 64 NW output columns: X rows are the chunk's activation rows, Y rows scatter to
// route_partials[(token * top_k + rank) * D + c].
struct GroupedDownArgs {
    ExpertTable tab;
    tf_expert_offsets off;
    ChunkList cl;
    const tf_prefill_pair *pairs;
    const half_t *acts;
    uint32_t acts_pair_base;
    half_t *route_partials;
    int D, F, top_k;
};
template <int SD>
__device__ __forceinline__ void grouped_down_body(const GroupedDownArgs &a, uint32_t id, uint8_t *lds) {
    const ExpertTable &tab = a.tab;
    const tf_expert_offsets &off = a.off;
    const ChunkList &cl = a.cl;
    const tf_prefill_pair *pairs = a.pairs;
    const half_t *acts = a.acts;
    const uint32_t acts_pair_base = a.acts_pair_base;
    half_t *route_partials = a.route_partials;
    const int D = a.D, F = a.F, top_k = a.top_k;
    tf_prefill_group ch;
    uint32_t chunk_index, col_tile;
    chunk_and_tile(id, (uint32_t)(D + kDownBN - 1) / kDownBN, chunk_index, col_tile);
    if (!get_chunk(cl, chunk_index, ch)) return;
    // everything taken from the work list is the same in all lanes: say so, the descriptors built from it live in
    // scalar registers
    ch.expert = uniform_u32(ch.expert);
    ch.pair_start = uniform_u32(ch.pair_start);
    ch.pair_count = uniform_u32(ch.pair_count);
    const uint8_t *base = uniform_ptr(expert_base(tab, ch.expert));
    if (!base) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n0 = (int)col_tile * kDownBN + wave * kQmmWaveN;
    QmmARows<kGroupedWaves> arow;
    arow.rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<half_t *>(acts + (size_t)(ch.pair_start - acts_pair_base) * F), 0, (int)0xFFFFFFFFu, 0x00020000);
#pragma unroll
    for (int q = 0; q < QmmGeom<kGroupedWaves>::kAChunks; ++q) {
        const uint32_t r = min((uint32_t)qmm_a_row_of<kGroupedWaves>(q), ch.pair_count - 1);
        qmm_a_rows_set(arow, q, (uint64_t)r * (uint64_t)F * 2u);
    }
    const uint8_t *w[2] = {base + off.down_W_off, base + off.down_W_off};
    const uint8_t *s[2] = {base + off.down_s_off, base + off.down_s_off};
    const uint8_t *b[2] = {base + off.down_b_off, base + off.down_b_off};
    const int row0[2] = {n0, n0 + 32}, limit[2] = {D, D};
    QmmBRows rows = make_b_rows<SD>(w, s, b, row0, limit, F >> 1, F >> 6, lane);
    const int row_tiles = (int)((ch.pair_count + 31) >> 5);
    float16_t acc[4][2];
    zero_acc(acc);
    qmm_k_loop<SD, kGroupedWaves>(F >> 6, arow, rows, (uint32_t)(uintptr_t)lds, lane, row_tiles, acc);
    __syncthreads();
    // where each row of the tile goes: route_partials row token * top_k + rank (D % 64 == 0 keeps the pieces aligned)
    uint32_t *row_slot = reinterpret_cast<uint32_t *>(lds + kQmmBM * (kDownBN * 2 + kOutPadBytes));
    if (threadIdx.x < ch.pair_count) {
        const tf_prefill_pair p = pairs[ch.pair_start + threadIdx.x];
        row_slot[threadIdx.x] = p.token * (uint32_t)top_k + p.rank;
    }
#pragma unroll
    for (int mt = 0; mt < 4; ++mt)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                out_tile_put<kDownBN>(lds, mt * 32 + acc_row(r, lane), wave * kQmmWaveN + j * 32 + acc_col(lane), acc[mt][j][r] * rows.post[j]);
    const int nb = (int)col_tile * kDownBN;
    out_tile_store<kDownBN>(lds, (int)ch.pair_count, min(kDownBN, D - nb), [&](int row) { return route_partials + (size_t)row_slot[row] * D + nb; });
}
template <int SD>
__global__ __launch_bounds__(64 * kGroupedWaves, 8 / kGroupedWaves) void grouped_down_mfma_kernel(GroupedDownArgs a) {
    __shared__ __align__(128) uint8_t lds[block_lds_bytes<kGroupedWaves, kDownBN>()];
    grouped_down_body<SD>(a, blockIdx.x, lds);
}
// the same launch with the tiles of a dense product (a shared expert's down projection; rows_vectorizable) ahead of the grouped tiles
template <int SD>
__global__ __launch_bounds__(64 * kGroupedWaves, 8 / kGroupedWaves) void grouped_down_and_dense_kernel(GroupedDownArgs a, uint32_t dense_blocks,
                                                                                                     DenseArgs dense) {
    static_assert(kDownBN == kQmmBN && kGroupedWaves == 4, "the two roles share one LDS layout");
    __shared__ __align__(128) uint8_t lds[block_lds_bytes<kGroupedWaves, kDownBN>()];
    if (blockIdx.x < dense_blocks) qmm_dense_body<SD, true>(dense, blockIdx.x, lds);
    else grouped_down_body<SD>(a, blockIdx.x - dense_blocks, lds);
}

DenseArgs dense_args(const uint8_t *w, const uint8_t *s, const uint8_t *b, const half_t *x, long ldx, half_t *y, long ldy, int m, int n, int k) {
    const bool rows_vec = aligned16(y) && n % 8 == 0 && ldy % 8 == 0;   // whole 16-byte pieces of output rows
    return DenseArgs{w, s, b, x, ldx, y, ldy, m, n, k, rows_vec};
}
DenseGegluArgs dense_geglu_args(const tf_projection *gate, const tf_projection *up, const half_t *x, long ldx, half_t *a, long lda, int m) {
    return DenseGegluArgs{at(gate->weights, gate->weights_offset), at(gate->scales, gate->scales_offset), at(gate->biases, gate->biases_offset),
                          at(up->weights, up->weights_offset),     at(up->scales, up->scales_offset),     at(up->biases, up->biases_offset),
                          x, ldx, a, lda, m, (int)gate->rows, (int)gate->cols};
}

}  // namespace

namespace tfk {

bool qmm_operands_ok(const void *w, const void *x, long ldx_halves, int k) {
    return aligned16(w) && aligned16(x) && (ldx_halves % 8 == 0) && k > 0 && (k % 64 == 0);
}

// The gate and the up matrix of a fused gate / up / GeGLU tile share one descriptor for their scales and one for their biases:
// the two arrays of a kind must lie within 2 GiB of each other (they do wherever an expert is one blob).
bool geglu_arrays_near(const tf_projection *gate, const tf_projection *up) {
    const size_t bytes = (size_t)gate->rows * (size_t)(gate->cols / 64) * 2u;
    auto near = [&](const uint8_t *a, const uint8_t *b) {
        const uintptr_t lo = (uintptr_t)(a < b ? a : b), hi = (uintptr_t)(a < b ? b : a);
        return hi - lo + bytes <= (size_t)0x7FFFFFFF;
    };
    return near(at(gate->scales, gate->scales_offset), at(up->scales, up->scales_offset)) &&
           near(at(gate->biases, gate->biases_offset), at(up->biases, up->biases_offset));
}

// a shared expert's tiles may ride in the grouped launches: its output rows leave as whole 16-byte pieces
bool dense_ride_ok(const DenseRide &ride) {
    return aligned16(ride.y) && ride.down->rows % 8 == 0 && ride.ldy % 8 == 0 && geglu_arrays_near(ride.gate, ride.up);
}

int32_t launch_grouped_phase1_mfma(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off,
                                   const ChunkList &cl, uint32_t n_chunks_upper, const tf_prefill_pair *pairs,
                                   const half_t *hidden, long hidden_stride, half_t *acts, uint32_t acts_pair_base, int d, int f,
                                   tf_dtype sd, const DenseRide *ride) {
    const uint32_t grouped = (uint32_t)((f + kP1BN - 1) / kP1BN) * ((n_chunks_upper + kChunkRun - 1) / kChunkRun * kChunkRun);
    const GroupedP1Args a = {tab, off, cl, pairs, hidden, hidden_stride, acts, acts_pair_base, d, f};
    if (ride) {
        // the shared expert's gate / up / GeGLU tiles ahead of the grouped tiles (the full-height, longest tiles first), padded
        // to a multiple of 8 blocks so that both kinds keep their XCDs
        const DenseGegluArgs dense = dense_geglu_args(ride->gate, ride->up, ride->x, ride->ldx, ride->acts, (long)ride->gate->rows, ride->rows);
        const uint32_t extra = (dense_grid((uint32_t)(ride->rows + kQmmBM - 1) / kQmmBM, (uint32_t)((int)ride->gate->rows + kGegluBN - 1) / kGegluBN) + kXcds - 1) / kXcds * kXcds;
        if (sd == TF_BF16) hipLaunchKernelGGL(grouped_phase1_and_dense_geglu_kernel<0>, dim3(grouped + extra), dim3(64 * kGroupedWaves), 0, st, a, extra, dense);
        else hipLaunchKernelGGL(grouped_phase1_and_dense_geglu_kernel<1>, dim3(grouped + extra), dim3(64 * kGroupedWaves), 0, st, a, extra, dense);
        return check_launch(ctx, "grouped_phase1_mfma + shared gate/up");
    }
    if (sd == TF_BF16) hipLaunchKernelGGL(grouped_phase1_mfma_kernel<0>, dim3(grouped), dim3(64 * kGroupedWaves), 0, st, a);
    else hipLaunchKernelGGL(grouped_phase1_mfma_kernel<1>, dim3(grouped), dim3(64 * kGroupedWaves), 0, st, a);
    return check_launch(ctx, "grouped_phase1_mfma");
}

int32_t launch_grouped_down_mfma(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off,
                                 const ChunkList &cl, uint32_t n_chunks_upper, const tf_prefill_pair *pairs, const half_t *acts,
                                 uint32_t acts_pair_base, half_t *route_partials, int d, int f, int top_k, tf_dtype sd, const DenseRide *ride) {
    const uint32_t grouped = (uint32_t)((d + kDownBN - 1) / kDownBN) * ((n_chunks_upper + kChunkRun - 1) / kChunkRun * kChunkRun);
    const GroupedDownArgs a = {tab, off, cl, pairs, acts, acts_pair_base, route_partials, d, f, top_k};
    if (ride) {
        const tf_projection *dn = ride->down;   // ride->y: 16-byte aligned rows of whole 16-byte pieces (dense_ride_ok)
        const DenseArgs dense = dense_args(at(dn->weights, dn->weights_offset), at(dn->scales, dn->scales_offset), at(dn->biases, dn->biases_offset),
                                           ride->acts, (long)dn->cols, ride->y, ride->ldy, ride->rows, (int)dn->rows, (int)dn->cols);
        const uint32_t extra = (dense_grid((uint32_t)(ride->rows + kQmmBM - 1) / kQmmBM, (uint32_t)((int)dn->rows + kQmmBN - 1) / kQmmBN) + kXcds - 1) / kXcds * kXcds;
        if (sd == TF_BF16) hipLaunchKernelGGL(grouped_down_and_dense_kernel<0>, dim3(grouped + extra), dim3(64 * kGroupedWaves), 0, st, a, extra, dense);
        else hipLaunchKernelGGL(grouped_down_and_dense_kernel<1>, dim3(grouped + extra), dim3(64 * kGroupedWaves), 0, st, a, extra, dense);
        return check_launch(ctx, "grouped_down_mfma + shared down");
    }
    if (sd == TF_BF16) hipLaunchKernelGGL(grouped_down_mfma_kernel<0>, dim3(grouped), dim3(64 * kGroupedWaves), 0, st, a);
    else hipLaunchKernelGGL(grouped_down_mfma_kernel<1>, dim3(grouped), dim3(64 * kGroupedWaves), 0, st, a);
    return check_launch(ctx, "grouped_down_mfma");
}

}  // namespace tfk

namespace {

// Y[m, n] = X[m, k] . W[n, k]^T on the matrix cores.  Operands as qmm_operands_ok() demands; ldx / ldy in halves.
// 128-row tiles even when they leave compute units idle (144 blocks at 2048 x 2112): 64-row blocks, twice as many, repeat
// each weight tile's dequantisation and measured slower (0.18 ms against 0.155 ms for the three shared-expert GEMMs).
int32_t launch_qmm_dense(tf_ctx *ctx, hipStream_t st, const uint8_t *w, const uint8_t *s, const uint8_t *b, const half_t *x, long ldx,
                         half_t *y, long ldy, int m, int n, int k, tf_dtype sd) {
    const dim3 grid(dense_grid((uint32_t)(m + kQmmBM - 1) / kQmmBM, (uint32_t)(n + kQmmBN - 1) / kQmmBN));
    const DenseArgs a = dense_args(w, s, b, x, ldx, y, ldy, m, n, k);
    if (a.rows_vectorizable) {
        if (sd == TF_BF16) hipLaunchKernelGGL((qmm_dense_kernel<0, true>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((qmm_dense_kernel<1, true>), grid, dim3(256), 0, st, a);
    } else {
        if (sd == TF_BF16) hipLaunchKernelGGL((qmm_dense_kernel<0, false>), grid, dim3(256), 0, st, a);
        else hipLaunchKernelGGL((qmm_dense_kernel<1, false>), grid, dim3(256), 0, st, a);
    }
    return check_launch(ctx, "int4_qmm");
}

// A[m, f] = GeGLU(half(X . gate^T), half(X . up^T)); a 16-byte aligned, lda % 8 == 0, f % 8 == 0, geglu_arrays_near(gate, up)
int32_t launch_qmm_dense_geglu(tf_ctx *ctx, hipStream_t st, const tf_projection *gate, const tf_projection *up, const half_t *x, long ldx,
                               half_t *a_out, long lda, int m, tf_dtype sd) {
    const int f = (int)gate->rows;
    // 2048 x 2112 makes 272 blocks for 256 CUs: the 16 CUs that get two set the time (79 us; a block alone takes 46 us).
    // 544 half-height blocks, which fill every CU twice, measured slower still (+8 us): a block's weight expansion costs
    // the same for 64 rows as for 128.
    const dim3 grid(dense_grid((uint32_t)(m + kQmmBM - 1) / kQmmBM, (uint32_t)(f + kGegluBN - 1) / kGegluBN));
    const DenseGegluArgs a = dense_geglu_args(gate, up, x, ldx, a_out, lda, m);
    if (sd == TF_BF16) hipLaunchKernelGGL(qmm_dense_geglu_kernel<0>, grid, dim3(256), 0, st, a);
    else hipLaunchKernelGGL(qmm_dense_geglu_kernel<1>, grid, dim3(256), 0, st, a);
    return check_launch(ctx, "prefill_shared_expert gate/up");
}

// [rows, intermediate] fp16 activations of the block form of the shared expert, owned by the context
int32_t shared_block_acts(tf_ctx *ctx, size_t halves, half_t *&out) {
    const size_t need = halves * sizeof(half_t);
    if (ctx->shared_block_acts_bytes < need) return scratch_too_small(ctx, "prefill_shared_expert", need, ctx->shared_block_acts_bytes);
    out = static_cast<half_t *>(ctx->shared_block_acts);
    return TF_OK;
}

constexpr uint32_t kSharedBlockMinRows = 8;   // fewer rows go through the single-row chain, bit-identical to decode

// ---- 8-bit projections over a block of rows ----------------------------------------------------------------------
// Y[M, N] = X[M, K] . W[N, K]^T on the matrix cores with the 8-bit weights expanded on the way into the instruction,
// w = half(q * s + b) - the rounding point of the 4-bit matrix-core path; GEGLU: two weight matrices,
// Y = half(gelu_tanh(half(gate)) * half(up)).  No LDS: a wave owns a 32 x 32 tile of the output and reads its operands
// straight from memory in the instruction's own layout; grid (N / 32, ceil(M / 32)), one wave per block (a block of a few
// dozen rows makes few tiles: they should land on as many CUs as possible).
// K is walked in runs of 32: lane (i, kb) takes bytes 32 p + 16 kb .. + 15 of weight row i and the same 16 activations of its
// activation row; the first 8 of each run feed one matrix instruction, the last 8 the next (the order of the contraction
// index is free as long as both operands agree).  Two quantization groups (128 k) are in
// flight while the previous two are multiplied.  K % 64 == 0, N % 32 == 0, rows 16-byte aligned.
template <bool GEGLU, int SD>
__global__ __launch_bounds__(64) void qmm8_nt_kernel(const half_t *X, long ldx, const uint8_t *W0, const uint8_t *S0, const uint8_t *B0, const uint8_t *W1,
                                                     const uint8_t *S1, const uint8_t *B1, half_t *Y, long ldy, int M, int N, int K) {
    constexpr int GB = 2;                    // groups per block of requests
    const int lane = threadIdx.x;
    const int i = lane & 31, kb = lane >> 5;
    const int m0 = blockIdx.y * 32, n0 = blockIdx.x * 32;
    const half_t *xr = X + (size_t)min(m0 + i, M - 1) * ldx + 16 * kb;
    const size_t wrow = (size_t)(n0 + i) * K + 16 * kb, sbrow = (size_t)(n0 + i) * (K >> 6) * 2;
    const int groups = K >> 6, blocks = (groups + GB - 1) / GB;
    float16_t acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc0[r] = acc1[r] = 0.0f;
    struct Operands {
        u32x4 a[GB][2][2];                   // [group][run of 32][first / last 8 activations]
        u32x4 w0[GB][2], w1[GB][2];          // [group][run]: 16 weights
        uint16_t s0[GB], b0[GB], s1[GB], b1[GB];
    };
    Operands op[2];
    auto request = [&](Operands &o, int blk) {
#pragma unroll
        for (int g = 0; g < GB; ++g) {
            const int grp = min(blk * GB + g, groups - 1);     // past the end: the last group again, never multiplied
#pragma unroll
            for (int run = 0; run < 2; ++run) {
                const int k = grp * 64 + run * 32;
                o.a[g][run][0] = load16(xr + k);
                o.a[g][run][1] = load16(xr + k + 8);
                o.w0[g][run] = load16(W0 + wrow + k);
                if constexpr (GEGLU) o.w1[g][run] = load16(W1 + wrow + k);
            }
            o.s0[g] = *reinterpret_cast<const uint16_t *>(S0 + sbrow + grp * 2);
            o.b0[g] = *reinterpret_cast<const uint16_t *>(B0 + sbrow + grp * 2);
            if constexpr (GEGLU) {
                o.s1[g] = *reinterpret_cast<const uint16_t *>(S1 + sbrow + grp * 2);
                o.b1[g] = *reinterpret_cast<const uint16_t *>(B1 + sbrow + grp * 2);
            }
        }
    };
    // 16 bytes -> 16 fp16 weights half(q s + b).  An 8-bit scale is a 255th of the group's range and usually lies below
    // fp16's normal range, where a direct conversion would drop mantissa bits: a bf16 scale goes in as its mantissa (in
    // [1, 2)) and its power of two (exact in fp16 down to 2^-24) separately, w = (q m) 2^e + b.
    auto expand = [&](const u32x4 w, uint16_t sv, uint16_t bv, half8_t &first, half8_t &last) {
        const float sf = sb_to_f32<SD>(sv);
        const half_t bh = (half_t)sb_to_f32<SD>(bv);
        half_t mh, ph;
        if constexpr (SD == 0) {
            const uint32_t bits = __float_as_uint(sf);
            mh = (half_t)__uint_as_float((bits & 0x807FFFFFu) | 0x3F800000u);
            ph = (half_t)__uint_as_float(bits & 0x7F800000u);      // 0 for a zero scale
        } else {
            mh = (half_t)sf;                                       // an fp16 scale is what it is
            ph = (half_t)1.0f;
        }
        const half2_t m2 = {mh, mh}, p2 = {ph, ph}, b2 = {bh, bh}, bias = {(half_t)1024.0f, (half_t)1024.0f};
        u32x4 lo, hi;
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const half2_t q = as_half2(__builtin_amdgcn_perm(0x64646464u, w[j >> 1], (j & 1) ? 0x04030402u : 0x04010400u)) - bias;
            const uint32_t v = as_u32(__builtin_elementwise_fma(q * m2, p2, b2));
            if (j < 4) lo[j] = v; else hi[j - 4] = v;
        }
        first = __builtin_bit_cast(half8_t, lo);
        last = __builtin_bit_cast(half8_t, hi);
    };
    auto multiply = [&](const Operands &o, int blk) {
#pragma unroll
        for (int g = 0; g < GB; ++g) {
            if (blk * GB + g >= groups) break;
#pragma unroll
            for (int run = 0; run < 2; ++run) {
                half8_t f0, l0;
                expand(o.w0[g][run], o.s0[g], o.b0[g], f0, l0);
                const half8_t af = __builtin_bit_cast(half8_t, o.a[g][run][0]), al = __builtin_bit_cast(half8_t, o.a[g][run][1]);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, f0, acc0, 0, 0, 0);
                acc0 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, l0, acc0, 0, 0, 0);
                if constexpr (GEGLU) {
                    half8_t f1, l1;
                    expand(o.w1[g][run], o.s1[g], o.b1[g], f1, l1);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(af, f1, acc1, 0, 0, 0);
                    acc1 = __builtin_amdgcn_mfma_f32_32x32x16_f16(al, l1, acc1, 0, 0, 0);
                }
            }
        }
    };
    request(op[0], 0);
    for (int blk = 0; blk < blocks; blk += 2) {
        request(op[1], blk + 1);
        multiply(op[0], blk);
        request(op[0], blk + 2);
        if (blk + 1 < blocks) multiply(op[1], blk + 1);
    }
    const int n = n0 + acc_col(lane);
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int m = m0 + acc_row(r, lane);
        if (m < M) {
            if constexpr (GEGLU) Y[(size_t)m * ldy + n] = (half_t)(gelu_tanh((float)(half_t)acc0[r]) * (float)(half_t)acc1[r]);
            else Y[(size_t)m * ldy + n] = (half_t)acc0[r];
        }
    }
}

// TF_ERR_UNAVAILABLE: the operands do not allow it; the caller falls back to the row-grouped kernels
int32_t shared8_block_mfma(tf_ctx *ctx, hipStream_t st, const tf_projection *gate, const tf_projection *up, const tf_projection *down, const half_t *x,
                           uint32_t x_stride, half_t *y, uint32_t y_stride, uint32_t rows, half_t *acts, tf_dtype sd) {
    const uint32_t f = gate->rows, d = gate->cols;
    const uint8_t *w[3] = {at(gate->weights, gate->weights_offset), at(up->weights, up->weights_offset), at(down->weights, down->weights_offset)};
    if (!(aligned16(w[0]) && aligned16(w[1]) && aligned16(w[2]) && aligned16(x) && x_stride % 8 == 0 && d % 64 == 0 && f % 64 == 0 &&
          (sd == TF_BF16 || sd == TF_FP16) && rows <= 65535u * 32u))
        return TF_ERR_UNAVAILABLE;
    const uint8_t *sc[3], *bi[3];
    const tf_projection *proj[3] = {gate, up, down};
    for (int p = 0; p < 3; ++p) {
        sc[p] = at(proj[p]->scales, proj[p]->scales_offset);
        bi[p] = at(proj[p]->biases, proj[p]->biases_offset);
    }
    const dim3 g1(f / 32, (rows + 31) / 32), g2(d / 32, (rows + 31) / 32);
    if (sd == TF_BF16) {
        hipLaunchKernelGGL((qmm8_nt_kernel<true, 0>), g1, dim3(64), 0, st, x, (long)x_stride, w[0], sc[0], bi[0], w[1], sc[1], bi[1], acts, (long)f, (int)rows,
                           (int)f, (int)d);
        hipLaunchKernelGGL((qmm8_nt_kernel<false, 0>), g2, dim3(64), 0, st, acts, (long)f, w[2], sc[2], bi[2], nullptr, nullptr, nullptr, y, (long)y_stride,
                           (int)rows, (int)d, (int)f);
    } else {
        hipLaunchKernelGGL((qmm8_nt_kernel<true, 1>), g1, dim3(64), 0, st, x, (long)x_stride, w[0], sc[0], bi[0], w[1], sc[1], bi[1], acts, (long)f, (int)rows,
                           (int)f, (int)d);
        hipLaunchKernelGGL((qmm8_nt_kernel<false, 1>), g2, dim3(64), 0, st, acts, (long)f, w[2], sc[2], bi[2], nullptr, nullptr, nullptr, y, (long)y_stride,
                           (int)rows, (int)d, (int)f);
    }
    return check_launch(ctx, "shared expert 8-bit block");
}

constexpr uint32_t kShared8MfmaMinRows = 16;   // fewer rows: a weight row against four activation rows at a time (tf_moe.hip)


}  // namespace

extern "C" {

int32_t tf_int4_qmm(tf_ctx *ctx, tf_stream stream, const void *weights, uint64_t weights_offset, const void *scales,
                    uint64_t scales_offset, const void *biases, uint64_t biases_offset, const void *x, uint64_t x_offset,
                    void *y, uint64_t y_offset, int32_t m, int32_t n, int32_t k, tf_dtype scale_dtype) {
    TF_REQUIRE(ctx, ctx && weights && scales && biases && x && y, TF_ERR_INVALID_ARGUMENT, "int4_qmm: null argument");
    // MPPPrefillInt4QMM.encode's guard list (MPPPrefillInt4QMM.swift:40-56): anything it refuses is "unavailable", not an error
    // (the tiles stage scales twelve bytes at a time: a matrix with fewer than six of them is left to the exact kernel)
    const bool shape_ok = m > 0 && n > 0 && k > 0 && (k % (int32_t)TF_GROUP_SIZE == 0) && (int64_t)n * (k / (int32_t)TF_GROUP_SIZE) >= 6;
    const bool offs_ok = scales_offset % 2 == 0 && biases_offset % 2 == 0 && x_offset % 2 == 0 && y_offset % 2 == 0;
    if (!shape_ok || !offs_ok || !(scale_dtype == TF_BF16 || scale_dtype == TF_FP16)) return fail(ctx, TF_ERR_UNAVAILABLE, "int4_qmm: unsupported shape or offsets");
    const uint8_t *w = at(weights, weights_offset);
    const half_t *xp = reinterpret_cast<const half_t *>(at(x, x_offset));
    if (!qmm_operands_ok(w, xp, k, k) || !aligned(at(y, y_offset), 2)) return fail(ctx, TF_ERR_UNAVAILABLE, "int4_qmm: operands are not 16-byte aligned");
    half_t *yp = reinterpret_cast<half_t *>(at(y, y_offset));
    return launch_qmm_dense(ctx, static_cast<hipStream_t>(stream), w, at(scales, scales_offset), at(biases, biases_offset), xp, k, yp, n, m,
                            n, k, scale_dtype);
}

}  // extern "C"

namespace {

// tf_prefill_shared_expert_int4_block.  With `plan`: nothing is launched; the arguments are checked as ever and, where the
// call would run the 4-bit matrix-core kernels, *plan describes them (plan->rows > 0) for a caller that places their tiles
// in launches of its own; plan->rows == 0: the call takes another route and is to be made as usual.
int32_t shared_expert_block_impl(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *y, uint64_t y_offset,
                                 const tf_projection *gate, const tf_projection *up, const tf_projection *down,
                                 void *scratch_gate, uint64_t scratch_gate_offset, uint64_t scratch_gate_length,
                                 void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length, void *scratch_act,
                                 uint64_t scratch_act_offset, uint64_t scratch_act_length, uint32_t query_count, uint32_t d,
                                 uint32_t intermediate, uint32_t x_stride_elements, uint32_t y_stride_elements,
                                 uint32_t weight_bits, tf_dtype scale_dtype, DenseRide *plan) {
    if (plan) plan->rows = 0;
    TF_REQUIRE(ctx, ctx != nullptr, TF_ERR_INVALID_ARGUMENT, "prefill_shared_expert: null context");
    TF_REQUIRE(ctx, weight_bits == 4 || weight_bits == 8, TF_ERR_UNSUPPORTED_BITS, "SharedExpert unsupported weight bits: %u", weight_bits);
    TF_REQUIRE(ctx, x && y && gate && up && down && scratch_gate && scratch_up && scratch_act, TF_ERR_INVALID_ARGUMENT,
               "prefill_shared_expert: null argument");
    TF_REQUIRE(ctx, d > 0, TF_ERR_INVALID_ARGUMENT, "prefill_shared_expert: d must be positive");
    TF_REQUIRE(ctx, intermediate > 0, TF_ERR_INVALID_ARGUMENT, "prefill_shared_expert: intermediate must be positive");
    TF_REQUIRE(ctx, x_stride_elements >= d, TF_ERR_INVALID_ARGUMENT, "prefill_shared_expert: x stride is too small");
    TF_REQUIRE(ctx, y_stride_elements >= d, TF_ERR_INVALID_ARGUMENT, "prefill_shared_expert: y stride is too small");
    TF_REQUIRE(ctx, gate->rows == intermediate && gate->cols == d && up->rows == intermediate && up->cols == d && down->rows == d &&
                        down->cols == intermediate,
               TF_ERR_DIMENSION_MISMATCH, "expected gate/up=(%u,%u) down=(%u,%u)", intermediate, d, d, intermediate);
    if (query_count == 0) return TF_OK;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const half_t *xp = reinterpret_cast<const half_t *>(at(x, x_offset));
    half_t *yp = reinterpret_cast<half_t *>(at(y, y_offset));
    const uint8_t *gw = at(gate->weights, gate->weights_offset), *uw = at(up->weights, up->weights_offset);
    const uint8_t *dw = at(down->weights, down->weights_offset);
    const bool pointers = gate->weights && gate->scales && gate->biases && up->weights && up->scales && up->biases && down->weights &&
                          down->scales && down->biases;
    const bool even = x_offset % 2 == 0 && y_offset % 2 == 0 && gate->scales_offset % 2 == 0 && gate->biases_offset % 2 == 0 &&
                      up->scales_offset % 2 == 0 && up->biases_offset % 2 == 0 && down->scales_offset % 2 == 0 && down->biases_offset % 2 == 0;
    const bool block_path = weight_bits == 4 && pointers && even && query_count >= kSharedBlockMinRows && (scale_dtype == TF_BF16 || scale_dtype == TF_FP16) &&
                            qmm_operands_ok(gw, xp, x_stride_elements, (int)d) && aligned16(uw) && aligned16(dw) &&
                            intermediate % TF_GROUP_SIZE == 0 && query_count <= (uint32_t)INT32_MAX && geglu_arrays_near(gate, up);
    if (plan && !block_path) return TF_OK;
    if (weight_bits == 8 && pointers && even && query_count >= 2) {
        // 8-bit projections.  Up to kShared8MfmaMinRows - 1 rows: rows in groups against each weight row, bit-identical to the
        // rows one by one.  From there on the matrix cores: every weight is rounded to fp16 as half(q s + b) first (the
        // reference's staged-affine rounding point), so a row agrees with the single-row chain within the 8-bit shared
        // expert's tolerance, not bit for bit (scales keep their precision down to 2^-24; weights themselves below fp16's
        // normal range, 6e-5, keep an absolute spacing of 6e-8).
        TF_REQUIRE(ctx, scratch_act_offset + (uint64_t)intermediate * 2 <= scratch_act_length, TF_ERR_SCRATCH_TOO_SMALL,
                   "SharedExpertInt8 scratch too small: scratchAct offset %llu + needed %llu exceeds length %llu",
                   (unsigned long long)scratch_act_offset, (unsigned long long)intermediate * 2, (unsigned long long)scratch_act_length);
        half_t *acts8 = nullptr;
        int32_t rc8 = shared_block_acts(ctx, (size_t)query_count * intermediate, acts8);
        if (rc8 != TF_OK) return rc8;
        if (query_count >= kShared8MfmaMinRows) {
            rc8 = shared8_block_mfma(ctx, st, gate, up, down, xp, x_stride_elements, yp, y_stride_elements, query_count, acts8, scale_dtype);
            if (rc8 != TF_ERR_UNAVAILABLE) return rc8;
        }
        rc8 = shared8_block(ctx, st, gate, up, down, xp, x_stride_elements, yp, y_stride_elements, query_count, acts8, scale_dtype);
        if (rc8 != TF_ERR_UNAVAILABLE) return rc8;
    }
    if (!block_path) {
        // PrefillSharedExpert.encodeBlock itself: the single-row chain once per row, every row through the same scratch
        for (uint32_t row = 0; row < query_count; ++row) {
            const uint64_t xo = x_offset + (uint64_t)row * x_stride_elements * 2, yo = y_offset + (uint64_t)row * y_stride_elements * 2;
            const int32_t rc = tf_shared_expert_int4(ctx, stream, x, xo, xo + (uint64_t)d * 2, gate, up, down, y, yo, yo + (uint64_t)d * 2,
                                                     scratch_gate, scratch_gate_offset, scratch_gate_length, scratch_up, scratch_up_offset,
                                                     scratch_up_length, scratch_act, scratch_act_offset, scratch_act_length, weight_bits,
                                                     scale_dtype);
            if (rc != TF_OK) return rc;
        }
        return TF_OK;
    }
    // the caller's scratch holds one row (the reference's contract); it must still be large enough for that row
    const uint64_t required = (uint64_t)intermediate * 2;
    TF_REQUIRE(ctx, scratch_gate_offset + required <= scratch_gate_length && scratch_up_offset + required <= scratch_up_length &&
                        scratch_act_offset + required <= scratch_act_length,
               TF_ERR_SCRATCH_TOO_SMALL, "SharedExpert scratch too small: need %llu bytes per intermediate buffer", (unsigned long long)required);
    half_t *acts = nullptr;
    int32_t rc = shared_block_acts(ctx, (size_t)query_count * intermediate, acts);
    if (rc != TF_OK) return rc;
    if (plan) {
        *plan = DenseRide{gate, up, down, xp, (long)x_stride_elements, acts, yp, (long)y_stride_elements, (int)query_count};
        return TF_OK;
    }
    rc = launch_qmm_dense_geglu(ctx, st, gate, up, xp, (long)x_stride_elements, acts, (long)intermediate, (int)query_count, scale_dtype);
    if (rc != TF_OK) return rc;
    return launch_qmm_dense(ctx, st, dw, at(down->scales, down->scales_offset), at(down->biases, down->biases_offset), acts, (long)intermediate,
                            yp, (long)y_stride_elements, (int)query_count, (int)d, (int)intermediate, scale_dtype);
}

}  // namespace

namespace tfk {

int32_t shared_expert_block_plan(tf_ctx *ctx, const void *x, uint64_t x_offset, void *y, uint64_t y_offset, const tf_projection *gate,
                                 const tf_projection *up, const tf_projection *down, void *scratch_gate, uint64_t scratch_gate_offset,
                                 uint64_t scratch_gate_length, void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length,
                                 void *scratch_act, uint64_t scratch_act_offset, uint64_t scratch_act_length, uint32_t query_count,
                                 uint32_t d, uint32_t intermediate, uint32_t x_stride_elements, uint32_t y_stride_elements,
                                 uint32_t weight_bits, tf_dtype scale_dtype, DenseRide *plan) {
    return shared_expert_block_impl(ctx, nullptr, x, x_offset, y, y_offset, gate, up, down, scratch_gate, scratch_gate_offset, scratch_gate_length,
                                    scratch_up, scratch_up_offset, scratch_up_length, scratch_act, scratch_act_offset, scratch_act_length,
                                    query_count, d, intermediate, x_stride_elements, y_stride_elements, weight_bits, scale_dtype, plan);
}

}  // namespace tfk

extern "C" {

int32_t tf_prefill_shared_expert_int4_block(tf_ctx *ctx, tf_stream stream, const void *x, uint64_t x_offset, void *y, uint64_t y_offset,
                                            const tf_projection *gate, const tf_projection *up, const tf_projection *down,
                                            void *scratch_gate, uint64_t scratch_gate_offset, uint64_t scratch_gate_length,
                                            void *scratch_up, uint64_t scratch_up_offset, uint64_t scratch_up_length, void *scratch_act,
                                            uint64_t scratch_act_offset, uint64_t scratch_act_length, uint32_t query_count, uint32_t d,
                                            uint32_t intermediate, uint32_t x_stride_elements, uint32_t y_stride_elements,
                                            uint32_t weight_bits, tf_dtype scale_dtype) {
    return shared_expert_block_impl(ctx, stream, x, x_offset, y, y_offset, gate, up, down, scratch_gate, scratch_gate_offset, scratch_gate_length,
                                    scratch_up, scratch_up_offset, scratch_up_length, scratch_act, scratch_act_offset, scratch_act_length,
                                    query_count, d, intermediate, x_stride_elements, y_stride_elements, weight_bits, scale_dtype, nullptr);
}

}  // extern "C"

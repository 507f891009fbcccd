// int4 x fp16 matrix multiply on the CDNA4 matrix cores: Y[M,N] = X[M,K] . W[N,K]^T with W in the affine group-64
// int4 layout.  A block of four (or eight) waves owns a 128 x 256 (or 128 x 512) output tile, each wave 128 rows x 64
// columns, and walks K one quantization group (64) at a time:
//
//   W   In v_mfma_f32_32x32x16_f16 lane (i, kb) supplies, for output column i, the 8 weights of k-slots 8 kb .. 8 kb + 7.
//       The lane reads 16 packed bytes of "its" row (32 nibbles: the kb-th half of the group) and expands one 32-bit
//       word (8 nibbles) per MFMA straight into the operand registers as half(q * s + b), the rounding point of the
//       reference's staged-affine path (tensorops.metal:57-94).  MFMA number d of the group then covers
//       k = {8d .. 8d+7} u {32+8d .. 32+8d+7}.  Reading "its" row straight from global memory would touch 32 cache
//       lines per load instruction; instead the load unit copies the packed rows into a wave-private LDS area two K
//       steps at a time (64 contiguous bytes per row, four lanes per row), and the lanes pick their 16 bytes there.
//       Scales and biases are loaded two groups at a time (one 32-bit load per row and array).
//   X   is copied by the load unit from global memory straight into LDS (global_load_lds_dwordx4: no staging registers,
//       no vector instructions), two K steps ahead, into a ring of three stages shared by the four waves.  A stage is
//       128 rows x 8 chunks of 16 bytes; chunk c of row r sits at position c ^ ((r >> 1) & 7) of its row, which keeps
//       the fragment reads free of bank conflicts although the copies land contiguously.
//   The fragment reads are software-pipelined by hand (the fragments of MFMA group d + 1 are requested before group d
//   is multiplied) and written as inline assembly with explicit waits: the compiler would otherwise make every LDS read
//   wait for all outstanding copies, the prefetched ones included.
//
// Row indirection makes the same loop serve the grouped expert GEMMs: X rows can be gathered through a row table
// (tokens routed to one expert) and Y rows scattered through another; row tiles beyond the rows present are skipped.
#pragma once

#include "tf_common.hpp"

namespace tfk {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kQmmBM = 128;      // rows per block tile (4 MFMA row tiles)
constexpr int kQmmWaveN = 64;    // columns per wave (2 MFMA column tiles)
constexpr int kQmmStageBytes = kQmmBM * 8 * 16;  // one X stage
constexpr int kQmmWBytes = 64 * 64;               // packed W rows of one wave for two K steps: 64 rows x 64 bytes
// A block is NW waves (4 or 8) that share the X ring: with 8 waves the same activation rows serve twice as many output
// columns, so a tile's activations are fetched half as often; such a block has a CU to itself.
template <int NW>
struct QmmGeom {
    static constexpr int kThreads = NW * 64;
    static constexpr int kBN = NW * kQmmWaveN;                                     // columns per block tile
    static constexpr int kAChunks = kQmmBM * 8 / kThreads;                         // 16-byte X chunks copied per thread and K step
    static constexpr int kLoopLdsBytes = 3 * kQmmStageBytes + NW * 2 * kQmmWBytes; // X ring + two W buffers per wave
};
constexpr int kQmmBN = QmmGeom<4>::kBN;
constexpr int kQmmLdsBytes = QmmGeom<4>::kLoopLdsBytes;

// 8 nibbles of one word -> 8 fp16 weights half(q * s + b) in element order.  A byte holds two neighbouring elements:
// v_perm_b32 copies it into both halves of a register, one v_and_or_b32 leaves the low nibble in the low half as
// 1024 + q (0x6400 | q) and the high nibble in place in the high half as 64 + q (0x5400 | q << 4); both offsets are
// removed exactly, and q * s + b is one fp16 fused multiply-add on fp16 copies of s and b: four instructions a pair.
// v_and_or_b32 takes no literal operands, so mask and exponent bits live in registers (see nibble_consts()).
struct NibbleConsts {
    uint32_t mask, exponents;
};
__device__ __forceinline__ NibbleConsts nibble_consts() {
    NibbleConsts c{0x00F0000Fu, 0x54006400u};
    asm("" : "+v"(c.mask), "+v"(c.exponents));   // opaque: kept in registers instead of being re-materialised as literals
    return c;
}
__device__ __forceinline__ half8_t dequant_word(uint32_t v, half2_t s2, half2_t b2, const NibbleConsts &c) {
    const half2_t offs = {(half_t)1024.0f, (half_t)64.0f};
    half2_t w[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const uint32_t both = __builtin_amdgcn_perm(0u, v, 0x0c000c00u | ((uint32_t)p << 16) | (uint32_t)p);
        const half2_t q = as_half2((both & c.mask) | c.exponents) - offs;
        w[p] = __builtin_elementwise_fma(q, s2, b2);
    }
    return half8_t{w[0][0], w[0][1], w[1][0], w[1][1], w[2][0], w[2][1], w[3][0], w[3][1]};
}

// A bf16 scale or bias times the row's power of two, as an fp16 pair.  The power of two goes into the exponent field while the
// value is widened to fp32 (one shift-and-add instead of a shift): exact for every normal value, since the row's largest value
// bounds the sum of the fields; zeros and subnormals come out below 2^-26 and round to fp16 zero.
template <int SD>
__device__ __forceinline__ half2_t sb_to_half2(uint16_t v, uint32_t pre) {
    half_t h;
    if constexpr (SD == 0) h = (half_t)__uint_as_float(((uint32_t)v << 16) + pre);
    else h = (half_t)sb_to_f32<SD>(v);          // fp16 scales are what they are
    return half2_t{h, h};
}

// 16-byte slot of X chunk (row r, chunk c of 8) inside one stage
__device__ __forceinline__ int a_slot(int r, int c) { return r * 8 + (c ^ ((r >> 1) & 7)); }

// What a thread needs to know about the X chunks it copies: slot (threads per block) q + threadIdx.x of every stage receives the chunk
// at byte offset off[q] + 128 kt of the tensor the descriptor covers (rows beyond the tile repeat a valid row; nobody
// reads what they produce).  32-bit offsets: the rows of one tile must lie within 4 GiB of the descriptor's base.
typedef __amdgpu_buffer_rsrc_t qmm_rsrc_t;
// 16 bytes per lane from a buffer straight into LDS: lane l's bytes land at dst + 16 l (dst wave-uniform)
__device__ __forceinline__ void lds_copy16(qmm_rsrc_t rsrc, uint32_t dst, uint32_t lane_offset, int uniform_offset) {
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void *)(uintptr_t)dst, 16, lane_offset, uniform_offset, 0, 0);
}
template <int NW>
struct QmmARows {
    qmm_rsrc_t rsrc;
    uint32_t off[QmmGeom<NW>::kAChunks];
};
template <int NW>
__device__ __forceinline__ int qmm_a_row_of(int q) { return (QmmGeom<NW>::kThreads * q + (int)threadIdx.x) >> 3; }
// row_byte_offset: where the row of slot group q starts, relative to the descriptor's base
template <int NW>
__device__ __forceinline__ void qmm_a_rows_set(QmmARows<NW> &a, int q, uint64_t row_byte_offset) {
    const int p = QmmGeom<NW>::kThreads * q + (int)threadIdx.x, r = p >> 3;
    a.off[q] = (uint32_t)row_byte_offset + (uint32_t)(((p & 7) ^ ((r >> 1) & 7)) * 16);
}

// The wave's weight rows (32 per column tile), as buffer descriptors over the whole matrices (scalar registers) plus
// per-lane byte offsets.  Columns beyond the matrix read zeros (the descriptor ends with the matrix); what such lanes
// compute is never stored.
//   copy_off[t]: where copy number t of a two-step block starts for this lane: row 16 (t & 1) + lane / 4 of column
//                tile t / 2, 16-byte piece (lane & 3) ^ ((row / 4) & 3) of the row's 64 bytes (the XOR keeps the later
//                reads free of bank conflicts);
//   sb_off[j]:   the lane's own row (lane & 31) of tile j in the scale / bias arrays.
//   pre[j] / post[j]: a power of two 2^e per weight row (as e << 23, added to a value's fp32 bits) and 2^-e.  The expansion
//                computes half(q s + b) with fp16 copies of s and b; a bf16 scale below fp16's normal range (6.1e-5) would lose
//                mantissa bits in that copy.  A wave whose first two groups show such a scale (qmm_normalise_small_rows) scans
//                its rows' scales and biases once, multiplies them by 2^e on their way into the expansion, with e chosen from
//                the largest of them over the whole row so that every |q s + b| 2^e stays below 2^15, and multiplies the rows'
//                sums by 2^-e when they leave.  Both scalings are exact: half((q s + b) 2^e) = half(q s + b) 2^e wherever the
//                right side is a normal fp16 number, and where it is not (weights below 6.1e-5) the scaled form keeps the
//                mantissa the unscaled one drops.  Rows whose first groups have ordinary scales are left alone (e = 0): a later
//                group with a tiny scale then carries at most 15 x 2^-25 of absolute error per weight, next to weights of at
//                least 6.1e-5 in the same row.
//   scan_off[j], groups: the lane's row in the scale / bias arrays (clamped into the matrix) and its length, for that scan.
struct QmmBRows {
    qmm_rsrc_t w[2], s[2], b[2];
    uint32_t copy_off[4];
    uint32_t sb_off[2];
    uint32_t pre[2];
    float post[2];
    uint32_t scan_off[2];
    int groups;
};
// scales and biases of the lane's rows for two consecutive groups (low half: even group)
struct QmmSB {
    uint32_t s[2], b[2];
};
// Largest biased exponent field among the bf16 values of a row of `row_bytes` bytes (>= 16) that starts `row_off` bytes into
// `rsrc`; 0 when all are zero or subnormal.  The row is read in 16-byte pieces, all requested before the first is looked at;
// the last piece ends with the row (it may overlap the one before: a maximum does not mind), so nothing outside the row is read
// and nothing needs masking.  The exponent fields of a word's two values are compared in place with packed 16-bit maxima.
typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
template <int PIECES>
__device__ __forceinline__ uint32_t row_max_exponent(qmm_rsrc_t rsrc, uint32_t row_off, uint32_t row_bytes) {
    u32x4 v[PIECES];
#pragma unroll
    for (int p = 0; p < PIECES; ++p)
        v[p] = __builtin_bit_cast(u32x4, __builtin_amdgcn_raw_buffer_load_b128(rsrc, row_off + min(16u * p, row_bytes - 16u), 0, 0));
    u16x2 m = {0, 0};
#pragma unroll
    for (int p = 0; p < PIECES; ++p)
#pragma unroll
        for (int w = 0; w < 4; ++w) m = __builtin_elementwise_max(m, __builtin_bit_cast(u16x2, v[p][w] & 0x7F807F80u));
    return (uint32_t)max(m[0], m[1]) >> 7;
}
__device__ __forceinline__ uint32_t row_max_exponent_any(qmm_rsrc_t rsrc, uint32_t row_off, int groups) {
    const uint32_t row_bytes = (uint32_t)groups * 2u;
    uint32_t e = 0;
    if (groups < 8) {   // rows of fewer than 8 values: value by value
        for (int g = 0; g < groups; ++g) e = max(e, ((uint32_t)__builtin_amdgcn_raw_buffer_load_b16(rsrc, row_off + 2u * g, 0, 0) >> 7) & 0xFFu);
        return e;
    }
    for (uint32_t done = 0; done < row_bytes; done += 128u)      // 128 bytes (a row of 4096 columns) a round trip
        e = max(e, row_max_exponent<8>(rsrc, row_off + min(done, row_bytes - 16u), min(128u, max(row_bytes - done, 16u))));
    return e;
}
// sb: the scales of the wave's first two groups.  Wave-uniform decision; only bf16 scales need it.
__device__ __forceinline__ void qmm_normalise_small_rows(QmmBRows &rows, const uint32_t first_scales[2]) {
    bool small = false;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t lo = (first_scales[j] >> 7) & 0xFFu, hi = (first_scales[j] >> 23) & 0xFFu;   // exponent fields of the two bf16 values
        small = small || (lo != 0u && lo < 113u) || (hi != 0u && hi < 113u);                        // 2^-14 = fp16's smallest normal number
    }
    if (__builtin_amdgcn_ballot_w64(small) == 0ull) return;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        // every |s| < 2^(es - 126) and every |b| < 2^(eb - 126): with top = max(es + 4, eb), 15 |s| and |b| lie below 2^(top - 126),
        // and 2^(140 - top) brings them below 2^14, their sum below 2^15
        const uint32_t es = row_max_exponent_any(rows.s[j], rows.scan_off[j], rows.groups), eb = row_max_exponent_any(rows.b[j], rows.scan_off[j], rows.groups);
        const uint32_t top = max(es + 4u, eb);
        const int shift = top == 0u ? 0 : min(max(140 - (int)top, -100), 100);
        rows.pre[j] = (uint32_t)shift << 23;
        rows.post[j] = __uint_as_float((uint32_t)(127 - shift) << 23);
    }
}

// single (wave-uniform): the pair has only its first group (the last pair of an odd number of groups); a 32-bit load
// would run past the end of the last row.  Both arms issue the same number of loads.
__device__ __forceinline__ void qmm_sb_load(QmmSB &sb, const QmmBRows &rows, int pair, bool single) {
    if (single) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            sb.s[j] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rows.s[j], rows.sb_off[j], pair * 4, 0);
            sb.b[j] = (uint16_t)__builtin_amdgcn_raw_buffer_load_b16(rows.b[j], rows.sb_off[j], pair * 4, 0);
        }
    } else {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            sb.s[j] = __builtin_amdgcn_raw_buffer_load_b32(rows.s[j], rows.sb_off[j], pair * 4, 0);
            sb.b[j] = __builtin_amdgcn_raw_buffer_load_b32(rows.b[j], rows.sb_off[j], pair * 4, 0);
        }
    }
}
// packed W rows of K steps 2 pair, 2 pair + 1 -> the wave's LDS buffer at byte address `dst` (wave-uniform)
__device__ __forceinline__ void qmm_w_copy(const QmmBRows &rows, int pair, uint32_t dst) {
#pragma unroll
    for (int t = 0; t < 4; ++t) lds_copy16(rows.w[t >> 1], dst + t * 1024u, rows.copy_off[t], pair * 64);
}

// X tile of step kt -> LDS stage at byte address `stage` (wave-uniform); COPIES copies of 64 x 16 bytes per wave.  Copy q of
// the block covers rows 8 NW q .. 8 NW (q + 1) - 1, so a block that multiplies RT row tiles needs the first
// ceil(4 RT / NW) of the kAChunks copies only; the rows of the others are never read.
template <int NW, int COPIES>
__device__ __forceinline__ void qmm_a_copy(const QmmARows<NW> &a, int kt, uint32_t stage) {
    static_assert(COPIES >= 1 && COPIES <= QmmGeom<NW>::kAChunks, "copies per step");
    const uint32_t wave_base = stage + (threadIdx.x >> 6) * 1024u;
#pragma unroll
    for (int q = 0; q < COPIES; ++q) lds_copy16(a.rsrc, wave_base + (uint32_t)q * (uint32_t)(QmmGeom<NW>::kThreads * 16), a.off[q], kt * 128);
}

// ds_read_b128 at addr + OFFSET, invisible to the compiler's memory tracking (see the header comment)
template <int OFFSET>
__device__ __forceinline__ u32x4 lds_read16(uint32_t addr) {
    u32x4 v;
    asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}

// One K group for this wave: acc[mt][j] += X[mt*32.., group] . W_j[.., group]^T for the row tiles mt < RT, out of LDS
// stage STAGE.  frag[d]: LDS byte address of this lane's fragment for MFMA d in row tile 0 of stage 0.
// The fragments of MFMA group d + 1 are requested before group d is multiplied, and the weights of group d + 1 are
// expanded between the MFMAs of group d.
template <int SD, int RT, int STAGE, int HALF>
__device__ __forceinline__ void qmm_group(const u32x4 w[2], const QmmSB &sb, const uint32_t pre[2], const uint32_t frag[4], const NibbleConsts &nc,
                                          float16_t acc[4][2]) {
    half2_t s2[2], b2[2];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        s2[j] = sb_to_half2<SD>((uint16_t)(HALF ? sb.s[j] >> 16 : sb.s[j] & 0xFFFFu), pre[j]);
        b2[j] = sb_to_half2<SD>((uint16_t)(HALF ? sb.b[j] >> 16 : sb.b[j] & 0xFFFFu), pre[j]);
    }
    constexpr int base = STAGE * kQmmStageBytes;
    half8_t bf0 = dequant_word(w[0][0], s2[0], b2[0], nc);
    half8_t bf1 = dequant_word(w[1][0], s2[1], b2[1], nc);
    u32x4 af[2][4];
    af[0][0] = lds_read16<base>(frag[0]);
    if constexpr (RT > 1) af[0][1] = lds_read16<base + 4096>(frag[0]);
    if constexpr (RT > 2) af[0][2] = lds_read16<base + 8192>(frag[0]);
    if constexpr (RT > 3) af[0][3] = lds_read16<base + 12288>(frag[0]);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        // fragments of the next MFMA group first: they arrive while this group is multiplied
        if (d < 3) {
            af[(d + 1) & 1][0] = lds_read16<base>(frag[d + 1]);
            if constexpr (RT > 1) af[(d + 1) & 1][1] = lds_read16<base + 4096>(frag[d + 1]);
            if constexpr (RT > 2) af[(d + 1) & 1][2] = lds_read16<base + 8192>(frag[d + 1]);
            if constexpr (RT > 3) af[(d + 1) & 1][3] = lds_read16<base + 12288>(frag[d + 1]);
        }
        // this group's RT reads are older than the RT just requested
        constexpr int newer = RT;
        if (d < 3) {
            if constexpr (newer == 1) asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(af[d & 1][0]));
            if constexpr (newer == 2) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(af[d & 1][0]), "+v"(af[d & 1][1]));
            if constexpr (newer == 3) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(af[d & 1][0]), "+v"(af[d & 1][1]), "+v"(af[d & 1][2]));
            if constexpr (newer == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(af[d & 1][0]), "+v"(af[d & 1][1]), "+v"(af[d & 1][2]), "+v"(af[d & 1][3]));
        } else {
            if constexpr (RT == 1) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[d & 1][0]));
            if constexpr (RT == 2) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[d & 1][0]), "+v"(af[d & 1][1]));
            if constexpr (RT == 3) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[d & 1][0]), "+v"(af[d & 1][1]), "+v"(af[d & 1][2]));
            if constexpr (RT == 4) asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(af[d & 1][0]), "+v"(af[d & 1][1]), "+v"(af[d & 1][2]), "+v"(af[d & 1][3]));
        }
        half8_t nf0 = bf0, nf1 = bf1;
#pragma unroll
        for (int mt = 0; mt < RT; ++mt) {
            const half8_t a8 = __builtin_bit_cast(half8_t, af[d & 1][mt]);
            acc[mt][0] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a8, bf0, acc[mt][0], 0, 0, 0);
            acc[mt][1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a8, bf1, acc[mt][1], 0, 0, 0);
            // the next group's weights are expanded between the MFMAs
            if (d < 3 && mt == 0) nf0 = dequant_word(w[0][d + 1], s2[0], b2[0], nc);
            if (d < 3 && mt == (RT > 1 ? 1 : 0)) nf1 = dequant_word(w[1][d + 1], s2[1], b2[1], nc);
        }
        bf0 = nf0;
        bf1 = nf1;
    }
}

// The K loop.  The X tile of step kt lives in LDS stage kt % 3; the packed W rows of steps 2p, 2p + 1 in the wave's
// buffer p & 1, the scales / biases of those two groups in register slot p & 1.
// Even step kt = 2p:  barrier; request X(kt + 2), W(p + 1); multiply with the W words read from LDS at the end of the
//                     previous step; request the scales of pair p + 1; wait for X(kt + 1) (the AC + 8 newer
//                     requests stay in flight).
// Odd step:           barrier; request X(kt + 2); multiply; wait for X(kt + 1), W(p + 1) and the scales (the AC
//                     newer requests stay in flight); read the W words of both steps of pair p + 1 from LDS, switch
//                     to its scales.
// Requests are unconditional: past the end they repeat the last step or pair, which nobody reads, so that the number
// of requests in flight is the same at every wait.
template <int SD, int RT, int NW>
struct QmmLoop {
    // X copies per step and thread: those that carry rows of the RT row tiles.  A block with a single row tile keeps all
    // of them (the others re-read valid rows out of L2): without them chunks of 32 to 128 tokens measured 5 % slower.
    static constexpr int AC = RT == 1 ? QmmGeom<NW>::kAChunks : (4 * RT + NW - 1) / NW;
    const QmmARows<NW> &a;
    QmmBRows &rows;
    uint32_t lds;
    uint32_t frag[4];
    uint32_t wread;      // this lane's 16 bytes of column tile 0, first step of a pair, in the wave's W buffer 0
    uint32_t wbuf;       // the wave's W buffer 0
    int last, last_pair;
    bool odd_count;      // an odd number of K steps: the last pair has one group
    u32x4 w[2][2];       // [step of the pair][column tile]
    QmmSB sb, sb_next;
    uint32_t pb;         // (current pair & 1) * kQmmWBytes: which W buffer holds the current pair
    NibbleConsts nc;

    __device__ __forceinline__ void read_w(uint32_t at) {
        w[0][0] = lds_read16<0>(at);
        w[0][1] = lds_read16<2048>(at);
        w[1][0] = lds_read16<0>(at ^ 32u);
        w[1][1] = lds_read16<2048>(at ^ 32u);
        asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[1][0]), "+v"(w[1][1]));
    }

    template <int U3>
    __device__ __forceinline__ void even_step(int kt, float16_t acc[4][2]) {
        const int pair = kt >> 1;
        __builtin_amdgcn_s_barrier();
        qmm_a_copy<NW, AC>(a, min(kt + 2, last), lds + ((U3 + 2) % 3) * kQmmStageBytes);
        qmm_w_copy(rows, min(pair + 1, last_pair), wbuf + (pb ^ kQmmWBytes));
        qmm_group<SD, RT, U3, 0>(w[0], sb, rows.pre, frag, nc, acc);
        const int next_pair = min(pair + 1, last_pair);
        qmm_sb_load(sb_next, rows, next_pair, odd_count && next_pair == last_pair);
        // everything older than this step's AC + 4 + 4 requests (X, W, scales and biases) has landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AC + 8) : "memory");
    }
    template <int U3>
    __device__ __forceinline__ void odd_step(int kt, float16_t acc[4][2]) {
        __builtin_amdgcn_s_barrier();
        qmm_a_copy<NW, AC>(a, min(kt + 2, last), lds + ((U3 + 2) % 3) * kQmmStageBytes);
        qmm_group<SD, RT, U3, 1>(w[1], sb, rows.pre, frag, nc, acc);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AC) : "memory");   // only this step's X copies may still be on their way
        pb ^= kQmmWBytes;
        read_w(wread + pb);
        sb = sb_next;
    }

    __device__ __forceinline__ void run(int kt_count, int lane, float16_t acc[4][2]) {
        last = kt_count - 1;
        last_pair = last >> 1;
        odd_count = (kt_count & 1) != 0;
        const int i = lane & 31, kb = lane >> 5;
        const uint32_t frag0 = lds + (uint32_t)i * 128u + ((((uint32_t)kb * 4u) ^ (uint32_t)((i >> 1) & 7)) << 4);
#pragma unroll
        for (int d = 0; d < 4; ++d) frag[d] = frag0 ^ ((uint32_t)d << 4);   // lds is 128-byte aligned
        wbuf = lds + 3 * kQmmStageBytes + (threadIdx.x >> 6) * (2 * kQmmWBytes);   // NW such pairs of buffers follow the X ring
        wread = wbuf + (uint32_t)i * 64u + ((((uint32_t)kb) ^ (uint32_t)((i >> 2) & 3)) << 4);
        pb = 0;
        nc = nibble_consts();
        qmm_a_copy<NW, AC>(a, 0, lds);
        qmm_a_copy<NW, AC>(a, min(1, last), lds + kQmmStageBytes);
        qmm_w_copy(rows, 0, wbuf);
        qmm_sb_load(sb, rows, 0, odd_count && last_pair == 0);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        if constexpr (SD == 0) qmm_normalise_small_rows(rows, sb.s);
        read_w(wread);
        int kt0 = 0;
        for (; kt0 + 6 <= kt_count; kt0 += 6) {
            even_step<0>(kt0, acc);
            odd_step<1>(kt0 + 1, acc);
            even_step<2>(kt0 + 2, acc);
            odd_step<0>(kt0 + 3, acc);
            even_step<1>(kt0 + 4, acc);
            odd_step<2>(kt0 + 5, acc);
        }
        if (kt0 < kt_count) even_step<0>(kt0, acc);
        if (kt0 + 1 < kt_count) odd_step<1>(kt0 + 1, acc);
        if (kt0 + 2 < kt_count) even_step<2>(kt0 + 2, acc);
        if (kt0 + 3 < kt_count) odd_step<0>(kt0 + 3, acc);
        if (kt0 + 4 < kt_count) even_step<1>(kt0 + 4, acc);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // nothing may still be landing in LDS when the block moves on
        __builtin_amdgcn_s_barrier();
    }
};

template <int SD, int RT, int NW>
__device__ __forceinline__ void qmm_k_loop_rt(int kt_count, const QmmARows<NW> &a, QmmBRows &rows, uint32_t lds, int lane,
                                              float16_t acc[4][2]) {
    QmmLoop<SD, RT, NW> loop{a, rows, lds};
    loop.run(kt_count, lane, acc);
}

// row_tiles (1..4, block-uniform): 32-row tiles that hold rows; the others are not multiplied.
// lds: byte address of QmmGeom<NW>::kLoopLdsBytes of LDS, 128-byte aligned.
template <int SD, int NW>
__device__ __forceinline__ void qmm_k_loop(int kt_count, const QmmARows<NW> &a, QmmBRows &rows, uint32_t lds, int lane,
                                           int row_tiles, float16_t acc[4][2]) {
    switch (row_tiles) {
        case 1: qmm_k_loop_rt<SD, 1, NW>(kt_count, a, rows, lds, lane, acc); break;
        case 2: qmm_k_loop_rt<SD, 2, NW>(kt_count, a, rows, lds, lane, acc); break;
        case 3: qmm_k_loop_rt<SD, 3, NW>(kt_count, a, rows, lds, lane, acc); break;
        default: qmm_k_loop_rt<SD, 4, NW>(kt_count, a, rows, lds, lane, acc); break;
    }
}

// Accumulator element r of lane `lane` in a 32 x 32 block sits at (row, col):
__device__ __forceinline__ int acc_row(int r, int lane) { return (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3); }
__device__ __forceinline__ int acc_col(int lane) { return lane & 31; }

}  // namespace tfk

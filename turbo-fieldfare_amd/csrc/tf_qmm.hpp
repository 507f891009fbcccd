// int4 x fp16 matrix multiply on the CDNA4 matrix cores: Y[M,N] = X[M,K] . W[N,K]^T with W in the affine group-64
// int4 layout.  A block of four (or eight) waves owns a 128 x 256 (or 128 x 512) output tile, each wave 128 rows x 64
// columns, and walks K one quantization group (64) at a time:
//
//   W   In v_mfma_f32_32x32x16_f16 lane (i, kb) supplies, for output column i, the 8 weights of k-slots 8 kb .. 8 kb + 7.
//       The lane reads 16 packed bytes of "its" row (32 nibbles: the kb-th half of the group) and expands one 32-bit
//       word (8 nibbles) per MFMA round straight into the operand registers as half(q * s + b), the rounding point of the
//       reference's staged-affine path (tensorops.metal:57-94).  MFMA round d of the group then covers
//       k = {8d .. 8d+7} u {32+8d .. 32+8d+7}.  Reading "its" row straight from global memory would touch 32 cache
//       lines per load instruction; instead the load unit copies the packed rows into a wave-private LDS area two K
//       steps at a time (64 contiguous bytes per row, four lanes per row), and the lanes pick their 16 bytes there.
//       Scales and biases take the same road: a load of "its" rows' scales touches a cache line per lane, and the lines of a
//       row come round again every two steps, long after the X and W streams have pushed them out of the CU's cache (without
//       these loads the 2048-token prefill measured 10 % faster).  So every six steps the load unit copies twelve bytes - six
//       groups - of each of the wave's 64 rows per array into the wave's LDS (two instructions instead of twelve), and the
//       lanes read their two groups a pair from there.
//   X   is copied by the load unit from global memory straight into LDS (global_load_lds_dwordx4: no staging registers,
//       no vector instructions), two K steps ahead, into a ring of three stages shared by the four waves.  A stage is
//       128 rows x 8 chunks of 16 bytes; chunk c of row r sits at position c ^ ((r >> 1) & 7) of its row, which keeps
//       the fragment reads free of bank conflicts although the copies land contiguously.
//   The instruction stream of a K step is placed by hand: every MFMA, fragment read, wait and expansion instruction is a
//   volatile asm statement, in the order it is to issue.  Measured on this part, a wave's own vector instructions issue in
//   the shadow of its MFMAs as long as there are at most about five of them per MFMA (an MFMA holds the issue port for some
//   10 of its 32 cycles; with eight instructions per MFMA the pair takes 44 cycles instead of 32), and only when they are
//   spread out: left to the compiler, the 16 instructions that expand a word clump together between runs of back-to-back
//   MFMAs.  So a round (the 2 RT MFMAs of one 16-wide K slice) carries the expansion of the next round's two words in eight
//   parts of four instructions, one or more behind each MFMA; the last round of a step expands the first words of the next
//   step and reads that step's first fragments, after the block's one barrier of the step.
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
constexpr int kQmmSBWindowSteps = 6;              // K steps (groups) per staged window of scales / biases
constexpr int kQmmSBRowBytes = 2 * kQmmSBWindowSteps;   // per row and array, in memory
constexpr int kQmmSBSlotBytes = 16;               // per row and array in LDS: a 12-byte LDS-direct copy puts lane l's bytes at 16 l
constexpr int kQmmSBArrayBytes = 64 * kQmmSBSlotBytes;  // 64 rows (two column tiles) of one array
constexpr int kQmmSBBufBytes = 2048;              // one window: scales at 0, biases at kQmmSBArrayBytes; two such buffers per wave
static_assert(2 * kQmmSBArrayBytes <= kQmmSBBufBytes, "a window fits its buffer");
// A block is NW waves (4 or 8) that share the X ring: with 8 waves the same activation rows serve twice as many output
// columns, so a tile's activations are fetched half as often; such a block has a CU to itself.
template <int NW>
struct QmmGeom {
    static constexpr int kThreads = NW * 64;
    static constexpr int kBN = NW * kQmmWaveN;                                     // columns per block tile
    static constexpr int kAChunks = kQmmBM * 8 / kThreads;                         // 16-byte X chunks copied per thread and K step
    static constexpr int kWaveLdsBytes = kQmmWBytes + 2 * kQmmSBBufBytes;          // per wave: one W buffer, two scale windows
    static constexpr int kLoopLdsBytes = 3 * kQmmStageBytes + NW * kWaveLdsBytes;  // X ring + the waves' private areas
};
constexpr int kQmmBN = QmmGeom<4>::kBN;
constexpr int kQmmLdsBytes = QmmGeom<4>::kLoopLdsBytes;

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
//   sd / bd:     the scale and the bias arrays of BOTH column tiles under one descriptor each (the lower of the two arrays is
//                the base; they lie within 2 GiB of each other: two row ranges of one matrix, or gate and up of one expert).
//                Rows beyond a matrix are clamped to its last row (what such lanes compute is never stored).
//   sb_copy_off: where this lane's row starts in sd / bd when the lane copies for the wave: row lane & 31 of tile lane >> 5.
//   scan_s[j], scan_b[j], groups: the lane's own row (lane & 31) of tile j in sd / bd and its length, for the scan above.
//   s_end, b_end: where sd / bd end.  A copy that would reach past that end comes back as zeros, all of it: the last window of
//                the last row starts early enough to end with the array instead (qmm_sb_copy), and its readers allow for the
//                displacement (qmm_sb_read_tail).
struct QmmBRows {
    qmm_rsrc_t w[2], sd, bd;
    uint32_t copy_off[4];
    uint32_t sb_copy_off[2];   // [0]: in sd, [1]: in bd
    uint32_t pre[2];
    float post[2];
    uint32_t scan_s[2], scan_b[2];
    uint32_t s_end, b_end;     // bytes sd / bd cover
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
        const uint32_t es = row_max_exponent_any(rows.sd, rows.scan_s[j], rows.groups), eb = row_max_exponent_any(rows.bd, rows.scan_b[j], rows.groups);
        const uint32_t top = max(es + 4u, eb);
        const int shift = top == 0u ? 0 : min(max(140 - (int)top, -100), 100);
        rows.pre[j] = (uint32_t)shift << 23;
        rows.post[j] = __uint_as_float((uint32_t)(127 - shift) << 23);
    }
}

// Window `window` (groups 6 window .. 6 window + 5) of the wave's 64 rows: scales -> dst, biases -> dst + kQmmSBArrayBytes, twelve
// bytes a lane (lane l's land at 16 l).  Past the end of a row the copy takes what follows it; no step uses those groups.  A
// copy may not reach past the end of the arrays: where it would, it starts earlier by the excess.
__device__ __forceinline__ void qmm_sb_copy(const QmmBRows &rows, int window, uint32_t dst) {
    const uint32_t at = (uint32_t)window * kQmmSBRowBytes;
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rows.sd, (__attribute__((address_space(3))) void *)(uintptr_t)dst, 12,
                                             min(rows.sb_copy_off[0] + at, rows.s_end - kQmmSBRowBytes), 0, 0, 0);
    __builtin_amdgcn_raw_ptr_buffer_load_lds(rows.bd, (__attribute__((address_space(3))) void *)(uintptr_t)(dst + kQmmSBArrayBytes), 12,
                                             min(rows.sb_copy_off[1] + at, rows.b_end - kQmmSBRowBytes), 0, 0, 0);
}
template <int OFFSET>
__device__ __forceinline__ uint32_t lds_read4(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_b32 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
template <int OFFSET>
__device__ __forceinline__ uint32_t lds_read2(uint32_t addr) {
    uint32_t v;
    asm volatile("ds_read_u16 %0, %1 offset:%2" : "=v"(v) : "v"(addr), "n"(OFFSET));
    return v;
}
// The lane's scales and biases of pair PAIR (0..2) of the window at `at` (the lane's row of tile 0 in the scale area): LDS
// reads, to be waited for by the caller.
template <int PAIR>
__device__ __forceinline__ void qmm_sb_read(QmmSB &sb, uint32_t at) {
    sb.s[0] = lds_read4<PAIR * 4>(at);
    sb.s[1] = lds_read4<PAIR * 4 + 32 * kQmmSBSlotBytes>(at);
    sb.b[0] = lds_read4<PAIR * 4 + kQmmSBArrayBytes>(at);
    sb.b[1] = lds_read4<PAIR * 4 + kQmmSBArrayBytes + 32 * kQmmSBSlotBytes>(at);
}
// The same in a window that reaches past the end of the rows: the row that ends its array was copied from an earlier start, by a
// number of bytes that need not be a multiple of four, so the two values of a pair are read one by one.  Rare (the last
// window of a row): the reads are waited for on the spot.
template <int PAIR>
__device__ __forceinline__ void qmm_sb_read_tail(QmmSB &sb, const QmmBRows &rows, int window, uint32_t at) {
    const uint32_t reach = (uint32_t)(window + 1) * kQmmSBRowBytes;
    uint32_t lo[4], hi[4];
#pragma unroll
    for (int j = 0; j < 2; ++j) {
        const uint32_t ds = (uint32_t)max((int)(rows.scan_s[j] + reach) - (int)rows.s_end, 0), db = (uint32_t)max((int)(rows.scan_b[j] + reach) - (int)rows.b_end, 0);
        if (j == 0) {
            lo[0] = lds_read2<PAIR * 4>(at + ds);
            hi[0] = lds_read2<PAIR * 4 + 2>(at + ds);
            lo[2] = lds_read2<PAIR * 4 + kQmmSBArrayBytes>(at + db);
            hi[2] = lds_read2<PAIR * 4 + kQmmSBArrayBytes + 2>(at + db);
        } else {
            lo[1] = lds_read2<PAIR * 4 + 32 * kQmmSBSlotBytes>(at + ds);
            hi[1] = lds_read2<PAIR * 4 + 32 * kQmmSBSlotBytes + 2>(at + ds);
            lo[3] = lds_read2<PAIR * 4 + kQmmSBArrayBytes + 32 * kQmmSBSlotBytes>(at + db);
            hi[3] = lds_read2<PAIR * 4 + kQmmSBArrayBytes + 32 * kQmmSBSlotBytes + 2>(at + db);
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+v"(lo[0]), "+v"(lo[1]), "+v"(lo[2]), "+v"(lo[3]), "+v"(hi[0]), "+v"(hi[1]), "+v"(hi[2]), "+v"(hi[3]));
    sb.s[0] = lo[0] | (hi[0] << 16);
    sb.s[1] = lo[1] | (hi[1] << 16);
    sb.b[0] = lo[2] | (hi[2] << 16);
    sb.b[1] = lo[3] | (hi[3] << 16);
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

// One MFMA; everything that must keep its place in the instruction stream is a volatile asm statement.
__device__ __forceinline__ void mfma_slot(float16_t &acc, const u32x4 &a, const u32x4 &b) {
    asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(acc) : "v"(a), "v"(b));
}
// Expansion of nibbles into fp16 weights half(q * s + b).  A byte holds two neighbouring elements: v_perm_b32 copies it into
// both halves of a register, one v_and_or_b32 leaves the low nibble in the low half as 1024 + q (0x6400 | q) and the high
// nibble in place in the high half as 64 + q (0x5400 | q << 4); a packed add removes both offsets exactly, and q * s + b is
// one packed fp16 fused multiply-add on fp16 copies of s and b: four instructions a byte.  Two bytes of word `w` (P and
// P + 1) are expanded together, in two halves of four instructions that go behind two consecutive MFMAs; the result of a
// packed instruction is read two instructions later at the earliest (read in the very next one it needs a wait state).
template <int P>
__device__ __forceinline__ void expand_first(uint32_t w, uint32_t mask, uint32_t &t0, uint32_t &t1) {
    asm volatile("v_perm_b32 %0, 0, %2, %3\n\tv_perm_b32 %1, 0, %2, %4\n\tv_and_or_b32 %0, %0, %5, %6\n\tv_and_or_b32 %1, %1, %5, %6"
                 : "=&v"(t0), "=&v"(t1)
                 : "v"(w), "s"(0x0c000c00u | ((uint32_t)P << 16) | (uint32_t)P), "s"(0x0c000c00u | ((uint32_t)(P + 1) << 16) | (uint32_t)(P + 1)), "v"(mask),
                   "s"(0x54006400u));
}
__device__ __forceinline__ void expand_second(uint32_t t0, uint32_t t1, uint32_t s2, uint32_t b2, uint32_t &o0, uint32_t &o1) {
    asm volatile("v_pk_add_f16 %0, %2, %4\n\tv_pk_add_f16 %1, %3, %4\n\tv_pk_fma_f16 %0, %0, %5, %6\n\tv_pk_fma_f16 %1, %1, %5, %6"
                 : "=&v"(o0), "=&v"(o1)
                 : "v"(t0), "v"(t1), "s"(0xD400E400u), "v"(s2), "v"(b2));   // (-64, -1024): the offsets of the two nibble positions
}

struct BFrag {
    uint32_t r[4];
    __device__ __forceinline__ u32x4 tuple() const { return u32x4{r[0], r[1], r[2], r[3]}; }
};

template <int SD, int RT, int NW>
struct QmmLoop {
    static constexpr int AC = RT == 1 ? QmmGeom<NW>::kAChunks : (4 * RT + NW - 1) / NW;
    const QmmARows<NW> &a;
    QmmBRows &rows;
    uint32_t lds;
    uint32_t frag[4];
    uint32_t wread, wbuf;      // the wave's W buffer and this lane's 16 bytes of column tile 0, first step of a pair, in it
    uint32_t sbuf, sbread;     // the wave's two scale windows and this lane's row of tile 0 in the first
    uint32_t sbp;              // which window is current: 0 or kQmmSBBufBytes
    int last, last_pair;
    u32x4 w[2][2];             // [step of the pair][column tile]
    QmmSB sb;                  // scales and biases of the current pair
    uint32_t mask;
    u32x4 af[2][4];
    BFrag bc[2], bn[2];
    uint32_t s2c[2], b2c[2];   // this group's scale / bias pairs (fp16 x 2)
    uint32_t tmp[4][2];

    template <int OFF>
    __device__ __forceinline__ void read_frags(int buf, uint32_t at) {
        af[buf][0] = lds_read16<OFF>(at);
        if constexpr (RT > 1) af[buf][1] = lds_read16<OFF + 4096>(at);
        if constexpr (RT > 2) af[buf][2] = lds_read16<OFF + 8192>(at);
        if constexpr (RT > 3) af[buf][3] = lds_read16<OFF + 12288>(at);
    }
    // waits until at most NEWER LDS reads are outstanding and ties the fragments of `buf` to the wait
    template <int NEWER>
    __device__ __forceinline__ void wait_frags(int buf) {
        if constexpr (RT == 1) asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(af[buf][0]) : "n"(NEWER));
        if constexpr (RT == 2) asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(af[buf][0]), "+v"(af[buf][1]) : "n"(NEWER));
        if constexpr (RT == 3) asm volatile("s_waitcnt lgkmcnt(%3)" : "+v"(af[buf][0]), "+v"(af[buf][1]), "+v"(af[buf][2]) : "n"(NEWER));
        if constexpr (RT == 4) asm volatile("s_waitcnt lgkmcnt(%4)" : "+v"(af[buf][0]), "+v"(af[buf][1]), "+v"(af[buf][2]), "+v"(af[buf][3]) : "n"(NEWER));
    }
    __device__ __forceinline__ void scales_of(uint32_t s, uint32_t b, int j, bool high, uint32_t &s2, uint32_t &b2) {
        s2 = as_u32(sb_to_half2<SD>((uint16_t)(high ? s >> 16 : s & 0xFFFFu), rows.pre[j]));
        b2 = as_u32(sb_to_half2<SD>((uint16_t)(high ? b >> 16 : b & 0xFFFFu), rows.pre[j]));
    }
    // part I of the eight expansion parts of one MFMA round: words wa (column tile 0), wb (tile 1) -> bn, with scales s2x / b2x
    template <int I>
    __device__ __forceinline__ void part(uint32_t wa, uint32_t wb, const uint32_t s2x[2], const uint32_t b2x[2]) {
        constexpr int c = I >> 1, j = c >> 1, p = (c & 1) * 2;
        if constexpr ((I & 1) == 0) expand_first<p>(j ? wb : wa, mask, tmp[c][0], tmp[c][1]);
        else expand_second(tmp[c][0], tmp[c][1], s2x[j], b2x[j], bn[j].r[p], bn[j].r[p + 1]);
    }
    template <int FROM, int TO>
    __device__ __forceinline__ void parts(uint32_t wa, uint32_t wb, const uint32_t s2x[2], const uint32_t b2x[2]) {
        if constexpr (FROM < TO) {
            part<FROM>(wa, wb, s2x, b2x);
            parts<FROM + 1, TO>(wa, wb, s2x, b2x);
        }
    }
    // the 2 RT MFMAs of one round with the eight parts spread behind them
    template <int M>
    __device__ __forceinline__ void round_slots(int buf, uint32_t wa, uint32_t wb, const uint32_t s2x[2], const uint32_t b2x[2], float16_t acc[4][2]) {
        if constexpr (M < 2 * RT) {
            const u32x4 b = bc[M & 1].tuple();
            mfma_slot(acc[M >> 1][M & 1], af[buf][M >> 1], b);
            parts<M * 8 / (2 * RT), (M + 1) * 8 / (2 * RT)>(wa, wb, s2x, b2x);
            round_slots<M + 1>(buf, wa, wb, s2x, b2x, acc);
        }
    }
    __device__ __forceinline__ void advance_b() {
#pragma unroll
        for (int j = 0; j < 2; ++j) bc[j] = bn[j];
    }

    // One K step: rounds 0..2 expand this group's words 1..3; the last round expands word 0 of the next group, after the
    // block has met (every wave has its last fragments of this stage, and the copies of the next stage have landed).
    // Steps come in cycles of six, (U3, HALF) = (0,0) (1,1) (2,0) (0,1) (1,0) (2,1), one window of scales a cycle:
    //   every step:          X(kt + 3) is requested at the meeting point (AC copies);
    //   second steps (HALF): the next pair's W words and scales are read from LDS, then W of the pair after it is requested
    //                        into the same buffer (4 copies);
    //   step (0,1):          also the next cycle's window of scales and biases (2 copies), read from step (2,1) on.
    // What a step waits for was requested two steps earlier; the counts below are what may still be on its way at each wait.
    template <int U3, int HALF>
    __device__ __forceinline__ void step(int kt, float16_t acc[4][2]) {
        constexpr int base = U3 * kQmmStageBytes;
        constexpr bool kWindowStep = U3 == 0 && HALF == 1;            // requests the next window
        constexpr bool kAfterWindowStep = U3 == 1 && HALF == 0;       // the step after it
#pragma unroll
        for (int d = 0; d < 3; ++d) {
            read_frags<base>((d + 1) & 1, frag[d + 1]);
            wait_frags<RT>(d & 1);
            round_slots<0>(d & 1, w[HALF][0][d + 1], w[HALF][1][d + 1], s2c, b2c, acc);
            advance_b();
        }
        const int pair = kt >> 1;
        // X(kt + 1) has landed [second steps: also W and, where due, the window requested two steps ago]; younger requests may be
        // under way: after a second step its X, W (and window) copies, after a first step its X copies
        if constexpr (HALF == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AC + 4 + (kAfterWindowStep ? 2 : 0)) : "memory");
        else asm volatile("s_waitcnt vmcnt(%0)" ::"n"(AC) : "memory");
        wait_frags<0>(1);
        __builtin_amdgcn_s_barrier();
        qmm_a_copy<NW, AC>(a, min(kt + 3, last), lds + base);
        uint32_t s2n[2], b2n[2];
        uint32_t wa, wb;
        if constexpr (HALF == 1) {
            if constexpr (kWindowStep) qmm_sb_copy(rows, kt / kQmmSBWindowSteps + 1, sbuf + (sbp ^ kQmmSBBufBytes));
            // the next pair's words and scales
            w[0][0] = lds_read16<0>(wread);
            w[0][1] = lds_read16<2048>(wread);
            w[1][0] = lds_read16<0>(wread ^ 32u);
            w[1][1] = lds_read16<2048>(wread ^ 32u);
            if constexpr (U3 == 2) sbp ^= kQmmSBBufBytes;            // (2,1): the next pair opens the next window
            {
                const int window = kt / kQmmSBWindowSteps + (U3 == 2 ? 1 : 0);
                if ((window + 1) * kQmmSBWindowSteps <= rows.groups) qmm_sb_read<U3 == 1 ? 1 : U3 == 0 ? 2 : 0>(sb, sbread + sbp);
                else qmm_sb_read_tail<U3 == 1 ? 1 : U3 == 0 ? 2 : 0>(sb, rows, window, sbread + sbp);
            }
            read_frags<((U3 + 1) % 3) * kQmmStageBytes>(0, frag[0]);
            mfma_slot(acc[0][0], af[1][0], bc[0].tuple());
            // the eight word and scale reads are older than the fragment reads; the wait is also a compiler barrier: the copy
            // into the W buffer below must not be moved ahead of the reads of that buffer
            if constexpr (RT == 1) asm volatile("s_waitcnt lgkmcnt(1)" : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[1][0]), "+v"(w[1][1]), "+v"(sb.s[0]), "+v"(sb.s[1]), "+v"(sb.b[0]), "+v"(sb.b[1]) : : "memory");
            if constexpr (RT == 2) asm volatile("s_waitcnt lgkmcnt(2)" : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[1][0]), "+v"(w[1][1]), "+v"(sb.s[0]), "+v"(sb.s[1]), "+v"(sb.b[0]), "+v"(sb.b[1]) : : "memory");
            if constexpr (RT == 3) asm volatile("s_waitcnt lgkmcnt(3)" : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[1][0]), "+v"(w[1][1]), "+v"(sb.s[0]), "+v"(sb.s[1]), "+v"(sb.b[0]), "+v"(sb.b[1]) : : "memory");
            if constexpr (RT == 4) asm volatile("s_waitcnt lgkmcnt(4)" : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[1][0]), "+v"(w[1][1]), "+v"(sb.s[0]), "+v"(sb.s[1]), "+v"(sb.b[0]), "+v"(sb.b[1]) : : "memory");
            // the W buffer has been read: the pair after the next goes into it
            qmm_w_copy(rows, min(pair + 2, last_pair), wbuf);
#pragma unroll
            for (int j = 0; j < 2; ++j) scales_of(sb.s[j], sb.b[j], j, false, s2n[j], b2n[j]);
            wa = w[0][0][0];
            wb = w[0][1][0];
        } else {
            read_frags<((U3 + 1) % 3) * kQmmStageBytes>(0, frag[0]);
#pragma unroll
            for (int j = 0; j < 2; ++j) scales_of(sb.s[j], sb.b[j], j, true, s2n[j], b2n[j]);
            wa = w[1][0][0];
            wb = w[1][1][0];
            mfma_slot(acc[0][0], af[1][0], bc[0].tuple());
        }
        parts<0, 8 / (2 * RT)>(wa, wb, s2n, b2n);
        round_slots<1>(1, wa, wb, s2n, b2n, acc);
        advance_b();
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            s2c[j] = s2n[j];
            b2c[j] = b2n[j];
        }
    }

    __device__ __forceinline__ void run(int kt_count, int lane, float16_t acc[4][2]) {
        last = kt_count - 1;
        last_pair = last >> 1;
        const int i = lane & 31, kb = lane >> 5;
        const uint32_t frag0 = lds + (uint32_t)i * 128u + ((((uint32_t)kb * 4u) ^ (uint32_t)((i >> 1) & 7)) << 4);
#pragma unroll
        for (int d = 0; d < 4; ++d) frag[d] = frag0 ^ ((uint32_t)d << 4);
        wbuf = lds + 3 * kQmmStageBytes + (threadIdx.x >> 6) * QmmGeom<NW>::kWaveLdsBytes;   // NW such areas follow the X ring
        wread = wbuf + (uint32_t)i * 64u + ((((uint32_t)kb) ^ (uint32_t)((i >> 2) & 3)) << 4);
        sbuf = wbuf + kQmmWBytes;
        sbread = sbuf + (uint32_t)i * kQmmSBSlotBytes;
        sbp = 0;
        mask = 0x00F0000Fu;
        asm volatile("" : "+v"(mask));
        qmm_a_copy<NW, AC>(a, 0, lds);
        qmm_w_copy(rows, 0, wbuf);
        qmm_sb_copy(rows, 0, sbuf);
        qmm_a_copy<NW, AC>(a, min(1, last), lds + kQmmStageBytes);
        qmm_a_copy<NW, AC>(a, min(2, last), lds + 2 * kQmmStageBytes);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * AC) : "memory");
        __builtin_amdgcn_s_barrier();
        w[0][0] = lds_read16<0>(wread);
        w[0][1] = lds_read16<2048>(wread);
        w[1][0] = lds_read16<0>(wread ^ 32u);
        w[1][1] = lds_read16<2048>(wread ^ 32u);
        if (kQmmSBWindowSteps <= rows.groups) qmm_sb_read<0>(sb, sbread);
        else qmm_sb_read_tail<0>(sb, rows, 0, sbread);
        read_frags<0>(0, frag[0]);
        asm volatile("s_waitcnt lgkmcnt(%8)" : "+v"(w[0][0]), "+v"(w[0][1]), "+v"(w[1][0]), "+v"(w[1][1]), "+v"(sb.s[0]), "+v"(sb.s[1]), "+v"(sb.b[0]), "+v"(sb.b[1]) : "n"(RT) : "memory");
        qmm_w_copy(rows, min(1, last_pair), wbuf);
        if constexpr (SD == 0) qmm_normalise_small_rows(rows, sb.s);
#pragma unroll
        for (int j = 0; j < 2; ++j) scales_of(sb.s[j], sb.b[j], j, false, s2c[j], b2c[j]);
        parts<0, 8>(w[0][0][0], w[0][1][0], s2c, b2c);
        advance_b();
        int kt0 = 0;
        for (; kt0 + 6 <= kt_count; kt0 += 6) {
            step<0, 0>(kt0, acc);
            step<1, 1>(kt0 + 1, acc);
            step<2, 0>(kt0 + 2, acc);
            step<0, 1>(kt0 + 3, acc);
            step<1, 0>(kt0 + 4, acc);
            step<2, 1>(kt0 + 5, acc);
        }
        if (kt0 < kt_count) step<0, 0>(kt0, acc);
        if (kt0 + 1 < kt_count) step<1, 1>(kt0 + 1, acc);
        if (kt0 + 2 < kt_count) step<2, 0>(kt0 + 2, acc);
        if (kt0 + 3 < kt_count) step<0, 1>(kt0 + 3, acc);
        if (kt0 + 4 < kt_count) step<1, 0>(kt0 + 4, acc);
        // nothing may still be landing in LDS or in registers when the block moves on; the accumulators are read by ordinary
        // instructions from here on
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_nop 15\n\ts_nop 15" ::: "memory");
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

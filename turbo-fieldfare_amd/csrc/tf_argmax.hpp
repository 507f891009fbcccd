// Argmax over a whole grid without a second launch: every block folds its best {value, index} into a small set of 64-bit
// cells with one atomic max, and the block that finishes last turns the cells into the winning index.
#pragma once

#include "tf_common.hpp"

namespace tfk {

struct Best {
    float v;
    uint32_t idx;
};

__device__ __forceinline__ void better(Best &b, float v, uint32_t idx) {
    if (v > b.v || (v == b.v && idx < b.idx)) {
        b.v = v;
        b.idx = idx;
    }
}

// Cells live in device memory owned by the context: kHeadCells keys followed by a 32-bit ticket counter, all zero between
// calls.  Key = (orderable(value) << 32 | ~index): larger value wins, equal values resolve to the lower index, 0 means
// "nothing to report".
constexpr uint32_t kHeadCells = 64;

__device__ __forceinline__ unsigned long long best_key(float v, uint32_t idx) {
    if (idx == 0xFFFFFFFFu) return 0ull;
    uint32_t u = __float_as_uint(v);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);   // monotone map of finite floats onto unsigned integers
    return ((unsigned long long)u << 32) | (unsigned long long)(0xFFFFFFFFu - idx);
}

// Called by every thread of a 256-thread block after lane 0 of wave w has written the wave's best to sv[w] / si[w].
// Writes out_token[0] (0 when no block reported anything) from the last block to finish and leaves the cells zeroed.
// Fold and ticket are device-scope atomics performed at the memory side, and the ticket is only requested after the fold
// has returned, so the block that draws the last ticket finds every fold in the cells (read with atomics as well)
// without any cache write-back or invalidate.
__device__ __forceinline__ void fold_block_best(const float *sv, const uint32_t *si, unsigned long long *cells, uint32_t *out_token) {
    __shared__ uint32_t is_last;
    const int lane = threadIdx.x & 63;
    const int wib = threadIdx.x >> 6;
    __syncthreads();
    if (threadIdx.x == 0) {
        Best b{sv[0], si[0]};
        for (int w = 1; w < 4; ++w) better(b, sv[w], si[w]);
        const unsigned long long key = best_key(b.v, b.idx);
        unsigned long long seen = 0ull;
        if (key) seen = atomicMax(cells + (blockIdx.x % kHeadCells), key);
        // the ticket increment depends on the value the fold returned
        uint32_t one = 1u;
        const uint32_t seen_lo = (uint32_t)seen;
        asm volatile("" : "+v"(one) : "v"(seen_lo));
        unsigned int *ticket = reinterpret_cast<unsigned int *>(cells + kHeadCells);
        is_last = atomicAdd(ticket, one) == gridDim.x - 1 ? 1u : 0u;
    }
    __syncthreads();
    if (is_last && wib == 0) {
        unsigned long long key = __hip_atomic_exchange(cells + lane, 0ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const unsigned long long other = __shfl_xor(key, off, kWave);
            key = other > key ? other : key;
        }
        if (lane == 0) {
            out_token[0] = key ? 0xFFFFFFFFu - (uint32_t)(key & 0xFFFFFFFFull) : 0u;
            __hip_atomic_store(reinterpret_cast<unsigned int *>(cells + kHeadCells), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

}  // namespace tfk

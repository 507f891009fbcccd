// Shared pieces of the prefill / multi-token path: POD layouts, expert lookup, work lists.
#pragma once

#include "tf_gemv_kernels.hpp"
#include "tf_qmm.hpp"

namespace tfk {

// Where the expert blobs live: a table of up to 16 (id, pointer) bindings — the reference's streamed tile
// (PrefillGroupedRoutedMoE.swift:185-216) — or a resident pool indexed by expert id.
struct ExpertTable {
    const uint8_t *blob[TF_MAX_TILE_EXPERTS];
    uint32_t local_id[TF_MAX_TILE_EXPERTS];
    uint32_t live;
    const uint8_t *pool;
    uint64_t stride;
    uint32_t num_experts;
};

// nullptr when the expert is not bound in the tile (the reference's kernels skip such pairs, prefill.metal:611-618).
__device__ __forceinline__ const uint8_t *expert_base(const ExpertTable &t, uint32_t expert) {
    if (t.pool) {
        const uint32_t e = expert < t.num_experts ? expert : t.num_experts - 1;
        return t.pool + (uint64_t)e * t.stride;
    }
    for (uint32_t s = 0; s < t.live; ++s)
        if (t.local_id[s] == expert) return t.blob[s];
    return nullptr;
}

// Work list: runs of sorted pairs that share one expert, each at most kChunkPairs long.  Either a short list passed with
// the kernel arguments or a device array written by the grouping kernel (with its length in device memory).
constexpr uint32_t kChunkPairs = 128;
constexpr uint32_t kInlineChunks = 48;
struct ChunkList {
    uint32_t n;
    tf_prefill_group inline_chunks[kInlineChunks];
    const tf_prefill_group *dev;
    const uint32_t *dev_n;
};

__device__ __forceinline__ bool get_chunk(const ChunkList &cl, uint32_t i, tf_prefill_group &out) {
    if (cl.dev) {
        if (i >= *cl.dev_n) return false;
        out = cl.dev[i];
    } else {
        if (i >= cl.n) return false;
        out = cl.inline_chunks[i];
    }
    return true;
}

// A shared expert's block of rows riding along in the launches of the grouped matrix-core kernels: its gate / up / GeGLU
// tiles ahead of the grouped gate / up tiles, its down tiles ahead of the grouped down tiles.
struct DenseRide {
    const tf_projection *gate, *up, *down;
    const half_t *x;      // [rows, gate->cols], row stride ldx halves
    long ldx;
    half_t *acts;         // [rows, gate->rows] activations between the two launches
    half_t *y;            // [rows, down->rows], row stride ldy halves
    long ldy;
    int rows;
};

// Operands of the grouped expert stages, as the launch helpers pass them on.
struct GroupedGeom {
    const tf_prefill_pair *pairs;
    const half_t *hidden;
    long hidden_stride;
    half_t *acts;
    uint32_t acts_pair_base;
    half_t *route_partials;
    int d, f, top_k;
};

// The quad kernels (tf_prefill_quad.hip): grouped gate / up / GeGLU and down for chunks of a few pairs, weights streamed once per
// expert.  kQuadMaxD / kQuadMaxF: the widest rows they take; the caller checks alignment and shape (run_grouped).
constexpr int kQuadMaxD = 3072, kQuadMaxF = 1024;
int32_t launch_grouped_quad(tf_ctx *ctx, hipStream_t st, const ExpertTable &tab, const tf_expert_offsets &off, const ChunkList &cl,
                            uint32_t n_chunks_upper, const GroupedGeom &g, tf_dtype sd, uint32_t stream_pairs);

}  // namespace tfk

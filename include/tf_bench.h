/*
 * tf_bench.h — measurement helpers exported by the same library as tf_kernels.h.
 *
 * Nothing here has a counterpart in the reference and nothing here belongs to the
 * drop-in surface: a runtime binds tf_kernels.h only.  The launches below let a
 * benchmark measure, in the same run that times the kernels, what a chain of
 * dependent launches costs when it moves no data and what read rate the part
 * sustains (the latency floor and the streaming ceiling the kernels are held against).
 */
#ifndef TF_BENCH_H
#define TF_BENCH_H

#include "tf_kernels.h"

#ifdef __cplusplus
extern "C" {
#endif

/* A launch of `blocks` x `threads_per_block` that reads in_word[0] in every block and writes out_word[0] from one thread:
 * chained on a stream, what dependent launches of those shapes cost when they move no data (the latency floor of a
 * multi-launch step). */
int32_t tf_bench_empty_launch(tf_ctx *ctx, tf_stream stream, uint32_t blocks, uint32_t threads_per_block,
                              const void *in_word, void *out_word);
/* A plain streaming read of `bytes` (multiple of 4096, 16-byte aligned) with the access pattern and cache policy of the
 * row streamers and no arithmetic: the read rate this part sustains, to hold the GEMV kernels against beside the
 * published peak. */
int32_t tf_bench_stream_read(tf_ctx *ctx, tf_stream stream, const void *data, uint64_t bytes, void *out_word);

/* The first `stages` launches of tf_moe_decode_step with that call's arguments (1: router logits; 2: + top-8 and phase 1;
 * 3: the whole step): chains of 1, 2 and 3 stages replayed side by side give each kernel's share of the step, boundary to its
 * predecessor included, without bracketing events. */
int32_t tf_bench_moe_decode_step_stages(tf_ctx *ctx, tf_stream stream, const void *router_weights, uint64_t router_weights_offset,
                                        const void *router_scales, uint64_t router_scales_offset, const void *router_biases,
                                        uint64_t router_biases_offset, const void *router_x, const void *effective_scale,
                                        uint64_t effective_scale_offset, const void *per_expert_scale, uint64_t per_expert_scale_offset,
                                        const void *expert_pool, uint64_t expert_pool_stride, uint32_t num_experts,
                                        const tf_expert_offsets *routed_offsets, const void *x, void *acts, const void *residual, void *y,
                                        void *out_indices, void *out_weights, uint32_t d, uint32_t f, uint32_t top_k, tf_dtype scale_dtype,
                                        uint32_t stages);

#ifdef __cplusplus
}
#endif
#endif /* TF_BENCH_H */

// C++ mirror of the reference's Swift kernel wrappers (Sources/TurboFieldfare/Kernels/**) over the C ABI.
// Class and method names follow the Swift ones; a "buffer" is a device pointer, the "command buffer" is the context's
// stream.  Contract violations that trap in Swift (`precondition`) and errors that `throw` there surface as tf::Error.
#pragma once

#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/tf_kernels.h"

namespace tf {

struct Error : std::runtime_error {
    int32_t status;
    Error(int32_t s, const std::string &what) : std::runtime_error(what), status(s) {}
};

// MetalContext (Infrastructure/Metal/MetalContext.swift:51-214): device + one in-order queue.
class Context {
public:
    explicit Context(int32_t device = 0, tf_stream stream = nullptr) : stream_(stream) {
        const int32_t rc = tf_ctx_create(device, &ctx_);
        if (rc != TF_OK) throw Error(rc, tf_status_string(rc));
    }
    ~Context() { tf_ctx_destroy(ctx_); }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    tf_ctx *raw() const { return ctx_; }
    tf_stream stream() const { return stream_; }
    void check(int32_t rc) const {
        if (rc != TF_OK) throw Error(rc, tf_last_error(ctx_));
    }
    // The Swift wrappers size their scratch in `init` (MoE.swift:92-99, LMHeadChainInt4.swift:38-51); here one call raises the
    // context's limits for all of them.  Set-up time only.
    void reserve(const tf_scratch_limits &limits) const { check(tf_ctx_reserve(ctx_, &limits)); }
    // commandBuffer.commit + waitUntilCompleted + checkCommandBufferError (MetalContext.swift:22-26)
    void waitUntilCompleted() const { check(tf_stream_synchronize(ctx_, stream_)); }

private:
    tf_ctx *ctx_ = nullptr;
    tf_stream stream_ = nullptr;
};

// DequantInt4GEMV (Kernels/Quant/DequantInt4GEMV.swift)
class DequantInt4GEMV {
public:
    explicit DequantInt4GEMV(const Context &context) : c_(context) {}
    void encode(const void *weights, uint64_t weightsOffset, const void *scales, uint64_t scalesOffset, const void *biases,
                uint64_t biasesOffset, const void *x, uint64_t xOffset, void *y, uint64_t yOffset, uint32_t m, uint32_t n) const {
        c_.check(tf_dequant_int4_gemv(c_.raw(), c_.stream(), weights, weightsOffset, scales, scalesOffset, biases, biasesOffset, x,
                                      xOffset, y, yOffset, m, n, TF_BF16, TF_FP16));
    }

private:
    const Context &c_;
};

// DequantInt8GEMV (Kernels/Quant/DequantInt8GEMV.swift)
class DequantInt8GEMV {
public:
    explicit DequantInt8GEMV(const Context &context) : c_(context) {}
    void encode(const void *weights, uint64_t weightsOffset, const void *scales, uint64_t scalesOffset, const void *biases,
                uint64_t biasesOffset, const void *x, uint64_t xOffset, void *y, uint64_t yOffset, uint32_t m, uint32_t n) const {
        c_.check(tf_dequant_int8_gemv(c_.raw(), c_.stream(), weights, weightsOffset, scales, scalesOffset, biases, biasesOffset, x,
                                      xOffset, y, yOffset, m, n, TF_BF16, TF_FP16));
    }

private:
    const Context &c_;
};

using MoEExpertOffsets = tf_expert_offsets;   // Kernels/MoE/MoE.swift:4-29

// MoE (Kernels/MoE/MoE.swift:31-313)
class MoE {
public:
    static constexpr uint32_t maxStreamedExperts = TF_MAX_STREAMED_EXPERTS;
    explicit MoE(const Context &context) : c_(context) {}

    void encodeRouterGemma4(const void *weights, uint64_t weightsOffset, const void *scales, uint64_t scalesOffset,
                            const void *biases, uint64_t biasesOffset, const void *hidden, const void *effectiveScale,
                            uint64_t effectiveScaleOffset, const void *perExpertScale, uint64_t perExpertScaleOffset,
                            void *outIndices, void *outWeights, uint32_t numExperts, uint32_t d, uint32_t topK) const {
        c_.check(tf_router_gemma4(c_.raw(), c_.stream(), weights, weightsOffset, scales, scalesOffset, biases, biasesOffset, hidden,
                                  effectiveScale, effectiveScaleOffset, perExpertScale, perExpertScaleOffset, outIndices, outWeights,
                                  numExperts, d, topK));
    }
    // makeRoutedArgumentBuffer (MoE.swift:161-171): eight host-chosen blobs
    tf_routed_blobs makeRoutedArgumentBuffer(const std::vector<const void *> &routedBlobs, uint32_t topK) const {
        if (topK != maxStreamedExperts || routedBlobs.size() != topK) throw Error(TF_ERR_INVALID_ARGUMENT, "routedBlobs.count must equal topK == 8");
        tf_routed_blobs r = {};
        for (uint32_t i = 0; i < topK; ++i) r.blobs[i] = routedBlobs[i];
        return r;
    }
    // resident experts: the indices the router wrote are read by the kernels themselves
    static tf_routed_blobs residentPool(const void *pool, uint64_t stride, const uint32_t *deviceIndices, uint32_t numExperts) {
        tf_routed_blobs r = {};
        r.pool = pool;
        r.pool_stride = stride;
        r.indices = deviceIndices;
        r.num_experts = numExperts;
        return r;
    }
    void encodeRoutedPersistentPhase1U16Load(const tf_routed_blobs &routed, const MoEExpertOffsets &routedOffsets, const void *x,
                                             void *acts, uint32_t d, uint32_t f, uint32_t topK) const {
        c_.check(tf_moe_phase1_gate_up_act(c_.raw(), c_.stream(), &routed, &routedOffsets, x, acts, d, f, topK, TF_BF16));
    }
    void encodeRoutedPersistentPhase1SubsetU16Load(const tf_routed_blobs &routed, const MoEExpertOffsets &routedOffsets, const void *x,
                                                   void *acts, const uint32_t *activeSlots, uint32_t activeCount, uint32_t d,
                                                   uint32_t f, uint32_t topK) const {
        c_.check(tf_moe_phase1_gate_up_act_subset(c_.raw(), c_.stream(), &routed, &routedOffsets, x, acts, activeSlots, activeCount, d,
                                                  f, topK, TF_BF16));
    }
    void encodeRoutedPersistentPhase2Reduce(const tf_routed_blobs &routed, const MoEExpertOffsets &routedOffsets, const void *acts,
                                            const void *routingWeights, const void *residual, void *y, uint32_t d, uint32_t f,
                                            uint32_t topK) const {
        c_.check(tf_moe_phase2_down_reduce(c_.raw(), c_.stream(), &routed, &routedOffsets, acts, routingWeights, residual, y, d, f, topK,
                                           TF_BF16));
    }

private:
    const Context &c_;
};

// RoPE (Kernels/Primitives/RoPE.swift:4-90)
class RoPE {
public:
    explicit RoPE(const Context &context) : c_(context) {}
    void encodeDefaultNeox(void *data, uint64_t dataOffset, uint32_t position, uint32_t headDim, uint32_t numHeads, uint32_t numTokens,
                           float theta = 10000.0f) const {
        c_.check(tf_rope_default_neox(c_.raw(), c_.stream(), data, dataOffset, position, headDim, numHeads, numTokens, theta));
    }
    void encodeProportionalNeox(void *data, uint64_t dataOffset, uint32_t position, uint32_t headDim, uint32_t numHeads, uint32_t numTokens,
                                uint32_t rotatedPairs, float theta = 1000000.0f) const {
        c_.check(tf_rope_proportional_neox(c_.raw(), c_.stream(), data, dataOffset, position, headDim, numHeads, numTokens, rotatedPairs, theta));
    }

private:
    const Context &c_;
};

// RMSNorm (Kernels/Primitives/RMSNorm.swift:52-136)
class RMSNorm {
public:
    explicit RMSNorm(const Context &context) : c_(context) {}
    void encodeBF16W(const void *x, uint64_t xOffset, const void *weight, uint64_t weightOffset, void *out, uint64_t outOffset, uint32_t d,
                     float eps) const {
        c_.check(tf_rmsnorm_bf16w(c_.raw(), c_.stream(), x, xOffset, weight, weightOffset, out, outOffset, d, eps));
    }
    void encodeNoScale(const void *x, uint64_t xOffset, void *out, uint64_t outOffset, uint32_t d, float eps) const {
        c_.check(tf_rmsnorm_no_scale(c_.raw(), c_.stream(), x, xOffset, out, outOffset, d, eps));
    }
    void encodeBF16WPerHead(const void *x, uint64_t xOffset, const void *weight, uint64_t weightOffset, void *out, uint64_t outOffset,
                            uint32_t headDim, uint32_t numHeads, float eps) const {
        c_.check(tf_rmsnorm_bf16w_perhead(c_.raw(), c_.stream(), x, xOffset, weight, weightOffset, out, outOffset, headDim, numHeads, eps));
    }
    void encodeNoScalePerHead(const void *x, uint64_t xOffset, void *out, uint64_t outOffset, uint32_t headDim, uint32_t numHeads, float eps) const {
        c_.check(tf_rmsnorm_no_scale_perhead(c_.raw(), c_.stream(), x, xOffset, out, outOffset, headDim, numHeads, eps));
    }

private:
    const Context &c_;
};

// PrefillRMSNorm (Kernels/Prefill/Primitives/PrefillPrimitives.swift:41-71)
class PrefillRMSNorm {
public:
    explicit PrefillRMSNorm(const Context &context) : c_(context) {}
    void encodeBF16W(const void *x, uint64_t xOffset, const void *weight, uint64_t weightOffset, void *out, uint64_t outOffset, uint32_t t,
                     uint32_t d, float eps) const {
        c_.check(tf_prefill_rmsnorm_bf16w_block(c_.raw(), c_.stream(), x, xOffset, weight, weightOffset, out, outOffset, t, d, eps));
    }

private:
    const Context &c_;
};

// PrefillPerHeadNorm (Kernels/Prefill/Primitives/PrefillPerHeadNorm.swift:4-85)
class PrefillPerHeadNorm {
public:
    explicit PrefillPerHeadNorm(const Context &context) : c_(context) {}
    void encodeBF16W(const void *x, uint64_t xOffset, const void *weight, uint64_t weightOffset, void *out, uint64_t outOffset,
                     uint32_t queryCount, uint32_t headDim, uint32_t numHeads, uint32_t tokenStrideElements, float eps) const {
        c_.check(tf_prefill_rmsnorm_bf16w_perhead_block(c_.raw(), c_.stream(), x, xOffset, weight, weightOffset, out, outOffset, queryCount, headDim,
                                                        numHeads, tokenStrideElements, eps));
    }
    void encodeNoScale(const void *x, uint64_t xOffset, void *out, uint64_t outOffset, uint32_t queryCount, uint32_t headDim, uint32_t numHeads,
                       uint32_t tokenStrideElements, float eps) const {
        c_.check(tf_prefill_rmsnorm_no_scale_perhead_block(c_.raw(), c_.stream(), x, xOffset, out, outOffset, queryCount, headDim, numHeads,
                                                           tokenStrideElements, eps));
    }

private:
    const Context &c_;
};

// PrefillRoPE (Kernels/Prefill/Primitives/PrefillRoPE.swift:4-89)
class PrefillRoPE {
public:
    explicit PrefillRoPE(const Context &context) : c_(context) {}
    void encodeDefaultNeox(void *data, uint64_t dataOffset, uint32_t startPosition, uint32_t queryCount, uint32_t headDim, uint32_t numHeads,
                           uint32_t tokenStrideElements, float theta = 10000.0f) const {
        c_.check(tf_prefill_rope_default_neox_block(c_.raw(), c_.stream(), data, dataOffset, startPosition, queryCount, headDim, numHeads,
                                                    tokenStrideElements, theta));
    }
    void encodeProportionalNeox(void *data, uint64_t dataOffset, uint32_t startPosition, uint32_t queryCount, uint32_t headDim, uint32_t numHeads,
                                uint32_t rotatedPairs, uint32_t tokenStrideElements, float theta = 1000000.0f) const {
        c_.check(tf_prefill_rope_proportional_neox_block(c_.raw(), c_.stream(), data, dataOffset, startPosition, queryCount, headDim, numHeads,
                                                         rotatedPairs, tokenStrideElements, theta));
    }

private:
    const Context &c_;
};

// PrefillQKVEpilogue (Kernels/Prefill/Epilogues/PrefillQKVEpilogue.swift:4-122)
class PrefillQKVEpilogue {
public:
    explicit PrefillQKVEpilogue(const Context &context) : c_(context) {}
    void encode(void *q, uint64_t qOffset, void *k, uint64_t kOffset, void *v, uint64_t vOffset, const void *qWeight, uint64_t qWeightOffset,
                const void *kWeight, uint64_t kWeightOffset, uint32_t startPosition, uint32_t queryCount, uint32_t headDim, uint32_t numQHeads,
                uint32_t numKVHeads, uint32_t qTokenStrideElements, uint32_t kvTokenStrideElements, float theta, uint32_t rotatedPairs,
                float eps) const {
        c_.check(tf_prefill_qkv_epilogue_block(c_.raw(), c_.stream(), q, qOffset, k, kOffset, v, vOffset, qWeight, qWeightOffset, kWeight,
                                               kWeightOffset, startPosition, queryCount, headDim, numQHeads, numKVHeads, qTokenStrideElements,
                                               kvTokenStrideElements, theta, rotatedPairs, eps));
    }

private:
    const Context &c_;
};

// FusedQKVEpilogue (Kernels/Fusions/FusedQKVEpilogue.swift:10-100)
class FusedQKVEpilogue {
public:
    explicit FusedQKVEpilogue(const Context &context) : c_(context) {}
    void encode(void *q, uint64_t qOffset, void *k, uint64_t kOffset, void *v, uint64_t vOffset, const void *qWeight, uint64_t qWeightOffset,
                const void *kWeight, uint64_t kWeightOffset, uint32_t headDim, uint32_t numQHeads, uint32_t numKVHeads, uint32_t position,
                float theta, uint32_t rotatedPairs, float eps) const {
        c_.check(tf_fused_qkv_epilogue(c_.raw(), c_.stream(), q, qOffset, k, kOffset, v, vOffset, qWeight, qWeightOffset, kWeight, kWeightOffset,
                                       headDim, numQHeads, numKVHeads, position, theta, rotatedPairs, eps));
    }

private:
    const Context &c_;
};

// Attention (Kernels/Attention/Attention.swift:26-214): sliding-window and full-causal decode attention
using AttentionSplitGeometry = tf_attention_split_geometry_t;
class Attention {
public:
    explicit Attention(const Context &context) : c_(context) {}
    static AttentionSplitGeometry splitGeometry(uint32_t numQHeads, uint32_t numKVHeads, uint32_t seqLen, uint32_t kvStart, bool preferGQASWA) {
        AttentionSplitGeometry g{};
        tf_attention_split_geometry(numQHeads, numKVHeads, seqLen, kvStart, preferGQASWA ? 1 : 0, &g);
        return g;
    }
    // scale <= 0: 1 / sqrt(headDim), the reference's nil
    void encodeSWA(const void *q, uint64_t qOffset, const void *k, uint64_t kOffset, const void *v, uint64_t vOffset, void *out, uint64_t outOffset,
                   uint32_t headDim, uint32_t numQHeads, uint32_t numKVHeads, uint32_t seqLen, uint32_t window, float scale = 0.0f,
                   uint32_t ringCapacity = 0) const {
        c_.check(tf_attention_swa(c_.raw(), c_.stream(), q, qOffset, k, kOffset, v, vOffset, out, outOffset, headDim, numQHeads, numKVHeads, seqLen,
                                  window, scale, ringCapacity));
    }
    void encodeFull(const void *q, uint64_t qOffset, const void *k, uint64_t kOffset, const void *v, uint64_t vOffset, void *out, uint64_t outOffset,
                    uint32_t headDim, uint32_t numQHeads, uint32_t numKVHeads, uint32_t seqLen, float scale = 0.0f) const {
        c_.check(tf_attention_full(c_.raw(), c_.stream(), q, qOffset, k, kOffset, v, vOffset, out, outOffset, headDim, numQHeads, numKVHeads, seqLen,
                                   scale));
    }

private:
    const Context &c_;
};

// PrefillAttention (Kernels/Attention/PrefillAttention.swift:43-118)
using PrefillAttentionParams = tf_prefill_attention_params;
class PrefillAttention {
public:
    explicit PrefillAttention(const Context &context) : c_(context) {}
    void encodeCausal(const void *q, uint64_t qOffset, const void *k, uint64_t kOffset, const void *v, uint64_t vOffset, void *out, uint64_t outOffset,
                      const PrefillAttentionParams &params, uint32_t kvRingCapacity = 0) const {
        c_.check(tf_prefill_attention_causal(c_.raw(), c_.stream(), q, qOffset, k, kOffset, v, vOffset, out, outOffset, &params, kvRingCapacity));
    }

private:
    const Context &c_;
};

using SharedExpertProjection = tf_projection;   // Kernels/MoE/SharedExpertInt8.swift:9-31

// SharedExpertRuntime / SharedExpertInt4 (Kernels/MoE/SharedExpertInt4.swift): 4- or 8-bit projections
class SharedExpertRuntime {
public:
    SharedExpertRuntime(const Context &context, int weightBits) : c_(context), weightBits_(weightBits) {
        if (weightBits != 4 && weightBits != 8)
            throw Error(TF_ERR_UNSUPPORTED_BITS, "SharedExpert unsupported weight bits: " + std::to_string(weightBits));
    }
    struct Buffer {   // an MTLBuffer's (contents, length)
        void *ptr;
        uint64_t length;
    };
    void encode(Buffer x, uint64_t xOffset, const SharedExpertProjection &gate, const SharedExpertProjection &up,
                const SharedExpertProjection &down, Buffer y, uint64_t yOffset, Buffer scratchGate, uint64_t scratchGateOffset,
                Buffer scratchUp, uint64_t scratchUpOffset, Buffer scratchAct, uint64_t scratchActOffset) const {
        c_.check(tf_shared_expert_int4(c_.raw(), c_.stream(), x.ptr, xOffset, x.length, &gate, &up, &down, y.ptr, yOffset, y.length,
                                       scratchGate.ptr, scratchGateOffset, scratchGate.length, scratchUp.ptr, scratchUpOffset,
                                       scratchUp.length, scratchAct.ptr, scratchActOffset, scratchAct.length, (uint32_t)weightBits_,
                                       TF_BF16));
    }

private:
    const Context &c_;
    int weightBits_;
};

// PrefillSharedExpert (Kernels/Prefill/MoE/PrefillSharedExpert.swift:4-58): the shared expert over a block of rows
class PrefillSharedExpert {
public:
    PrefillSharedExpert(const Context &context, int weightBits = 8) : c_(context), weightBits_(weightBits) {
        if (weightBits != 4 && weightBits != 8)
            throw Error(TF_ERR_UNSUPPORTED_BITS, "SharedExpert unsupported weight bits: " + std::to_string(weightBits));
    }
    using Buffer = SharedExpertRuntime::Buffer;
    void encodeBlock(const void *x, uint64_t xOffset, void *y, uint64_t yOffset, const SharedExpertProjection &gate,
                     const SharedExpertProjection &up, const SharedExpertProjection &down, Buffer scratchGate, uint64_t scratchGateOffset,
                     Buffer scratchUp, uint64_t scratchUpOffset, Buffer scratchAct, uint64_t scratchActOffset, uint32_t queryCount,
                     uint32_t d, uint32_t intermediate, uint32_t xStrideElements, uint32_t yStrideElements) const {
        c_.check(tf_prefill_shared_expert_int4_block(c_.raw(), c_.stream(), x, xOffset, y, yOffset, &gate, &up, &down, scratchGate.ptr,
                                                     scratchGateOffset, scratchGate.length, scratchUp.ptr, scratchUpOffset,
                                                     scratchUp.length, scratchAct.ptr, scratchActOffset, scratchAct.length, queryCount, d,
                                                     intermediate, xStrideElements, yStrideElements, (uint32_t)weightBits_, TF_BF16));
    }

private:
    const Context &c_;
    int weightBits_;
};

// SharedExpertInt8 (Kernels/MoE/SharedExpertInt8.swift:54-170): gate, up and the activation in one launch, then the down GEMV
class SharedExpertInt8 {
public:
    explicit SharedExpertInt8(const Context &context) : c_(context) {}
    using Buffer = SharedExpertRuntime::Buffer;
    void encode(Buffer x, uint64_t xOffset, const SharedExpertProjection &gate, const SharedExpertProjection &up,
                const SharedExpertProjection &down, Buffer y, uint64_t yOffset, Buffer scratchAct, uint64_t scratchActOffset) const {
        c_.check(tf_shared_expert_int8(c_.raw(), c_.stream(), x.ptr, xOffset, x.length, &gate, &up, &down, y.ptr, yOffset, y.length,
                                       scratchAct.ptr, scratchActOffset, scratchAct.length, TF_BF16));
    }
    void encodePhase1(Buffer x, uint64_t xOffset, const SharedExpertProjection &gate, const SharedExpertProjection &up, Buffer scratchAct,
                      uint64_t scratchActOffset) const {
        c_.check(tf_shared_expert_int8_phase1(c_.raw(), c_.stream(), x.ptr, xOffset, x.length, &gate, &up, scratchAct.ptr, scratchActOffset,
                                              scratchAct.length, TF_BF16));
    }
    void encodeDown(const SharedExpertProjection &down, Buffer y, uint64_t yOffset, Buffer scratchAct, uint64_t scratchActOffset) const {
        c_.check(tf_shared_expert_int8_down(c_.raw(), c_.stream(), &down, y.ptr, yOffset, y.length, scratchAct.ptr, scratchActOffset,
                                            scratchAct.length, TF_BF16));
    }

private:
    const Context &c_;
};

// SharedExpertInt4 (Kernels/MoE/SharedExpertInt4.swift:6-100) is the 4-bit instance of the runtime.
struct SharedExpertInt4 : SharedExpertRuntime {
    explicit SharedExpertInt4(const Context &context) : SharedExpertRuntime(context, 4) {}
};

// LMHeadChainInt4 (Kernels/Fusions/LMHeadChainInt4.swift)
class LMHeadChainInt4 {
public:
    explicit LMHeadChainInt4(const Context &context) : c_(context) {}
    void encodeGreedyDecode(const void *hidden, uint64_t hiddenOffset, const void *normWeight, uint64_t normOffset,
                            const void *weights, uint64_t weightsOffset, const void *scales, uint64_t scalesOffset,
                            const void *biases, uint64_t biasesOffset, void *outToken, uint32_t d, uint32_t vocab,
                            float rmsEps = 1e-6f) const {
        c_.check(tf_lm_head_greedy_int4(c_.raw(), c_.stream(), hidden, hiddenOffset, normWeight, normOffset, weights, weightsOffset,
                                        scales, scalesOffset, biases, biasesOffset, outToken, d, vocab, rmsEps, TF_BF16));
    }

private:
    const Context &c_;
};

using PrefillTokenExpertPair = tf_prefill_pair;   // Kernels/Prefill/MoE/PrefillRouter.swift:5-28
using PrefillMoEGroup = tf_prefill_group;         // Kernels/Prefill/MoE/PrefillMoEGrouping.swift:4-14
using PrefillMoETile = tf_prefill_tile;           // :17-29

// PrefillRouter (Kernels/Prefill/MoE/PrefillRouter.swift:30-112)
class PrefillRouter {
public:
    explicit PrefillRouter(const Context &context) : c_(context) {}
    void encodeGemma4Block(const void *weights, uint64_t weightsOffset, const void *scales, uint64_t scalesOffset, const void *biases,
                           uint64_t biasesOffset, const void *hidden, uint64_t hiddenOffset, const void *effectiveScale,
                           uint64_t effectiveScaleOffset, const void *perExpertScale, uint64_t perExpertScaleOffset,
                           void *outIndices, uint64_t outIndicesOffset, void *outWeights, uint64_t outWeightsOffset,
                           uint32_t queryCount, uint32_t numExperts, uint32_t d, uint32_t topK, uint32_t hiddenStrideElements) const {
        c_.check(tf_prefill_router_gemma4_block(c_.raw(), c_.stream(), weights, weightsOffset, scales, scalesOffset, biases,
                                                biasesOffset, hidden, hiddenOffset, effectiveScale, effectiveScaleOffset, perExpertScale,
                                                perExpertScaleOffset, outIndices, outIndicesOffset, outWeights, outWeightsOffset,
                                                queryCount, numExperts, d, topK, hiddenStrideElements));
    }
    static std::vector<PrefillTokenExpertPair> makeTokenExpertPairs(const std::vector<uint32_t> &indices,
                                                                    const std::vector<uint16_t> &weightsF16, int queryCount, int topK) {
        if (queryCount < 0 || topK < 0 || indices.size() != (size_t)queryCount * topK || weightsF16.size() != indices.size())
            throw Error(TF_ERR_INVALID_ARGUMENT, "indices/weights count mismatch");
        std::vector<PrefillTokenExpertPair> pairs(indices.size());
        const int32_t rc = tf_prefill_make_token_expert_pairs(indices.data(), weightsF16.data(), queryCount, topK, pairs.data());
        if (rc != TF_OK) throw Error(rc, "makeTokenExpertPairs");
        return pairs;
    }

private:
    const Context &c_;
};

// PrefillMoEGroupedRoutes + PrefillMoEGrouping.groupTokenExpertPairs (Kernels/Prefill/MoE/PrefillMoEGrouping.swift:31-193)
struct PrefillMoEGroupedRoutes {
    std::vector<PrefillTokenExpertPair> sortedPairs;
    std::vector<uint32_t> perExpertOffsets, perExpertCounts;
    std::vector<PrefillMoEGroup> groups;
    std::vector<PrefillMoETile> tiles;
    int queryCount = 0;
    int maxPairsPerExpert() const { uint32_t m = 0; for (const auto &g : groups) m = g.pair_count > m ? g.pair_count : m; return (int)m; }
    int maxPairsPerTile() const { uint32_t m = 0; for (const auto &t : tiles) m = t.pair_count > m ? t.pair_count : m; return (int)m; }
    int maxLiveExpertsPerTile() const { uint32_t m = 0; for (const auto &t : tiles) m = t.group_count > m ? t.group_count : m; return (int)m; }
};

struct PrefillMoEGrouping {
    static PrefillMoEGroupedRoutes groupTokenExpertPairs(const std::vector<PrefillTokenExpertPair> &pairs, int queryCount, int topK,
                                                         int numExperts, int tileExpertCount = 16,
                                                         const std::vector<uint64_t> *expertSortKeys = nullptr) {
        PrefillMoEGroupedRoutes r;
        r.queryCount = queryCount;
        const size_t ne = numExperts > 0 ? (size_t)numExperts : 1;
        r.sortedPairs.resize(pairs.size());
        r.perExpertOffsets.resize(ne);
        r.perExpertCounts.resize(ne);
        r.groups.resize(pairs.size() < ne ? pairs.size() + 1 : ne);
        r.tiles.resize(r.groups.size());
        uint32_t ng = 0, nt = 0;
        const int32_t rc = tf_prefill_group_token_expert_pairs(
            pairs.data(), pairs.size(), queryCount, topK, numExperts, tileExpertCount, expertSortKeys ? expertSortKeys->data() : nullptr,
            expertSortKeys ? expertSortKeys->size() : 0, r.sortedPairs.data(), r.perExpertOffsets.data(), r.perExpertCounts.data(),
            r.groups.data(), &ng, r.tiles.data(), &nt);
        if (rc != TF_OK) throw Error(rc, "PrefillMoEGroupingError " + std::to_string(rc));
        r.groups.resize(ng);
        r.tiles.resize(nt);
        if (numExperts > 0) { r.perExpertOffsets.resize((size_t)numExperts); r.perExpertCounts.resize((size_t)numExperts); }
        return r;
    }
};

using PrefillGroupedRoutedMoEStreamedParams = tf_prefill_streamed_params;   // PrefillGroupedRoutedMoE.swift:104-183

// PrefillGroupedRoutedMoE (Kernels/Prefill/MoE/PrefillGroupedRoutedMoE.swift:338-463)
class PrefillGroupedRoutedMoE {
public:
    explicit PrefillGroupedRoutedMoE(const Context &context) : c_(context) {}
    // returns the micro-batch count, like the Swift method
    int encodeStreamedBatched(const void *hidden, uint64_t hiddenOffset, const void *sortedPairs, uint64_t sortedPairsOffset,
                              void *routePartials, uint64_t routePartialsOffset, void *gateUpActScratch, uint64_t gateUpActScratchOffset,
                              void *downScratch, uint64_t downScratchOffset, const std::vector<const void *> &bindingViews,
                              const PrefillGroupedRoutedMoEStreamedParams &params, const PrefillMoEGroup *tileGroups,
                              uint32_t tileGroupCount, int pairMicrobatchRows = 32) const {
        int32_t microbatches = 0;
        if (params.live_expert_count != bindingViews.size()) return 0;   // the Swift guard (:401-403)
        c_.check(tf_prefill_grouped_routed_moe_streamed(c_.raw(), c_.stream(), hidden, hiddenOffset, sortedPairs, sortedPairsOffset,
                                                        routePartials, routePartialsOffset, gateUpActScratch, gateUpActScratchOffset,
                                                        downScratch, downScratchOffset, bindingViews.data(), &params, tileGroups,
                                                        tileGroupCount, pairMicrobatchRows, &microbatches, TF_BF16));
        return microbatches;
    }

private:
    const Context &c_;
};

// PrefillMoE (Kernels/Prefill/MoE/PrefillMoE.swift)
class PrefillMoE {
public:
    explicit PrefillMoE(const Context &context) : c_(context) {}
    void encodeReduceTokenMajor(const void *routePartials, uint64_t routePartialsOffset, const void *routeWeights,
                                uint64_t routeWeightsOffset, void *h2, uint64_t h2Offset, uint32_t queryCount, uint32_t topK,
                                uint32_t d) const {
        c_.check(tf_prefill_moe_reduce_token_major(c_.raw(), c_.stream(), routePartials, routePartialsOffset, routeWeights,
                                                   routeWeightsOffset, h2, h2Offset, queryCount, topK, d));
    }

private:
    const Context &c_;
};


// FusedPostAttentionSetup (Kernels/Fusions/FusedPostAttentionSetup.swift)
class FusedPostAttentionSetup {
public:
    explicit FusedPostAttentionSetup(const Context &context) : c_(context) {}
    void encode(void *hidden, const void *attn, void *denseX, void *routedX, void *routerX, const void *postAttentionWeight,
                uint64_t postAttentionWeightOffset, const void *preFFNWeight, uint64_t preFFNWeightOffset, const void *preFFN2Weight,
                uint64_t preFFN2WeightOffset, uint32_t d, float eps) const {
        c_.check(tf_fused_post_attn_setup(c_.raw(), c_.stream(), hidden, attn, denseX, routedX, routerX, postAttentionWeight,
                                          postAttentionWeightOffset, preFFNWeight, preFFNWeightOffset, preFFN2Weight, preFFN2WeightOffset,
                                          d, eps));
    }

private:
    const Context &c_;
};

// FusedLayerTail (Kernels/Fusions/FusedLayerTail.swift)
class FusedLayerTail {
public:
    explicit FusedLayerTail(const Context &context) : c_(context) {}
    void encode(const void *h2, const void *h1, void *hidden, const void *postFFN2Weight, uint64_t postFFN2WeightOffset,
                const void *postFFNWeight, uint64_t postFFNWeightOffset, uint32_t d, float eps, float layerScalar) const {
        c_.check(tf_fused_layer_tail(c_.raw(), c_.stream(), h2, h1, hidden, postFFN2Weight, postFFN2WeightOffset, postFFNWeight,
                                     postFFNWeightOffset, d, eps, layerScalar));
    }

private:
    const Context &c_;
};

// PrefillPostAttentionSetup (Kernels/Prefill/Epilogues/PrefillPostAttentionSetup.swift)
class PrefillPostAttentionSetup {
public:
    explicit PrefillPostAttentionSetup(const Context &context) : c_(context) {}
    void encode(void *hidden, uint64_t hiddenOffset, const void *attn, uint64_t attnOffset, void *denseX, uint64_t denseXOffset,
                void *routedX, uint64_t routedXOffset, void *routerX, uint64_t routerXOffset, const void *postAttentionWeight,
                uint64_t postAttentionWeightOffset, const void *preFFNWeight, uint64_t preFFNWeightOffset, const void *preFFN2Weight,
                uint64_t preFFN2WeightOffset, uint32_t queryCount, uint32_t d, uint32_t hiddenStrideElements,
                uint32_t attnStrideElements, uint32_t denseStrideElements, uint32_t routedStrideElements,
                uint32_t routerStrideElements, float eps) const {
        c_.check(tf_prefill_post_attn_setup_block(c_.raw(), c_.stream(), hidden, hiddenOffset, attn, attnOffset, denseX, denseXOffset,
                                                  routedX, routedXOffset, routerX, routerXOffset, postAttentionWeight,
                                                  postAttentionWeightOffset, preFFNWeight, preFFNWeightOffset, preFFN2Weight,
                                                  preFFN2WeightOffset, queryCount, d, hiddenStrideElements, attnStrideElements,
                                                  denseStrideElements, routedStrideElements, routerStrideElements, eps));
    }

private:
    const Context &c_;
};

// PrefillLayerTail (Kernels/Prefill/Epilogues/PrefillLayerTail.swift)
class PrefillLayerTail {
public:
    explicit PrefillLayerTail(const Context &context) : c_(context) {}
    void encode(const void *h2, uint64_t h2Offset, const void *h1, uint64_t h1Offset, void *hidden, uint64_t hiddenOffset,
                const void *postFFN2Weight, uint64_t postFFN2WeightOffset, const void *postFFNWeight, uint64_t postFFNWeightOffset,
                uint32_t queryCount, uint32_t d, uint32_t h2StrideElements, uint32_t h1StrideElements, uint32_t hiddenStrideElements,
                float eps, float layerScalar) const {
        c_.check(tf_prefill_layer_tail_block(c_.raw(), c_.stream(), h2, h2Offset, h1, h1Offset, hidden, hiddenOffset, postFFN2Weight,
                                             postFFN2WeightOffset, postFFNWeight, postFFNWeightOffset, queryCount, d, h2StrideElements,
                                             h1StrideElements, hiddenStrideElements, eps, layerScalar));
    }

private:
    const Context &c_;
};


// EmbedLookupInt4 (Kernels/Quant/EmbedLookupInt4.swift); tableRows bounds the token (see tf_embed_lookup_int4)
class EmbedLookupInt4 {
public:
    explicit EmbedLookupInt4(const Context &context) : c_(context) {}
    void encode(const void *table, uint64_t tableOffset, const void *scales, uint64_t scalesOffset, const void *biases,
                uint64_t biasesOffset, void *out, uint64_t outOffset, uint32_t tokenId, uint32_t d, float outScale,
                uint32_t tableRows) const {
        c_.check(tf_embed_lookup_int4(c_.raw(), c_.stream(), table, tableOffset, scales, scalesOffset, biases, biasesOffset, out, outOffset,
                                      tokenId, d, outScale, tableRows));
    }

private:
    const Context &c_;
};

// PrefillEmbedLookupInt4 (Kernels/Prefill/Primitives/PrefillPrimitives.swift:4-39)
class PrefillEmbedLookupInt4 {
public:
    explicit PrefillEmbedLookupInt4(const Context &context) : c_(context) {}
    void encode(const void *table, uint64_t tableOffset, const void *scales, uint64_t scalesOffset, const void *biases,
                uint64_t biasesOffset, const void *tokens, uint64_t tokensOffset, void *out, uint64_t outOffset, uint32_t t, uint32_t d,
                float outScale, uint32_t tableRows) const {
        c_.check(tf_prefill_embed_lookup_int4_block(c_.raw(), c_.stream(), table, tableOffset, scales, scalesOffset, biases, biasesOffset,
                                                    tokens, tokensOffset, out, outOffset, t, d, outScale, tableRows));
    }

private:
    const Context &c_;
};

// LogitSoftcapSoftmax, Sample, SampleTopK64 (Kernels/Sampling/LogitOutput.swift)
class LogitSoftcapSoftmax {
public:
    explicit LogitSoftcapSoftmax(const Context &context) : c_(context) {}
    void encode(const void *logits, void *probs, uint32_t v, float softcap = 30.0f) const {
        c_.check(tf_logit_softcap_softmax(c_.raw(), c_.stream(), logits, probs, v, softcap, TF_FP16));
    }

private:
    const Context &c_;
};

class Sample {
public:
    explicit Sample(const Context &context) : c_(context) {}
    void encode(const void *probs, void *outToken, uint32_t v, float temperature, uint32_t topK, float topP, uint64_t seed,
                uint32_t position = 0) const {
        c_.check(tf_sample(c_.raw(), c_.stream(), probs, outToken, v, temperature, topK, topP, seed, position));
    }

private:
    const Context &c_;
};

class SampleTopK64 {
public:
    SampleTopK64(const Context &context, uint32_t vocab) : c_(context), vocab_(vocab) {
        if (vocab == 0 || vocab > 262144) throw Error(TF_ERR_INVALID_ARGUMENT, "unsupportedVocabulary");
    }
    void encode(const void *probs, void *outToken, float temperature, float topP, uint64_t seed) const {
        c_.check(tf_sample_topk64(c_.raw(), c_.stream(), probs, outToken, vocab_, temperature, topP, seed));
    }

private:
    const Context &c_;
    uint32_t vocab_;
};


// FusedQKVGEMV (Kernels/Fusions/FusedQKVGEMV.swift)
class FusedQKVGEMV {
public:
    explicit FusedQKVGEMV(const Context &context) : c_(context) {}
    void encode(const void *qWeights, uint64_t qWeightsOffset, const void *qScales, uint64_t qScalesOffset, const void *qBiases,
                uint64_t qBiasesOffset, const void *kWeights, uint64_t kWeightsOffset, const void *kScales, uint64_t kScalesOffset,
                const void *kBiases, uint64_t kBiasesOffset, const void *vWeights, uint64_t vWeightsOffset, const void *vScales,
                uint64_t vScalesOffset, const void *vBiases, uint64_t vBiasesOffset, const void *x, void *qOut, uint64_t qOutOffset,
                void *kOut, uint64_t kOutOffset, void *vOut, uint64_t vOutOffset, uint32_t qRows, uint32_t kvRows, uint32_t n) const {
        c_.check(tf_fused_qkv_gemv(c_.raw(), c_.stream(), qWeights, qWeightsOffset, qScales, qScalesOffset, qBiases, qBiasesOffset, kWeights,
                                   kWeightsOffset, kScales, kScalesOffset, kBiases, kBiasesOffset, vWeights, vWeightsOffset, vScales,
                                   vScalesOffset, vBiases, vBiasesOffset, x, qOut, qOutOffset, kOut, kOutOffset, vOut, vOutOffset, qRows, kvRows,
                                   n, TF_BF16));
    }

private:
    const Context &c_;
};

// MPPPrefillInt4QMM (Kernels/TensorCore/MPPPrefillInt4QMM.swift)
class MPPPrefillInt4QMM {
public:
    enum class Path { affineThreadgroupF16, unavailable };
    static constexpr int tileK = TF_GROUP_SIZE;
    explicit MPPPrefillInt4QMM(const Context &context) : c_(context) {}
    bool isAvailable() const { return true; }
    Path encode(const void *weights, uint64_t weightsOffset, const void *scales, uint64_t scalesOffset, const void *biases,
                uint64_t biasesOffset, const void *x, uint64_t xOffset, void *y, uint64_t yOffset, int m, int n, int k) const {
        const int32_t rc = tf_int4_qmm(c_.raw(), c_.stream(), weights, weightsOffset, scales, scalesOffset, biases, biasesOffset, x, xOffset,
                                       y, yOffset, m, n, k, TF_BF16);
        if (rc == TF_ERR_UNAVAILABLE) return Path::unavailable;
        c_.check(rc);
        return Path::affineThreadgroupF16;
    }

private:
    const Context &c_;
};

}  // namespace tf

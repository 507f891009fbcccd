"""The BASELINE configurations at their full sizes on the GPU, through the C ABI:
config 2 (lm_head 262144 x 2816: persistent tiles, refills, the 64 argmax cells and the ticket all in play),
config 3 (a few tokens over the 128-expert pool) and config 4 (2048 tokens x 128 experts, Zipf routing, matrix cores).
Planted rows follow LMHeadChainInt4Tests.swift:136-193; the prefill checks follow PrefillGroupedRoutedMoETests+Execution."""
import ctypes as C

import numpy as np
import pytest
import torch

import refcases
from gpu_helpers import ctx, dev, host, tfk, within_north_star, zeros_bytes
from oracle import tfo
from test_gpu_prefill import device_grouping

pytestmark = pytest.mark.gpu
D, F, E, TOPK, V = 2816, 704, 128, 8, 262144


# ------------------------------------------------------------------------------------------------ config 2
@pytest.fixture(scope="module")
def head():
    rng = np.random.default_rng(0x1E4D)
    W = rng.integers(0, 256, (V, D // 2), dtype=np.uint8)
    s = rng.uniform(0.005, 0.02, (V, D // 64)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, (V, D // 64)).astype(np.float32)
    hidden = refcases.normal_f16(D, 0x1E4D)
    norm = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, D).astype(np.float32))
    return dict(W=W, s=s, b=b, hidden=hidden, norm=norm)


def for_device(bits_bf16, kind):
    """The oracle reads bf16 scales.  Every bf16 value in fp16's range is also an fp16 value, so the fp16 run gets the same
    numbers in the other encoding and one reference serves both."""
    if kind == tfk.TF_BF16:
        return bits_bf16
    return tfo.bf16_array_to_float(bits_bf16.ravel()).astype(np.float16).view(np.uint16).reshape(bits_bf16.shape)


def plant(W, S, B, rows, x_bits):
    """Rows that beat every random row by construction: weight 15 where the activation is positive, 0 elsewhere, the
    largest scale, no bias.  Returns copies; the originals stay random."""
    W, S, B = W.copy(), S.copy(), B.copy()
    nib = np.where(tfo.from_f16_bits(x_bits) > 0, 15, 0).astype(np.uint8)
    packed = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8)
    for r in rows:
        W[r], S[r], B[r] = packed, tfo.bf16_bits(0.02), tfo.bf16_bits(0.0)
    return W, S, B


def gpu_head(head, dW, S, B, kind, logits=False):
    k = ctx()
    dh, dn, dS, dB = dev(head["hidden"]), dev(head["norm"]), dev(for_device(S, kind)), dev(for_device(B, kind))
    tok = zeros_bytes(4, 0xEE)
    k.lm_head_greedy(dh, dn, dW, dS, dB, tok, D, V, scale_dtype=kind)
    out = None
    if logits:
        out = zeros_bytes(V * 4)
        k.check(k.lib.tf_lm_head_logits_int4(k.handle, None, dh.data_ptr(), 0, dn.data_ptr(), 0, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0,
                                             out.data_ptr(), 0, D, V, 1e-6, kind, tfk.TF_FP32))
        out = host(out, np.float32, V)
    return int(host(tok, np.uint32, 1)[0]), out


@pytest.mark.parametrize("kind", [tfk.TF_BF16, tfk.TF_FP16], ids=["bf16", "fp16"])
def test_lm_head_full_vocabulary(head, kind):
    W = head["W"]
    S, B = tfo.bf16_bits_array(head["s"]).reshape(head["s"].shape), tfo.bf16_bits_array(head["b"]).reshape(head["b"].shape)

    def cpu(Wc, Sc, Bc, **kw):
        return tfo.lm_head_cpu_greedy(head["hidden"], head["norm"], Wc, Sc, Bc, threads=8, **kw)

    # random rows: the token and every fp32 logit
    tok_ref, logits_ref = cpu(W, S, B, want_logits=True)
    tok, logits = gpu_head(head, dev(W), S, B, kind, logits=True)
    assert tok == tok_ref
    assert tfo.rel_error(logits, logits_ref) < tfo.Tolerance.fp16Reduction
    assert within_north_star(logits, logits_ref)
    assert int(np.argmax(logits)) == tok_ref
    # two identical winners far apart, an odd and an even row (different places in their tiles): the lower index
    Wp, Sp, Bp = plant(W, S, B, [17, 262000], head["hidden"])
    dWp = dev(Wp)
    assert cpu(Wp, Sp, Bp) == 17
    assert gpu_head(head, dWp, Sp, Bp, kind)[0] == 17
    # the first of the pair produces a non-finite logit (one of its scales is +inf): skipped, the far one wins
    Sn = Sp.copy()
    Sn[17, 3] = 0x7F80
    assert cpu(Wp, Sn, Bp) == 262000
    assert gpu_head(head, dWp, Sn, Bp, kind)[0] == 262000
    del dWp
    # a single winner three rows before the end
    Wt, St, Bt = plant(W, S, B, [V - 3], head["hidden"])
    assert cpu(Wt, St, Bt) == V - 3
    assert gpu_head(head, dev(Wt), St, Bt, kind)[0] == V - 3


# ------------------------------------------------------------------------------------------------ configs 3 and 4
@pytest.fixture(scope="module")
def pool():
    """The 128-expert pool of the production shape, one blob per expert in the reference's order."""
    blobs, off = [], None
    for e in range(E):
        blob, off = tfo.make_blob(refcases.synthetic_int4(F, D, 0x9001 + e, "g"), refcases.synthetic_int4(F, D, 0x9001 + e, "u"),
                                  refcases.synthetic_int4(D, F, 0x9001 + e, "d"))
        blobs.append(blob)
    stride = (blobs[0].size + 16383) // 16384 * 16384
    pool_np = np.zeros((E, stride), np.uint8)
    for e, b in enumerate(blobs):
        pool_np[e, :b.size] = b
    return dict(blobs=blobs, off=off, stride=stride, flat=pool_np.ravel(), dev=dev(pool_np))


SENTINEL = 0xD630


def run_block(pool, hidden, idx, w_bits):
    """device grouping -> grouped experts over the resident pool -> token-major reduce."""
    T = hidden.shape[0]
    k = ctx()
    g = device_grouping(idx, w_bits, T, TOPK, E)
    n = T * TOPK
    acts = zeros_bytes(n * F * 2)
    partials = torch.full((n * D,), SENTINEL, dtype=torch.int16, device="cuda").view(torch.uint8) if SENTINEL < 0x8000 else \
        torch.full((n * D,), SENTINEL - 0x10000, dtype=torch.int16, device="cuda").view(torch.uint8)
    h2 = zeros_bytes(T * D * 2)
    koff = tfk.ExpertOffsets(*pool["off"].as_tuple())
    d_hidden, d_w = dev(hidden), dev(np.ascontiguousarray(w_bits, np.uint16))
    k.check(k.lib.tf_prefill_grouped_routed_moe_resident(k.handle, None, d_hidden.data_ptr(), 0, D, g["sorted_pairs"].data_ptr(),
                                                         g["chunks"].data_ptr(), g["n_chunks"].data_ptr(), g["cap"], n, pool["dev"].data_ptr(),
                                                         pool["stride"], E, C.byref(koff), acts.data_ptr(), partials.data_ptr(), D, F, TOPK, tfk.TF_BF16))
    k.check(k.lib.tf_prefill_moe_reduce_token_major(k.handle, None, partials.data_ptr(), 0, d_w.data_ptr(), 0, h2.data_ptr(), 0, T, TOPK, D))
    sp = host(g["sorted_pairs"], np.uint32, n * 4).reshape(n, 4)
    return dict(sorted_pairs=np.array([tuple(r) for r in sp], tfo.PAIR_DTYPE), partials=host(partials, np.uint16, n * D).reshape(T, TOPK, D),
                h2=tfo.from_f16_bits(host(h2, np.uint16, T * D)).reshape(T, D), counts=host(g["counts"], np.uint32, E),
                n_chunks=int(host(g["n_chunks"], np.uint32, 1)[0]))


def oracle_rows(pool, hidden, w_bits, r, tokens):
    """partials and h2 of the listed tokens from the oracle (the pairs of those tokens only)."""
    T = hidden.shape[0]
    sp = r["sorted_pairs"]
    pairs = sp[np.isin(sp["token"], tokens)]
    want = tfo.prefill_route_partials(pairs, T, hidden.ravel(), D, pool["flat"], pool["stride"], pool["off"], TOPK, D, F, fill_bits=0,
                                      threads=8).reshape(T, TOPK, D)
    h2 = tfo.from_f16_bits(tfo.prefill_reduce_token_major(want.ravel(), np.ascontiguousarray(w_bits, np.uint16).ravel(), T, TOPK, D)).reshape(T, D)
    return want, h2


def decode_rows(pool, hidden, idx, w_bits):
    """Every token through the batch-1 kernels (phase 1 + phase 2 with the token's own experts)."""
    T = hidden.shape[0]
    k = ctx()
    koff = tfk.ExpertOffsets(*pool["off"].as_tuple())
    d_idx, d_x, d_w = dev(np.ascontiguousarray(idx, np.uint32)), dev(hidden), dev(np.ascontiguousarray(w_bits, np.uint16))
    res, acts, y = zeros_bytes(D * 2), zeros_bytes(TOPK * F * 2), zeros_bytes(T * D * 2)
    for t in range(T):
        routed = tfk.RoutedBlobs()
        routed.pool, routed.pool_stride, routed.indices, routed.num_experts = pool["dev"].data_ptr(), pool["stride"], d_idx.data_ptr() + t * TOPK * 4, E
        k.check(k.lib.tf_moe_phase1_gate_up_act(k.handle, None, C.byref(routed), C.byref(koff), d_x.data_ptr() + t * D * 2, acts.data_ptr(), D, F, TOPK,
                                                tfk.TF_BF16))
        k.check(k.lib.tf_moe_phase2_down_reduce(k.handle, None, C.byref(routed), C.byref(koff), acts.data_ptr(), d_w.data_ptr() + t * TOPK * 2,
                                                res.data_ptr(), y.data_ptr() + t * D * 2, D, F, TOPK, tfk.TF_BF16))
    return tfo.from_f16_bits(host(y, np.uint16, T * D)).reshape(T, D)


def zipf_block(T):
    """configs[4]'s routing: 8 distinct experts per token drawn with Zipf(1.1) popularity, seeded."""
    rng = np.random.default_rng(0xC0F4)
    p = 1.0 / np.arange(1, E + 1) ** 1.1
    p /= p.sum()
    idx = np.stack([rng.choice(E, size=TOPK, replace=False, p=p) for _ in range(T)]).astype(np.uint32)
    w_bits = tfo.to_f16_bits(rng.dirichlet(np.ones(TOPK), T).astype(np.float32)).reshape(T, TOPK)
    hidden = rng.standard_normal((T, D)).astype(np.float16).view(np.uint16)
    return idx, w_bits, hidden


def test_prefill_2048_tokens_over_128_experts(pool):
    T = 2048
    idx, w_bits, hidden = zipf_block(T)
    r = run_block(pool, hidden, idx, w_bits)
    counts = r["counts"]
    assert counts.sum() == T * TOPK and counts.max() > 4 * 128 and r["n_chunks"] > E       # several full 128-pair chunks of one expert
    # every route row was written
    assert not np.any(np.all(r["partials"] == SENTINEL, axis=2))
    # oracle on tokens of the most popular expert (first, middle and last chunk of its group), of the rarest expert, and a few more
    sp = r["sorted_pairs"]
    hot, rare = int(np.argmax(counts)), int(np.argmin(np.where(counts > 0, counts, 1 << 30)))
    hot_tokens = sp["token"][sp["expert"] == hot]
    pick = np.unique(np.concatenate([hot_tokens[:6], hot_tokens[len(hot_tokens) // 2 - 3:len(hot_tokens) // 2 + 3], hot_tokens[-6:],
                                     sp["token"][sp["expert"] == rare][:4], [0, T - 1]])).astype(np.uint32)
    want_p, want_h2 = oracle_rows(pool, hidden, w_bits, r, pick)
    scale = float(np.max(np.abs(tfo.from_f16_bits(want_p[pick]))))
    for t in pick:
        assert within_north_star(tfo.from_f16_bits(r["partials"][t]), tfo.from_f16_bits(want_p[t]), abs_=2e-3 * max(1.0, scale)), t
        assert within_north_star(r["h2"][t], want_h2[t], abs_=2e-3 * max(1.0, scale)), t
    # every token of the block against the batch-1 kernels on that token
    dec = decode_rows(pool, hidden, idx, w_bits)
    err = np.max(np.abs(dec - r["h2"]), axis=1)
    bound = 4e-3 * np.maximum(1.0, np.max(np.abs(dec), axis=1))
    assert np.all(err <= bound), (int(np.argmax(err - bound)), float(np.max(err - bound)))
    # and the batch-1 kernels against the all-fp32 reference on three of the sampled tokens
    for t in pick[:3]:
        ref = tfo.moe_apply_streamed_routed([pool["blobs"][int(e)] for e in idx[t]], pool["off"], tfo.from_f16_bits(hidden[t]), np.zeros(D, np.float32),
                                            tfo.from_f16_bits(w_bits[t]), D, F, threads=8)
        assert tfo.rel_error(r["h2"][t], ref) < tfo.Tolerance.fp16ChainedReduction


@pytest.mark.parametrize("M", [2, 4, 8, 16])
def test_few_tokens_over_the_128_expert_pool(pool, M):
    rng = np.random.default_rng(0x3300 + M)
    logits = rng.standard_normal((M, E))                     # seeded random router logits: experts are shared across tokens
    idx = np.argsort(-logits, axis=1, kind="stable")[:, :TOPK].astype(np.uint32)
    top = np.take_along_axis(logits, idx.astype(np.int64), axis=1)
    prob = np.exp(top - top.max(axis=1, keepdims=True))
    w_bits = tfo.to_f16_bits((prob / prob.sum(axis=1, keepdims=True)).astype(np.float32)).reshape(M, TOPK)
    hidden = rng.standard_normal((M, D)).astype(np.float16).view(np.uint16)
    r = run_block(pool, hidden, idx, w_bits)
    assert not np.any(np.all(r["partials"] == SENTINEL, axis=2))
    want_p, want_h2 = oracle_rows(pool, hidden, w_bits, r, np.arange(M, dtype=np.uint32))
    scale = float(np.max(np.abs(tfo.from_f16_bits(want_p))))
    assert within_north_star(tfo.from_f16_bits(r["partials"]), tfo.from_f16_bits(want_p), abs_=1e-3 * max(1.0, scale))
    assert within_north_star(r["h2"], want_h2, abs_=1e-3 * max(1.0, scale))
    dec = decode_rows(pool, hidden, idx, w_bits)
    assert np.max(np.abs(dec - r["h2"])) <= 4e-3 * max(1.0, float(np.max(np.abs(dec))))


def few_tokens_inputs(M, seed, copy_of=None):
    """Router operands of the production shape and M token rows; copy_of: {row: source row} duplicates (tokens that share all eight experts)."""
    rng = np.random.default_rng(seed)
    W, S, B = refcases.synthetic_int8(E, D, seed)
    router_x = np.stack([refcases.normal_f16(D, seed * 64 + r) for r in range(M)])
    routed_x = rng.standard_normal((M, D)).astype(np.float16).view(np.uint16)
    for row, src in (copy_of or {}).items():
        router_x[row] = router_x[src]
    eff = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, D).astype(np.float32) / np.float32(np.sqrt(D)))
    pes = tfo.bf16_bits_array(rng.uniform(0.6, 1.4, E).astype(np.float32))
    return W, S, B, router_x, routed_x, eff, pes


def run_few_tokens(pool, W, S, B, router_x, routed_x, eff, pes, expect=tfk.TF_OK):
    M = router_x.shape[0]
    k = ctx()
    n = M * TOPK
    koff = tfk.ExpertOffsets(*pool["off"].as_tuple())
    keep = [dev(a) for a in (W, S, B, router_x, eff, pes, routed_x)]
    dW, dS, dB, dh, de, dp, dx = keep
    idx, wts = zeros_bytes(n * 4, 0xEE), zeros_bytes(n * 2, 0xEE)
    acts = zeros_bytes(n * F * 2)
    partials = torch.full((n * D,), SENTINEL - 0x10000, dtype=torch.int16, device="cuda").view(torch.uint8)
    h2 = torch.full((M * D,), SENTINEL - 0x10000, dtype=torch.int16, device="cuda").view(torch.uint8)
    rc = k.lib.tf_prefill_routed_moe_few_tokens(k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dh.data_ptr(), 0, de.data_ptr(), 0,
                                                dp.data_ptr(), 0, idx.data_ptr(), 0, wts.data_ptr(), 0, M, E, D, TOPK, D, dx.data_ptr(), 0, D,
                                                pool["dev"].data_ptr(), pool["stride"], C.byref(koff), acts.data_ptr(), partials.data_ptr(),
                                                h2.data_ptr(), 0, F, tfk.TF_BF16)
    assert rc == expect, k.last_error()
    k.synchronize()
    return dict(idx=host(idx, np.uint32, n).reshape(M, TOPK), w_bits=host(wts, np.uint16, n).reshape(M, TOPK),
                partials=host(partials, np.uint16, n * D).reshape(M, TOPK, D), h2_bits=host(h2, np.uint16, M * D).reshape(M, D))


def pairs_of(idx, w_bits):
    """token-major pairs of a routing (every pair of a token, in rank order): the layout the oracle's grouped path takes"""
    M = idx.shape[0]
    pairs = np.zeros(M * TOPK, tfo.PAIR_DTYPE)
    pairs["token"] = np.repeat(np.arange(M, dtype=np.uint32), TOPK)
    pairs["rank"] = np.tile(np.arange(TOPK, dtype=np.uint32), M)
    pairs["expert"] = np.minimum(idx.ravel(), E - 1)
    pairs["weight_bits"] = w_bits.ravel().astype(np.uint32)
    return pairs


@pytest.mark.parametrize("M,copy_of", [(1, None), (2, None), (2, {1: 0}), (3, {2: 0}), (4, None), (5, {1: 0, 3: 0, 4: 0}), (8, {5: 1, 7: 1}), (16, None),
                                       (32, {31: 0})])
def test_few_tokens_in_one_call_of_three_launches(pool, M, copy_of):
    # tf_prefill_routed_moe_few_tokens against the calls it replaces (router block + grouping, grouped experts over the resident
    # pool, token-major reduce) and against the oracle, production shape, 128 experts.  Rows copied from another row choose that
    # row's eight experts: the owner of an expert then serves several tokens (and a first pair several followers in the down launch).
    # Up to five rows run the three launches of their own; more rows are the three calls made inside (bit-identical to them).
    W, S, B, router_x, routed_x, eff, pes = few_tokens_inputs(M, 0x7E0 + M, copy_of)
    got = run_few_tokens(pool, W, S, B, router_x, routed_x, eff, pes)
    assert not np.any(np.all(got["partials"] == SENTINEL, axis=2))
    assert not np.any(np.all(got["h2_bits"] == SENTINEL, axis=1))
    # the router's outputs: the block router's (its logits are summed in another order: same experts away from near ties, weights to fp16 rounding)
    k = ctx()
    keep = [dev(a) for a in (W, S, B, router_x, eff, pes)]
    idx2, wts2 = zeros_bytes(M * TOPK * 4), zeros_bytes(M * TOPK * 2)
    k.check(k.lib.tf_prefill_router_gemma4_block(k.handle, None, keep[0].data_ptr(), 0, keep[1].data_ptr(), 0, keep[2].data_ptr(), 0, keep[3].data_ptr(), 0,
                                                 keep[4].data_ptr(), 0, keep[5].data_ptr(), 0, idx2.data_ptr(), 0, wts2.data_ptr(), 0, M, E, D, TOPK, D))
    ref_idx = host(idx2, np.uint32, M * TOPK).reshape(M, TOPK)
    ref_w = tfo.from_f16_bits(host(wts2, np.uint16, M * TOPK)).reshape(M, TOPK)
    assert np.array_equal(got["idx"], ref_idx)
    assert np.max(np.abs(tfo.from_f16_bits(got["w_bits"]) - ref_w)) <= 2e-3
    for row, src in (copy_of or {}).items():
        assert np.array_equal(got["idx"][row], got["idx"][src])
    if M >= 8 or copy_of:
        assert len(np.unique(got["idx"])) < M * TOPK          # experts are shared between tokens
    # the grouped path on the same routing
    r = run_block(pool, routed_x, got["idx"], got["w_bits"])
    scale = float(np.max(np.abs(tfo.from_f16_bits(r["partials"]))))
    assert within_north_star(tfo.from_f16_bits(got["partials"]), tfo.from_f16_bits(r["partials"]), abs_=1e-3 * max(1.0, scale))
    assert within_north_star(tfo.from_f16_bits(got["h2_bits"]), r["h2"], abs_=1e-3 * max(1.0, scale))
    # the reduce is exact given the partials: fused multiply-adds in rank order
    want_h2 = tfo.prefill_reduce_token_major(got["partials"].ravel(), got["w_bits"].ravel(), M, TOPK, D).reshape(M, D)
    assert np.array_equal(got["h2_bits"], want_h2)
    # the oracle, every pair (up to 16 tokens) or the pairs of four tokens
    tokens = np.arange(M, dtype=np.uint32) if M <= 16 else np.array([0, 1, M // 2, M - 1], np.uint32)
    pairs = pairs_of(got["idx"], got["w_bits"])
    pairs = pairs[np.isin(pairs["token"], tokens)]
    want = tfo.prefill_route_partials(pairs, M, routed_x.ravel(), D, pool["flat"], pool["stride"], pool["off"], TOPK, D, F, fill_bits=0,
                                      threads=8).reshape(M, TOPK, D)
    assert within_north_star(tfo.from_f16_bits(got["partials"][tokens]), tfo.from_f16_bits(want[tokens]), abs_=1e-3 * max(1.0, scale))


def test_few_tokens_in_one_call_when_a_token_has_fewer_than_eight_finite_logits(pool):
    # 123 of the 128 router rows carry a NaN scale: every token has five finite logits, the selection fills ranks 5..7 with
    # expert 0 at weight zero (the reference's rule for unfilled places), and nothing is shared between blocks.  Every pair's
    # partial result is still that pair's expert applied to its token.
    M = 4
    W, S, B, router_x, routed_x, eff, pes = few_tokens_inputs(M, 0x7F5)
    S = S.copy()
    live = [3, 17, 64, 90, 127]
    for e in range(E):
        if e not in live:
            S.reshape(E, -1)[e, :] = 0x7FC0
    got = run_few_tokens(pool, W, S, B, router_x, routed_x, eff, pes)
    for t in range(M):
        assert sorted(got["idx"][t][:5]) == live and list(got["idx"][t][5:]) == [0, 0, 0]
        assert list(got["w_bits"][t][5:]) == [0, 0, 0]
    pairs = pairs_of(got["idx"], got["w_bits"])
    want = tfo.prefill_route_partials(pairs, M, routed_x.ravel(), D, pool["flat"], pool["stride"], pool["off"], TOPK, D, F, fill_bits=0,
                                      threads=8).reshape(M, TOPK, D)
    scale = float(np.max(np.abs(tfo.from_f16_bits(want))))
    assert within_north_star(tfo.from_f16_bits(got["partials"]), tfo.from_f16_bits(want), abs_=1e-3 * max(1.0, scale))
    want_h2 = tfo.prefill_reduce_token_major(got["partials"].ravel(), got["w_bits"].ravel(), M, TOPK, D).reshape(M, D)
    assert np.array_equal(got["h2_bits"], want_h2)


def test_few_tokens_in_one_call_back_to_back_and_replayed_from_a_graph(pool):
    # Calls of different sizes in a row on one stream without a host wait (the context's logits scratch and the outputs pass
    # from launch to launch through device memory), then the same calls captured into a graph on a side stream and replayed three
    # times with an eager call between the replays: every output bit for bit what the call gives when it runs alone.
    sizes = [3, 1, 4, 2]
    k = ctx()
    koff = tfk.ExpertOffsets(*pool["off"].as_tuple())
    cases = []
    for i, M in enumerate(sizes):
        W, S, B, router_x, routed_x, eff, pes = few_tokens_inputs(M, 0x7A00 + i, {M - 1: 0} if M > 1 else None)
        alone = run_few_tokens(pool, W, S, B, router_x, routed_x, eff, pes)
        cases.append(dict(M=M, alone=alone, ins=[dev(a) for a in (W, S, B, router_x, eff, pes, routed_x)]))

    def outputs(M):
        n = M * TOPK
        return dict(idx=zeros_bytes(n * 4, 0xEE), wts=zeros_bytes(n * 2, 0xEE), acts=zeros_bytes(n * F * 2), partials=zeros_bytes(n * D * 2, 0xEE),
                    h2=zeros_bytes(M * D * 2, 0xEE))

    def call(c, o, stream):
        dW, dS, dB, dh, de, dp, dx = c["ins"]
        k.check(k.lib.tf_prefill_routed_moe_few_tokens(k.handle, stream, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dh.data_ptr(), 0,
                                                       de.data_ptr(), 0, dp.data_ptr(), 0, o["idx"].data_ptr(), 0, o["wts"].data_ptr(), 0, c["M"], E, D, TOPK,
                                                       D, dx.data_ptr(), 0, D, pool["dev"].data_ptr(), pool["stride"], C.byref(koff), o["acts"].data_ptr(),
                                                       o["partials"].data_ptr(), o["h2"].data_ptr(), 0, F, tfk.TF_BF16))

    def check(c, o, what):
        M, a = c["M"], c["alone"]
        n = M * TOPK
        assert np.array_equal(host(o["idx"], np.uint32, n).reshape(M, TOPK), a["idx"]), what
        assert np.array_equal(host(o["wts"], np.uint16, n).reshape(M, TOPK), a["w_bits"]), what
        assert np.array_equal(host(o["partials"], np.uint16, n * D).reshape(M, TOPK, D), a["partials"]), what
        assert np.array_equal(host(o["h2"], np.uint16, M * D).reshape(M, D), a["h2_bits"]), what

    outs = [outputs(c["M"]) for c in cases]
    for c, o in zip(cases, outs):
        call(c, o, None)
    k.synchronize()
    for i, (c, o) in enumerate(zip(cases, outs)):
        check(c, o, ("in a row", i))
    side = torch.cuda.Stream()
    gouts = [outputs(c["M"]) for c in cases]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for c, o in zip(cases, gouts):
                call(c, o, side.cuda_stream)
    for replay in range(3):
        for o in gouts:
            for name in ("idx", "wts", "partials", "h2"):
                o[name].fill_(0xEE)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for i, (c, o) in enumerate(zip(cases, gouts)):
            check(c, o, ("replay", replay, i))
        o = outputs(cases[replay]["M"])               # an eager call between the replays
        call(cases[replay], o, None)
        k.synchronize()
        check(cases[replay], o, ("eager after replay", replay))


def test_few_tokens_in_one_call_refuses_what_it_does_not_serve(pool):
    W, S, B, router_x, routed_x, eff, pes = few_tokens_inputs(33, 0x7F9)
    got = run_few_tokens(pool, W, S, B, router_x, routed_x, eff, pes, expect=tfk.TF_ERR_UNAVAILABLE)
    assert np.all(got["idx"] == 0xEEEEEEEE) and np.all(got["h2_bits"] == SENTINEL)       # nothing was enqueued


# ------------------------------------------------------------------------------------------------ config 4, second half
F_SHARED = 2112


def test_prefill_2048_tokens_routed_and_shared_expert_in_one_call(pool):
    # configs[4] in full: the routed experts "plus a shared-expert int4 FFN applied to all tokens".  The call the benchmark's
    # 2048-token figure is measured on (tf_prefill_grouped_routed_moe_resident_shared: the shared expert's dense tiles ahead of
    # the routed tiles in the same two launches) against the two calls it replaces, at 2048 tokens x 128 experts x production
    # widths: every route partial and every shared output bit for bit, no row of either left unwritten, padding untouched; the
    # shared expert's block entry alone at 2048 rows against the oracle (PrefillSharedExpertTests.swift:89,177,243 checks the
    # block against its rows; SharedExpertInt4Tests.swift:52 gives the 6e-3 against the CPU reference).
    T, y_stride = 2048, D + 8
    idx, w_bits, hidden = zipf_block(T)
    k = ctx()
    n = T * TOPK
    g = device_grouping(idx, w_bits, T, TOPK, E)
    koff = tfk.ExpertOffsets(*pool["off"].as_tuple())
    d_hidden = dev(hidden)
    mats = [refcases.synthetic_int4(F_SHARED, D, 0xA77, "g"), refcases.synthetic_int4(F_SHARED, D, 0xA77, "u"), refcases.synthetic_int4(D, F_SHARED, 0xA77, "d")]
    tens = [[dev(a) for a in m] for m in mats]
    gate, up, down = tfk.projection(*tens[0], F_SHARED, D), tfk.projection(*tens[1], F_SHARED, D), tfk.projection(*tens[2], D, F_SHARED)
    scratch = [zeros_bytes(F_SHARED * 2) for _ in range(3)]
    y_sentinel = int(np.float16(-7.25).view(np.uint16))

    def run(one_call):
        acts = zeros_bytes(n * F * 2)
        partials = torch.full((n * D,), SENTINEL - 0x10000, dtype=torch.int16, device="cuda").view(torch.uint8)
        y = dev(np.full((T, y_stride), y_sentinel, np.uint16))
        routed = (k.handle, None, d_hidden.data_ptr(), 0, D, g["sorted_pairs"].data_ptr(), g["chunks"].data_ptr(), g["n_chunks"].data_ptr(),
                  g["cap"], n, pool["dev"].data_ptr(), pool["stride"], E, C.byref(koff), acts.data_ptr(), partials.data_ptr(), D, F, TOPK, tfk.TF_BF16)
        shared_a = (d_hidden.data_ptr(), 0, y.data_ptr(), 0, C.byref(gate), C.byref(up), C.byref(down))
        shared_s = tuple(v for s_ in scratch for v in (s_.data_ptr(), 0, F_SHARED * 2))
        if one_call:
            k.check(k.lib.tf_prefill_grouped_routed_moe_resident_shared(*routed, *shared_a, *shared_s, T, F_SHARED, D, y_stride, 4))
        else:
            k.check(k.lib.tf_prefill_grouped_routed_moe_resident(*routed))
            k.check(k.lib.tf_prefill_shared_expert_int4_block(k.handle, None, *shared_a, *shared_s, T, D, F_SHARED, D, y_stride, 4, tfk.TF_BF16))
        return host(partials, np.uint16, n * D).reshape(T, TOPK, D), host(y, np.uint16, T * y_stride).reshape(T, y_stride)

    two_p, two_y = run(False)
    one_p, one_y = run(True)
    assert np.array_equal(one_p, two_p)
    assert np.array_equal(one_y, two_y)
    for p_, y_ in ((two_p, two_y), (one_p, one_y)):
        assert not np.any(np.all(p_ == SENTINEL, axis=2))                    # every route row written
        assert not np.any(np.all(y_[:, :D] == y_sentinel, axis=1))           # every shared row written
        assert np.all(y_[:, D:] == y_sentinel)                               # padding between rows untouched
    # the shared expert at 2048 rows against the oracle: the first and last row of the block, both sides of the 128-row tile
    # boundaries, and a seeded sample
    rows = sorted({0, 1, 127, 128, 129, 1023, 1024, 2046, 2047} | set(np.random.default_rng(0x5A4E).integers(0, T, 8).tolist()))
    for r in rows:
        ref = tfo.shared_expert_ref(mats[0], mats[1], mats[2], tfo.from_f16_bits(hidden[r]), threads=8)
        got = tfo.from_f16_bits(one_y[r, :D])
        assert tfo.rel_error(got, ref) < 6e-3, r
        assert within_north_star(got, ref, abs_=1e-3 * max(1.0, float(np.max(np.abs(ref))))), r
    # and the routed half of the merged call is the one the test above checks against the oracle: same grouping, same partials
    # as the two-call path it already covers (bit equality above), so one sampled token against the oracle suffices here
    sp = host(g["sorted_pairs"], np.uint32, n * 4).reshape(n, 4)
    r_ = dict(sorted_pairs=np.array([tuple(v) for v in sp], tfo.PAIR_DTYPE))
    pick = np.array([0, T - 1], np.uint32)
    want_p, _ = oracle_rows(pool, hidden, w_bits, r_, pick)
    scale = float(np.max(np.abs(tfo.from_f16_bits(want_p[pick]))))
    for tkn in pick:
        assert within_north_star(tfo.from_f16_bits(one_p[tkn]), tfo.from_f16_bits(want_p[tkn]), abs_=2e-3 * max(1.0, scale)), tkn

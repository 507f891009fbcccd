"""GPU parity of the prefill / multi-token path through the C ABI: per-token router, device grouping, grouped routed experts
(reference-shaped streamed tile and resident pool; row-streaming and matrix-core variants), token-major reduce, int4 QMM.
Cases restate PrefillRouterTests, PrefillGroupedRoutedMoETests+Execution, PrefillMoETests, MPPPrefillInt4QMMTests."""
import ctypes as C

import numpy as np
import pytest
import torch

import refcases
from gpu_helpers import device_view, ctx, dev, host, tfk, within_north_star, zeros_bytes
from oracle import tfo

pytestmark = pytest.mark.gpu


def prefill_router(W, S, B, hidden_bits, stride, eff_bits, pes_bits, rows, top_k=8, hidden_off=0):
    e, d = W.shape
    k = ctx()
    hid = dev(hidden_bits, hidden_off)
    before = host(hid, np.uint8).copy()
    idx, wts = zeros_bytes(rows * top_k * 4), zeros_bytes(rows * top_k * 2)
    dW, dS, dB, dE, dP = dev(W), dev(S), dev(B), dev(eff_bits), dev(pes_bits)   # keep the tensors alive across the call
    k.check(k.lib.tf_prefill_router_gemma4_block(k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0,
                                                 hid.data_ptr(), hidden_off, dE.data_ptr(), 0, dP.data_ptr(), 0,
                                                 idx.data_ptr(), 0, wts.data_ptr(), 0, rows, e, d, top_k, stride))
    torch.cuda.synchronize()
    assert np.array_equal(host(hid, np.uint8), before), "router wrote into the hidden block"
    return host(idx, np.uint32, rows * top_k).reshape(rows, top_k), tfo.from_f16_bits(host(wts, np.uint16, rows * top_k)).reshape(rows, top_k)


def decode_router(W, S, B, hidden_bits, eff_bits, pes_bits):
    e, d = W.shape
    idx, wts = zeros_bytes(32), zeros_bytes(16)
    ctx().router_gemma4(dev(W), dev(S), dev(B), dev(hidden_bits), dev(eff_bits), dev(pes_bits), idx, wts, e, d)
    return host(idx, np.uint32, 8), tfo.from_f16_bits(host(wts, np.uint16, 8))


@pytest.mark.parametrize("stride_pad,hidden_off", [(13, 0), (16, 0), (0, 32)])
def test_block_router_matches_repeated_scalar_rows(stride_pad, hidden_off):
    # PrefillRouterTests.swift:33-103
    experts, d, rows = 16, 128, 3
    rng = tfo.SplitMix64(0x9A7E2026)
    weights = np.stack([rng.uniform_array(-0.04, 0.04, d) + np.float32(e) * np.float32(0.015) for e in range(experts)])
    stride = d + stride_pad
    hidden = np.full(rows * stride, tfo.f16_bits(-31.0), np.uint16)
    for r in range(rows):
        hidden[r * stride:r * stride + d] = tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, d))
    eff = tfo.bf16_bits_array(rng.uniform_array(0.5, 1.5, d) / np.sqrt(np.float32(d)))
    pes = tfo.bf16_bits_array(rng.uniform_array(0.6, 1.4, experts))
    W, S, B = tfo.quantize_int8(weights)
    got_idx, got_w = prefill_router(W, S, B, hidden, stride, eff, pes, rows, hidden_off=hidden_off)
    for r in range(rows):
        row_bits = hidden[r * stride:r * stride + d]
        d_idx, d_w = decode_router(W, S, B, row_bits, eff, pes)
        assert list(got_idx[r]) == list(d_idx)
        assert np.max(np.abs(got_w[r] - d_w)) <= 5e-3
        ref_idx, ref_w, _ = tfo.router_reference(W, S, B, tfo.from_f16_bits(row_bits), tfo.bf16_array_to_float(eff), tfo.bf16_array_to_float(pes))
        assert list(got_idx[r]) == list(ref_idx) and np.max(np.abs(got_w[r] - ref_w)) <= 5e-3


def test_block_router_near_tie_and_generic_topk():
    # PrefillRouterTests.swift:105-146: same near-tie winner as the scalar path
    experts, d = 16, 128
    gains = [1.0 - e * 0.05 for e in range(7)] + [0.5, 0.5 * (1 + 1e-4)] + [0.4 - (e - 9) * 0.02 for e in range(9, 16)]
    pattern = (np.float32(0.25) + ((np.arange(d) * 37 + 11) % 97).astype(np.float32) / np.float32(97.0))
    weights = np.array(gains, np.float32)[:, None] * pattern[None, :]
    W, S, B = tfo.quantize_int8(weights.astype(np.float32))
    hid = tfo.to_f16_bits(np.ones(d, np.float32))
    eff, pes = tfo.bf16_bits_array(np.ones(d, np.float32)), tfo.bf16_bits_array(np.ones(experts, np.float32))
    got_idx, _ = prefill_router(W, S, B, hid, d, eff, pes, 1)
    assert list(got_idx[0]) == list(decode_router(W, S, B, hid, eff, pes)[0]) == [0, 1, 2, 3, 4, 5, 6, 8]
    # generic top_k (PrefillRouter.swift:62: 1...64): top-3 is the prefix of top-8, weights are a softmax over three
    idx3, w3 = prefill_router(W, S, B, hid, d, eff, pes, 1, top_k=3)
    assert list(idx3[0]) == [0, 1, 2] and abs(float(w3.sum()) - 1.0) < 2e-3
    k = ctx()
    z = zeros_bytes(64)
    bad = k.lib.tf_prefill_router_gemma4_block(k.handle, None, z.data_ptr(), 0, z.data_ptr(), 0, z.data_ptr(), 0, z.data_ptr(), 0, z.data_ptr(), 0,
                                               z.data_ptr(), 0, z.data_ptr(), 0, z.data_ptr(), 0, 1, 16, 128, 65, 128)
    assert bad == tfk.TF_ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("rows,experts,d", [(200, 128, 2816), (97, 48, 704), (65, 128, 128)])
def test_block_router_many_tokens_on_matrix_cores(rows, experts, d):
    # more than 64 tokens take the matrix-core projection: same logits (to 1e-4) and, away from near ties, the same
    # experts in the same order as the reference's scalar arithmetic
    rng = np.random.default_rng(rows * 7 + experts)
    W, S, B = refcases.synthetic_int8(experts, d, 0xB10C + rows)
    hidden = np.concatenate([refcases.normal_f16(d, 0x500 + r) for r in range(rows)])
    eff_f = rng.uniform(0.5, 1.5, d).astype(np.float32) / np.float32(np.sqrt(d))
    pes_f = rng.uniform(0.6, 1.4, experts).astype(np.float32)
    eff, pes = tfo.bf16_bits_array(eff_f), tfo.bf16_bits_array(pes_f)
    got_idx, got_w = prefill_router(W, S, B, hidden, d, eff, pes, rows)
    logits = device_view(ctx().lib.tf_prefill_router_logits(ctx().handle), rows * experts, "<f4").reshape(rows, experts)
    pinned = 0
    for r in range(rows):
        ref_idx, ref_w, ref_logits = tfo.router_reference(W, S, B, tfo.from_f16_bits(hidden[r * d:(r + 1) * d]), tfo.bf16_array_to_float(eff),
                                                          tfo.bf16_array_to_float(pes))
        assert tfo.rel_error(logits[r], ref_logits) < 1e-4
        srt = np.sort(ref_logits)[::-1]
        if np.min(srt[:8] - srt[1:9]) > 1e-4 * np.max(np.abs(srt)):
            pinned += 1
            assert list(got_idx[r]) == list(ref_idx)
            assert np.max(np.abs(got_w[r] - ref_w)) < 5e-3
    assert pinned > rows // 2


def device_grouping(idx, wts_bits, T, top_k, E):
    k = ctx()
    n = T * top_k
    cap = E + n // 64 + 1
    sp, offs, cnts = zeros_bytes(n * 16), zeros_bytes(E * 4), zeros_bytes(E * 4)
    chunks, nch = zeros_bytes(cap * 12), zeros_bytes(4)
    d_idx, d_w = dev(np.ascontiguousarray(idx, np.uint32)), dev(np.ascontiguousarray(wts_bits, np.uint16))
    k.check(k.lib.tf_prefill_group_pairs_device(k.handle, None, d_idx.data_ptr(), d_w.data_ptr(), T, top_k, E, sp.data_ptr(),
                                                offs.data_ptr(), cnts.data_ptr(), chunks.data_ptr(), nch.data_ptr()))
    return dict(sorted_pairs=sp, offsets=offs, counts=cnts, chunks=chunks, n_chunks=nch, cap=cap, keep=(d_idx, d_w))


# one 256-thread block up to 32 tokens, three launches over up to 64 token segments beyond (ragged last batches, an odd top-k,
# more tokens than 64 segments of 32, the largest expert count)
@pytest.mark.parametrize("T,top_k,E", [(4, 3, 6), (32, 8, 128), (33, 8, 128), (100, 5, 7), (300, 8, 128), (2048, 8, 128), (2049, 8, 200),
                                       (4096, 8, 128), (4100, 8, 256), (16, 8, 16)])
def test_device_grouping_equals_host_grouping(T, top_k, E):
    rng = np.random.default_rng(T + E)
    p = 1.0 / np.arange(1, E + 1) ** 1.1
    p /= p.sum()
    idx = np.stack([rng.choice(E, size=top_k, replace=False, p=p) for _ in range(T)]).astype(np.uint32)
    w = rng.integers(1, 0x3C00, (T, top_k)).astype(np.uint16)
    g = device_grouping(idx, w, T, top_k, E)
    pairs = tfk.make_token_expert_pairs(idx.ravel(), w.ravel(), T, top_k)
    ref = tfk.group_token_expert_pairs([(q.token, q.expert, q.rank, q.weight_bits_and_reserved) for q in pairs[:T * top_k]], T, top_k, E)
    got = host(g["sorted_pairs"], np.uint32, T * top_k * 4).reshape(-1, 4)
    assert [tuple(int(v) for v in r) for r in got] == ref["sorted_pairs"]
    assert list(host(g["offsets"], np.uint32, E)) == ref["per_expert_offsets"]
    assert list(host(g["counts"], np.uint32, E)) == ref["per_expert_counts"]
    nch = int(host(g["n_chunks"], np.uint32, 1)[0])
    chunks = host(g["chunks"], np.uint32, nch * 3).reshape(nch, 3)
    covered = []
    for e, s, c in chunks:
        assert 1 <= c <= 128 and all(int(x) == int(e) for x in got[s:s + c, 1])
        covered.extend(range(int(s), int(s + c)))
    assert covered == list(range(T * top_k)) and nch <= g["cap"]


@pytest.mark.parametrize("T,E,d,top_k", [(1, 128, 2816, 8), (2, 128, 2816, 8), (16, 128, 2816, 8), (32, 128, 2816, 8), (31, 200, 704, 8), (7, 16, 128, 3),
                                         (33, 128, 2816, 8), (12, 64, 256, 12)])
def test_router_block_and_grouping_in_one_call_equal_the_two_calls(T, E, d, top_k):
    # tf_prefill_router_group_block = tf_prefill_router_gemma4_block + tf_prefill_group_pairs_device, every output of both bit
    # for bit: up to 32 tokens (and top-k <= 8) the selection and the grouping share one launch; 33 tokens and a top-12 are
    # forwarded to the two calls.  The two calls are the ones the oracle and the host grouping check above.
    rng = np.random.default_rng(T * 31 + E)
    W, S, B = refcases.synthetic_int8(E, d, 0x6A0 + T)
    hidden = np.concatenate([refcases.normal_f16(d, 0x700 + r) for r in range(T)])
    eff = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, d).astype(np.float32) / np.float32(np.sqrt(d)))
    pes = tfo.bf16_bits_array(rng.uniform(0.6, 1.4, E).astype(np.float32))
    k = ctx()
    dW, dS, dB, dh, de, dp = dev(W), dev(S), dev(B), dev(hidden), dev(eff), dev(pes)
    n = T * top_k
    cap = E + n // 64 + 1

    def outputs():
        return dict(idx=zeros_bytes(n * 4, 0xEE), wts=zeros_bytes(n * 2, 0xEE), sp=zeros_bytes(n * 16, 0xEE), offs=zeros_bytes(E * 4, 0xEE),
                    cnts=zeros_bytes(E * 4, 0xEE), chunks=zeros_bytes(cap * 12, 0xEE), nch=zeros_bytes(4, 0xEE))

    router = (k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dh.data_ptr(), 0, de.data_ptr(), 0, dp.data_ptr(), 0)
    two, one = outputs(), outputs()
    k.check(k.lib.tf_prefill_router_gemma4_block(*router, two["idx"].data_ptr(), 0, two["wts"].data_ptr(), 0, T, E, d, top_k, d))
    k.check(k.lib.tf_prefill_group_pairs_device(k.handle, None, two["idx"].data_ptr(), two["wts"].data_ptr(), T, top_k, E, two["sp"].data_ptr(),
                                                two["offs"].data_ptr(), two["cnts"].data_ptr(), two["chunks"].data_ptr(), two["nch"].data_ptr()))
    k.check(k.lib.tf_prefill_router_group_block(*router, one["idx"].data_ptr(), 0, one["wts"].data_ptr(), 0, T, E, d, top_k, d, one["sp"].data_ptr(),
                                                one["offs"].data_ptr(), one["cnts"].data_ptr(), one["chunks"].data_ptr(), one["nch"].data_ptr()))
    nch = int(host(two["nch"], np.uint32, 1)[0])
    assert 1 <= nch <= cap and nch == int(host(one["nch"], np.uint32, 1)[0])
    for name, count in (("idx", n * 4), ("wts", n * 2), ("sp", n * 16), ("offs", E * 4), ("cnts", E * 4), ("chunks", nch * 12)):
        assert np.array_equal(host(one[name], np.uint8, count), host(two[name], np.uint8, count)), name
    # every token's experts are the reference router's
    got = host(one["idx"], np.uint32, n).reshape(T, top_k)
    if top_k == 8:
        for r in (0, T - 1):
            ref_idx, _, _ = tfo.router_reference(W, S, B, tfo.from_f16_bits(hidden[r * d:(r + 1) * d]), tfo.bf16_array_to_float(eff),
                                                 tfo.bf16_array_to_float(pes))
            assert list(got[r]) == list(ref_idx)
    # a refused call launches nothing
    bad = outputs()
    rc = k.lib.tf_prefill_router_group_block(*router, bad["idx"].data_ptr(), 0, bad["wts"].data_ptr(), 0, T, E, d, 65, d, bad["sp"].data_ptr(),
                                             bad["offs"].data_ptr(), bad["cnts"].data_ptr(), bad["chunks"].data_ptr(), bad["nch"].data_ptr())
    assert rc == tfk.TF_ERR_INVALID_ARGUMENT
    rc = k.lib.tf_prefill_router_group_block(*router, bad["idx"].data_ptr(), 0, bad["wts"].data_ptr(), 0, T, E, d, top_k, d, bad["sp"].data_ptr(),
                                             bad["offs"].data_ptr(), None, bad["chunks"].data_ptr(), bad["nch"].data_ptr())
    assert rc == tfk.TF_ERR_INVALID_ARGUMENT
    k.synchronize()
    assert all(np.all(host(bad[name], np.uint8) == 0xEE) for name in bad)


def test_router_block_and_grouping_in_one_call_with_equal_logits():
    # Three router rows are byte-for-byte the same: a token that picks one of them has three equal scores among its best eight.
    # Ties go to the lower index in both forms of the call, and the one-launch form equals the two calls bit for bit.
    T, E, d, top_k = 16, 128, 2816, 8
    rng = np.random.default_rng(0x71E5)
    W, S, B = refcases.synthetic_int8(E, d, 0x71E)
    W, S, B = W.copy(), S.copy(), B.copy()
    for dup in (40, 77):
        W[dup], S[dup], B[dup] = W[3], S[3], B[3]
    hidden = np.concatenate([refcases.normal_f16(d, 0x7100 + r) for r in range(T)])
    eff = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, d).astype(np.float32) / np.float32(np.sqrt(d)))
    pes = tfo.bf16_bits_array(rng.uniform(0.6, 1.4, E).astype(np.float32))
    k = ctx()
    dW, dS, dB, dh, de, dp = dev(W), dev(S), dev(B), dev(hidden), dev(eff), dev(pes)
    n = T * top_k
    cap = E + n // 64 + 1
    outs = [dict(idx=zeros_bytes(n * 4, 0xEE), wts=zeros_bytes(n * 2, 0xEE), sp=zeros_bytes(n * 16, 0xEE), offs=zeros_bytes(E * 4, 0xEE),
                 cnts=zeros_bytes(E * 4, 0xEE), chunks=zeros_bytes(cap * 12, 0xEE), nch=zeros_bytes(4, 0xEE)) for _ in range(2)]
    two, one = outs
    router = (k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dh.data_ptr(), 0, de.data_ptr(), 0, dp.data_ptr(), 0)
    k.check(k.lib.tf_prefill_router_gemma4_block(*router, two["idx"].data_ptr(), 0, two["wts"].data_ptr(), 0, T, E, d, top_k, d))
    k.check(k.lib.tf_prefill_group_pairs_device(k.handle, None, two["idx"].data_ptr(), two["wts"].data_ptr(), T, top_k, E, two["sp"].data_ptr(),
                                                two["offs"].data_ptr(), two["cnts"].data_ptr(), two["chunks"].data_ptr(), two["nch"].data_ptr()))
    k.check(k.lib.tf_prefill_router_group_block(*router, one["idx"].data_ptr(), 0, one["wts"].data_ptr(), 0, T, E, d, top_k, d, one["sp"].data_ptr(),
                                                one["offs"].data_ptr(), one["cnts"].data_ptr(), one["chunks"].data_ptr(), one["nch"].data_ptr()))
    idx = host(two["idx"], np.uint32, n).reshape(T, top_k)
    tied = [t_ for t_ in range(T) if {3, 40, 77} <= set(idx[t_].tolist())]
    assert len(tied) >= 1, "no token picked the three equal rows: the case tests nothing"
    for t_ in tied:      # ties go to the lower index, in this order
        pos = [list(idx[t_]).index(e) for e in (3, 40, 77)]
        assert pos == sorted(pos) and pos[2] - pos[0] == 2
    nch = int(host(two["nch"], np.uint32, 1)[0])
    for name, count in (("idx", n * 4), ("wts", n * 2), ("sp", n * 16), ("offs", E * 4), ("cnts", E * 4), ("chunks", nch * 12)):
        assert np.array_equal(host(one[name], np.uint8, count), host(two[name], np.uint8, count)), name


def test_streamed_batched_matches_reference_across_partial_microbatch():
    # PrefillGroupedRoutedMoETests+Execution.swift:8-103
    d = f = 64
    rows, top_k = 3, 2
    rank_w = lambda r: tfo.f16_bits(0.125 + r * 0.0625)
    raw = [(0, 2, 0), (0, 0, 1), (1, 1, 0), (1, 2, 1), (2, 0, 0), (2, 1, 1)]
    routes = tfk.group_token_expert_pairs([(t, e, r, rank_w(r)) for t, e, r in raw], rows, top_k, 16, 16)
    pool, off, stride = refcases.synthetic_expert_pool(16, d, f)
    hidden = tfo.to_f16_bits(((np.arange(rows * d) % 17) - 8).astype(np.float32) * np.float32(0.01))
    sp_np = np.array(routes["sorted_pairs"], np.uint32)
    expected = tfo.prefill_route_partials(np.array([tuple(r) for r in sp_np], tfo.PAIR_DTYPE), rows, hidden, d, pool, stride, off,
                                          top_k, d, f, fill_bits=tfo.f16_bits(-77.0))
    k = ctx()
    # every expert lives in its own allocation at a non-zero offset (64 + 16 * index), as in the reference test
    blob_t, ptrs = [], (C.c_void_p * 16)()
    for i in range(16):
        prefix = 64 + i * 16
        t = dev(pool[i * stride:(i + 1) * stride], prefix)
        blob_t.append(t)
        ptrs[i] = t.data_ptr() + prefix
    params = tfk.StreamedParams()
    params.pair_start, params.pair_count, params.d, params.routed_intermediate = 0, len(raw), d, f
    params.top_k, params.hidden_stride_elements, params.live_expert_count = top_k, d, 16
    for i in range(16):
        params.local_expert[i] = i
    for name, v in zip([n for n, _ in tfo.ExpertOffsets._fields_], off.as_tuple()):
        setattr(params, name, v)
    groups = (tfk.PrefillGroup * len(routes["groups"]))(*[tfk.PrefillGroup(*g) for g in routes["groups"]])
    out = dev(np.full(rows * top_k * d, tfo.f16_bits(-77.0), np.uint16))
    scratch_act, scratch_down = zeros_bytes(3 * 4 * f * 2), zeros_bytes(4 * d * 2)
    nmb = C.c_int32(0)
    d_hidden, d_sp = dev(hidden), dev(sp_np)
    rc = k.lib.tf_prefill_grouped_routed_moe_streamed(k.handle, None, d_hidden.data_ptr(), 0, d_sp.data_ptr(), 0, out.data_ptr(), 0,
                                                      scratch_act.data_ptr(), 0, scratch_down.data_ptr(), 0, C.cast(ptrs, C.c_void_p), C.byref(params),
                                                      C.cast(groups, C.c_void_p), len(routes["groups"]), 4, C.byref(nmb), tfk.TF_BF16)
    assert rc == tfk.TF_OK, k.last_error()
    got = tfo.from_f16_bits(host(out, np.uint16, rows * top_k * d))
    assert nmb.value == 2
    assert np.max(np.abs(got - tfo.from_f16_bits(expected))) <= 0.0015
    del blob_t


def scales_as_fp16(blob, off, d, f):
    """The same expert with its bf16 scales and biases rewritten as fp16 of the same value (a bf16 value inside fp16's normal
    range converts exactly; the rare bias below it becomes zero)."""
    out = blob.copy()
    for name, count in (("gate_s_off", f * d // 64), ("gate_b_off", f * d // 64), ("up_s_off", f * d // 64), ("up_b_off", f * d // 64),
                        ("down_s_off", d * f // 64), ("down_b_off", d * f // 64)):
        at = getattr(off, name)
        bf = out[at:at + 2 * count].view(np.uint16)
        val = (bf.astype(np.uint32) << 16).view(np.float32)
        h = val.astype(np.float16)
        h[h.astype(np.float32) != val] = 0
        out[at:at + 2 * count] = h.view(np.uint8)
    return out


def bf16_pool_matching(blob_fp16, off, d, f):
    """Inverse of scales_as_fp16 for a blob whose fp16 scales all came from bf16 values."""
    out = blob_fp16.copy()
    for name, count in (("gate_s_off", f * d // 64), ("gate_b_off", f * d // 64), ("up_s_off", f * d // 64), ("up_b_off", f * d // 64),
                        ("down_s_off", d * f // 64), ("down_b_off", d * f // 64)):
        at = getattr(off, name)
        val = out[at:at + 2 * count].view(np.float16).astype(np.float32)
        out[at:at + 2 * count] = (val.view(np.uint32) >> 16).astype(np.uint16).view(np.uint8)
    return out


def resident_pipeline(T, E, d, f, top_k, seed, zipf=False, from_router=True, fp16_scales=False):
    """router block -> device grouping -> grouped experts (resident pool) -> token-major reduce; returns everything needed to check."""
    rng = np.random.default_rng(seed)
    blobs, off = [], None
    for e in range(E):
        blob, off = tfo.make_blob(refcases.synthetic_int4(f, d, seed + e, "g"), refcases.synthetic_int4(f, d, seed + e, "u"),
                                  refcases.synthetic_int4(d, f, seed + e, "d"))
        blobs.append(blob)
    if fp16_scales:
        blobs = [scales_as_fp16(b, off, d, f) for b in blobs]
    stride = (blobs[0].size + 255) // 256 * 256
    pool_np = np.zeros((E, stride), np.uint8)
    for e, b in enumerate(blobs):
        pool_np[e, :b.size] = b
    hidden = rng.standard_normal((T, d)).astype(np.float16).view(np.uint16)
    k = ctx()
    if from_router:
        rW, rS, rB = refcases.synthetic_int8(E, d, seed)
        eff = tfo.bf16_bits_array((rng.uniform(0.5, 1.5, d) / np.sqrt(d)).astype(np.float32))
        pes = tfo.bf16_bits_array(rng.uniform(0.6, 1.4, E).astype(np.float32))
        idx, w = prefill_router(rW, rS, rB, hidden.ravel(), d, eff, pes, T, top_k=top_k)
        w_bits = tfo.to_f16_bits(w)
    else:
        p = 1.0 / np.arange(1, E + 1) ** 1.1
        p /= p.sum()
        idx = np.stack([rng.choice(E, size=top_k, replace=False, p=p if zipf else None) for _ in range(T)]).astype(np.uint32)
        w_bits = tfo.to_f16_bits(rng.dirichlet(np.ones(top_k), T).astype(np.float32))
    g = device_grouping(idx, w_bits, T, top_k, E)
    n = T * top_k
    acts, partials, h2 = zeros_bytes(n * f * 2), zeros_bytes(n * d * 2), zeros_bytes(T * d * 2)
    koff = tfk.ExpertOffsets(*off.as_tuple())
    d_pool, d_hidden, d_w = dev(pool_np), dev(hidden), dev(np.ascontiguousarray(w_bits, np.uint16))
    k.check(k.lib.tf_prefill_grouped_routed_moe_resident(k.handle, None, d_hidden.data_ptr(), 0, d, g["sorted_pairs"].data_ptr(),
                                                         g["chunks"].data_ptr(), g["n_chunks"].data_ptr(), g["cap"], n, d_pool.data_ptr(),
                                                         stride, E, C.byref(koff), acts.data_ptr(), partials.data_ptr(), d, f, top_k,
                                                         tfk.TF_FP16 if fp16_scales else tfk.TF_BF16))
    k.check(k.lib.tf_prefill_moe_reduce_token_major(k.handle, None, partials.data_ptr(), 0, d_w.data_ptr(), 0, h2.data_ptr(), 0, T, top_k, d))
    sp = host(g["sorted_pairs"], np.uint32, n * 4).reshape(n, 4)
    return dict(blobs=blobs, off=off, pool=pool_np.ravel(), stride=stride, hidden=hidden, idx=np.asarray(idx), w_bits=np.asarray(w_bits).reshape(T, top_k),
                sorted_pairs=np.array([tuple(r) for r in sp], tfo.PAIR_DTYPE), partials=host(partials, np.uint16, n * d),
                h2=tfo.from_f16_bits(host(h2, np.uint16, T * d)).reshape(T, d))


def check_against_oracle(r, T, d, f, top_k, abs_tol, rel_tol=1e-2):
    want_partials = tfo.prefill_route_partials(r["sorted_pairs"], T, r["hidden"].ravel(), d, r["pool"], r["stride"], r["off"], top_k, d, f,
                                               fill_bits=0, threads=8)
    got, want = tfo.from_f16_bits(r["partials"]), tfo.from_f16_bits(want_partials)
    assert within_north_star(got, want, rel=rel_tol, abs_=abs_tol)
    want_h2 = tfo.from_f16_bits(tfo.prefill_reduce_token_major(want_partials, r["w_bits"].ravel(), T, top_k, d)).reshape(T, d)
    assert within_north_star(r["h2"], want_h2, rel=rel_tol, abs_=abs_tol)
    # and against the all-fp32 reference the decode path is judged by (Moe.swift:60-89)
    for t in range(min(T, 3)):
        ref = tfo.moe_apply_streamed_routed([r["blobs"][int(e)] for e in r["idx"][t]], r["off"], tfo.from_f16_bits(r["hidden"][t]),
                                            np.zeros(d, np.float32), tfo.from_f16_bits(r["w_bits"][t]), d, f, threads=8)
        assert tfo.rel_error(r["h2"][t], ref) < tfo.Tolerance.fp16ChainedReduction


@pytest.mark.parametrize("M", [2, 4, 8, 12, 16, 24])
def test_small_m_resident_pipeline_matches_oracle(M):
    # BASELINE config 3: M tokens, top-8 over the production expert shape; below five pairs per expert on average (M = 2, 4,
    # 8, 12, 16 here) the quad kernels serve the call, from there on the matrix-core tiles
    E, d, f, top_k = 32, 2816, 704, 8
    r = resident_pipeline(M, E, d, f, top_k, 0x300 + M)
    scale = float(np.max(np.abs(tfo.from_f16_bits(r["partials"]))))
    check_against_oracle(r, M, d, f, top_k, abs_tol=1e-3 * max(1.0, scale))


def test_small_m_equals_decode_step_per_token():
    # the multi-token pipeline and the batch-1 decode kernels must agree token by token (same arithmetic up to fp16 rounding of partials)
    E, d, f, top_k, M = 16, 2816, 704, 8, 4
    r = resident_pipeline(M, E, d, f, top_k, 0x3AA)
    k = ctx()
    koff = tfk.ExpertOffsets(*r["off"].as_tuple())
    d_pool = dev(r["pool"])
    for t in range(M):
        d_idx, d_x, d_w, d_res = dev(r["idx"][t].astype(np.uint32)), dev(r["hidden"][t]), dev(r["w_bits"][t]), zeros_bytes(d * 2)
        routed = k.routed_from_pool(d_pool, r["stride"], d_idx, E)
        acts, y = zeros_bytes(8 * f * 2), zeros_bytes(d * 2)
        k.moe_phase1(routed, koff, d_x, acts, d, f)
        k.moe_phase2(routed, koff, acts, d_w, d_res, y, d, f)
        dec = tfo.from_f16_bits(host(y, np.uint16, d))
        assert np.max(np.abs(dec - r["h2"][t])) <= 4e-3 * max(1.0, float(np.max(np.abs(dec))))


@pytest.mark.parametrize("T,E,d,f", [(10, 32, 2816, 704), (4, 16, 512, 128), (6, 16, 512, 128), (2, 8, 3072, 1024), (3, 8, 3072, 1024),
                                     (5, 16, 64, 64)])
def test_quad_kernels_long_chunks_and_row_widths(T, E, d, f):
    # Zipf-skewed routing with few pairs per expert on average: some chunks are longer than the quad kernels' LDS image and go
    # through in batches; rows of one pass, of a partly filled last pass and of the widest supported rows
    top_k = 8
    r = resident_pipeline(T, E, d, f, top_k, 0x4400 + T, zipf=True, from_router=False)
    assert np.bincount(r["idx"].ravel(), minlength=E).max() > 8 or T <= 8
    scale = float(np.max(np.abs(tfo.from_f16_bits(r["partials"]))))
    check_against_oracle(r, T, d, f, top_k, abs_tol=1e-3 * max(1.0, scale))


@pytest.mark.parametrize("T,E,d,f,fp16_scales,pad", [(3, 16, 1536, 128, False, 0), (5, 64, 2048, 256, True, 8), (2, 32, 4096, 64, False, 0),
                                                     (7, 128, 2304, 192, True, 24), (4, 12, 2816, 1024, False, 16)])
def test_few_tokens_in_one_call_other_row_widths_and_fp16_scales(T, E, d, f, fp16_scales, pad):
    # tf_prefill_routed_moe_few_tokens away from the production shape: rows that take tiles of four rows in three passes (1536),
    # one row in one or two passes (2048, 4096), two mirrored rows with a partly filled pass (2304, 2816); down rows of 2, 6, 8, 32
    # chunks; 12 to 128 experts; scales as fp16; token rows `pad` halves apart beyond their length (the router's rows and the
    # experts' rows with different strides, both buffers entered at a byte offset).  Routing = the block router's, partials = the
    # oracle's for those pairs, h2 = the reduce of the partials bit for bit.
    top_k, seed = 8, 0x5F00 + T
    rng = np.random.default_rng(seed)
    blobs, off = [], None
    for e in range(E):
        blob, off = tfo.make_blob(refcases.synthetic_int4(f, d, seed + e, "g"), refcases.synthetic_int4(f, d, seed + e, "u"),
                                  refcases.synthetic_int4(d, f, seed + e, "d"))
        blobs.append(blob)
    oracle_blobs = blobs
    if fp16_scales:
        blobs = [scales_as_fp16(b, off, d, f) for b in blobs]
        oracle_blobs = [bf16_pool_matching(b, off, d, f) for b in blobs]
    stride = (blobs[0].size + 255) // 256 * 256
    pool_np, oracle_pool = np.zeros((E, stride), np.uint8), np.zeros((E, stride), np.uint8)
    for e in range(E):
        pool_np[e, :blobs[e].size] = blobs[e]
        oracle_pool[e, :blobs[e].size] = oracle_blobs[e]
    router_x = np.concatenate([refcases.normal_f16(d, seed * 8 + r) for r in range(T)])
    router_x[(T - 1) * d:] = router_x[:d]                     # the last row chooses the first row's experts
    routed_x = rng.standard_normal((T, d)).astype(np.float16).view(np.uint16)
    rW, rS, rB = refcases.synthetic_int8(E, d, seed)
    eff = tfo.bf16_bits_array((rng.uniform(0.5, 1.5, d) / np.sqrt(d)).astype(np.float32))
    pes = tfo.bf16_bits_array(rng.uniform(0.6, 1.4, E).astype(np.float32))
    k = ctx()
    n = T * top_k
    koff = tfk.ExpertOffsets(*off.as_tuple())
    # strided copies of the two activation blocks, filled with a value no row holds
    rs_, xs_, r_off, x_off = d + pad, d + 2 * pad, 32 if pad else 0, 64 if pad else 0
    router_buf = np.full(r_off // 2 + T * rs_, tfo.f16_bits(-31.0), np.uint16)
    routed_buf = np.full(x_off // 2 + T * xs_, tfo.f16_bits(-31.0), np.uint16)
    for r in range(T):
        router_buf[r_off // 2 + r * rs_:r_off // 2 + r * rs_ + d] = router_x[r * d:(r + 1) * d]
        routed_buf[x_off // 2 + r * xs_:x_off // 2 + r * xs_ + d] = routed_x[r]
    dW, dS, dB, dh, de, dp, dx, d_pool = (dev(a) for a in (rW, rS, rB, router_buf, eff, pes, routed_buf, pool_np))
    idx, wts = zeros_bytes(n * 4, 0xEE), zeros_bytes(n * 2, 0xEE)
    acts, partials, h2 = zeros_bytes(n * f * 2), zeros_bytes(n * d * 2, 0xEE), zeros_bytes(T * d * 2, 0xEE)
    k.check(k.lib.tf_prefill_routed_moe_few_tokens(k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dh.data_ptr(), r_off, de.data_ptr(), 0,
                                                   dp.data_ptr(), 0, idx.data_ptr(), 0, wts.data_ptr(), 0, T, E, d, top_k, rs_, dx.data_ptr(), x_off, xs_,
                                                   d_pool.data_ptr(), stride, C.byref(koff), acts.data_ptr(), partials.data_ptr(), h2.data_ptr(), 0, f,
                                                   tfk.TF_FP16 if fp16_scales else tfk.TF_BF16))
    got_idx, got_w = host(idx, np.uint32, n).reshape(T, top_k), host(wts, np.uint16, n).reshape(T, top_k)
    ref_idx, ref_w = prefill_router(rW, rS, rB, router_x, d, eff, pes, T)
    assert np.array_equal(got_idx, ref_idx) and np.array_equal(got_idx[T - 1], got_idx[0])
    assert np.max(np.abs(tfo.from_f16_bits(got_w) - ref_w)) <= 2e-3
    pairs = np.zeros(n, tfo.PAIR_DTYPE)
    pairs["token"], pairs["rank"] = np.repeat(np.arange(T, dtype=np.uint32), top_k), np.tile(np.arange(top_k, dtype=np.uint32), T)
    pairs["expert"], pairs["weight_bits"] = got_idx.ravel(), got_w.ravel().astype(np.uint32)
    want = tfo.prefill_route_partials(pairs, T, routed_x.ravel(), d, oracle_pool.ravel(), stride, off, top_k, d, f, fill_bits=0, threads=8)
    got_p = host(partials, np.uint16, n * d)
    scale = float(np.max(np.abs(tfo.from_f16_bits(want))))
    assert within_north_star(tfo.from_f16_bits(got_p), tfo.from_f16_bits(want), abs_=1e-3 * max(1.0, scale))
    assert np.array_equal(host(h2, np.uint16, T * d), tfo.prefill_reduce_token_major(got_p, got_w.ravel(), T, top_k, d))


@pytest.mark.parametrize("T", [6, 12, 24])
def test_grouped_experts_fp16_scales_equal_bf16_scales(T):
    # the reference's expert blobs carry bf16 scales, and so does the oracle; the fp16 variant of the grouped kernels is pinned
    # on pools whose scales hold the same values in either type: every partial must come out bit-identical (quad kernels at 6
    # and 12 tokens, matrix-core tiles at 24)
    E, d, f, top_k = 32, 2816, 704, 8
    a = resident_pipeline(T, E, d, f, top_k, 0x5500 + T, from_router=False, fp16_scales=True)
    blobs16 = a["blobs"]
    k = ctx()
    pool = np.zeros((E, a["stride"]), np.uint8)
    for e, b in enumerate(blobs16):
        pool[e, :b.size] = bf16_pool_matching(b, a["off"], d, f)
    n = T * top_k
    g = device_grouping(a["idx"], a["w_bits"], T, top_k, E)
    acts, partials = zeros_bytes(n * f * 2), zeros_bytes(n * d * 2)
    koff = tfk.ExpertOffsets(*a["off"].as_tuple())
    d_pool, d_hidden = dev(pool), dev(a["hidden"])
    k.check(k.lib.tf_prefill_grouped_routed_moe_resident(k.handle, None, d_hidden.data_ptr(), 0, d, g["sorted_pairs"].data_ptr(),
                                                         g["chunks"].data_ptr(), g["n_chunks"].data_ptr(), g["cap"], n, d_pool.data_ptr(),
                                                         a["stride"], E, C.byref(koff), acts.data_ptr(), partials.data_ptr(), d, f, top_k, tfk.TF_BF16))
    assert np.array_equal(host(partials, np.uint16, n * d), a["partials"])
    # and the bf16 run itself is the one the oracle checks
    b = dict(a, pool=pool.ravel(), blobs=[pool[e, :blobs16[0].size] for e in range(E)], partials=host(partials, np.uint16, n * d))
    scale = float(np.max(np.abs(tfo.from_f16_bits(b["partials"]))))
    check_against_oracle(b, T, d, f, top_k, abs_tol=2e-3 * max(1.0, scale))


@pytest.mark.parametrize("T,E,d,f,zipf", [(64, 16, 2816, 704, True), (96, 8, 512, 128, False), (200, 16, 256, 192, True)])
def test_grouped_gemm_on_matrix_cores_matches_oracle(T, E, d, f, zipf):
    # BASELINE config 4 in miniature: enough pairs per expert for the MFMA path (pairs >= 8 * experts), Zipf-skewed routing
    top_k = 8
    r = resident_pipeline(T, E, d, f, top_k, 0x400 + T, zipf=zipf, from_router=False)
    scale = float(np.max(np.abs(tfo.from_f16_bits(r["partials"]))))
    check_against_oracle(r, T, d, f, top_k, abs_tol=2e-3 * max(1.0, scale))


@pytest.mark.parametrize("T,E,d,f,shared_f,y_stride,bits", [
    (64, 16, 2816, 704, 2112, 2816, 4),    # production row widths; routed tiles and shared tiles in the same two launches
    (200, 16, 256, 192, 128, 264, 4),      # two row tiles of the shared expert, padded output rows
    (1100, 8, 128, 64, 64, 128, 4),        # nine shared row tiles: the shared tiles numbered by XCD
    (96, 8, 512, 128, 192, 515, 4),        # output rows that cannot leave as 16-byte pieces: the two calls one after the other
    (6, 32, 2816, 704, 2112, 2816, 4),     # quad kernels serve the routed pairs: likewise
    (64, 16, 512, 128, 192, 512, 8),       # 8-bit shared expert: likewise
    (65, 16, 2816, 704, 2112, 2816, -4),   # the first case with the same bits read as fp16 scales and biases (other numbers, the same equality)
])
def test_routed_and_shared_expert_in_one_call_equal_the_two_calls(T, E, d, f, shared_f, y_stride, bits):
    top_k = 8
    sd = tfk.TF_FP16 if bits < 0 else tfk.TF_BF16
    bits = abs(bits)
    r = resident_pipeline(T, E, d, f, top_k, 0x6600 + T, zipf=True, from_router=False)
    k = ctx()
    n = T * top_k
    g = device_grouping(r["idx"], r["w_bits"], T, top_k, E)
    koff = tfk.ExpertOffsets(*r["off"].as_tuple())
    d_pool, d_hidden = dev(r["pool"]), dev(r["hidden"])
    if bits == 4:
        mats = [refcases.synthetic_int4(shared_f, d, 0x77, "g"), refcases.synthetic_int4(shared_f, d, 0x77, "u"), refcases.synthetic_int4(d, shared_f, 0x77, "d")]
    else:
        mats = [refcases.synthetic_int8(shared_f, d, 0x78), refcases.synthetic_int8(shared_f, d, 0x79), refcases.synthetic_int8(d, shared_f, 0x7A)]
    t = [[dev(a) for a in m] for m in mats]
    gate, up, down = tfk.projection(*t[0], shared_f, d), tfk.projection(*t[1], shared_f, d), tfk.projection(*t[2], d, shared_f)
    scratch = [zeros_bytes(shared_f * 2) for _ in range(3)]
    sentinel = np.float16(-7.25).view(np.uint16)

    def run(one_call):
        acts, partials = zeros_bytes(n * f * 2), zeros_bytes(n * d * 2)
        y = dev(np.full((T, y_stride), sentinel, np.uint16))
        routed = (k.handle, None, d_hidden.data_ptr(), 0, d, g["sorted_pairs"].data_ptr(), g["chunks"].data_ptr(), g["n_chunks"].data_ptr(),
                  g["cap"], n, d_pool.data_ptr(), r["stride"], E, C.byref(koff), acts.data_ptr(), partials.data_ptr(), d, f, top_k, sd)
        shared_a = (d_hidden.data_ptr(), 0, y.data_ptr(), 0, C.byref(gate), C.byref(up), C.byref(down))
        shared_s = tuple(v for s_ in scratch for v in (s_.data_ptr(), 0, shared_f * 2))
        if one_call:
            k.check(k.lib.tf_prefill_grouped_routed_moe_resident_shared(*routed, *shared_a, *shared_s, T, shared_f, d, y_stride, bits))
        else:
            k.check(k.lib.tf_prefill_grouped_routed_moe_resident(*routed))
            k.check(k.lib.tf_prefill_shared_expert_int4_block(k.handle, None, *shared_a, *shared_s, T, d, shared_f, d, y_stride, bits, sd))
        return host(partials, np.uint16, n * d), host(y, np.uint16, T * y_stride).reshape(T, y_stride)

    want_partials, want_y = run(False)
    got_partials, got_y = run(True)
    assert np.array_equal(got_partials, want_partials)
    assert np.array_equal(got_y, want_y)
    assert np.all(got_y[:, d:] == sentinel) and not np.any(np.all(got_y[:, :d] == sentinel, axis=1))
    # the separate calls are the ones the oracle checks
    assert sd != tfk.TF_BF16 or np.array_equal(want_partials, r["partials"])
    # a refused shared expert launches nothing, the routed stages included
    acts, partials = zeros_bytes(n * f * 2), zeros_bytes(n * d * 2)
    y = zeros_bytes(T * y_stride * 2)
    rc = k.lib.tf_prefill_grouped_routed_moe_resident_shared(
        k.handle, None, d_hidden.data_ptr(), 0, d, g["sorted_pairs"].data_ptr(), g["chunks"].data_ptr(), g["n_chunks"].data_ptr(), g["cap"], n,
        d_pool.data_ptr(), r["stride"], E, C.byref(koff), acts.data_ptr(), partials.data_ptr(), d, f, top_k, sd, d_hidden.data_ptr(), 0,
        y.data_ptr(), 0, C.byref(gate), C.byref(up), C.byref(gate), *(v for s_ in scratch for v in (s_.data_ptr(), 0, shared_f * 2)), T, shared_f,
        d, y_stride, bits)
    assert rc == tfk.TF_ERR_DIMENSION_MISMATCH
    assert not host(partials, np.uint16, n * d).any()


def test_token_major_reduce_matches_cpu_reference():
    # PrefillMoETests.swift:11-44
    rows, top_k, d = 3, 8, 64
    rng = tfo.SplitMix64(0x4D0E2026)
    partials = tfo.to_f16_bits(rng.uniform_array(-2.0, 2.0, rows * top_k * d))
    weights = tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, rows * top_k))
    h2 = dev(np.full(rows * d, tfo.f16_bits(-19.0), np.uint16))
    k = ctx()
    d_p, d_w = dev(partials), dev(weights)
    k.check(k.lib.tf_prefill_moe_reduce_token_major(k.handle, None, d_p.data_ptr(), 0, d_w.data_ptr(), 0, h2.data_ptr(), 0, rows, top_k, d))
    got = tfo.from_f16_bits(host(h2, np.uint16, rows * d))
    want = tfo.from_f16_bits(tfo.prefill_reduce_token_major(partials, weights, rows, top_k, d))
    assert np.max(np.abs(got - want)) <= 2e-3
    assert k.lib.tf_prefill_moe_reduce_token_major(k.handle, None, h2.data_ptr(), 0, h2.data_ptr(), 0, h2.data_ptr(), 0, 0, 8, 64) == tfk.TF_ERR_INVALID_ARGUMENT


def mpp_inputs(m, n, k, adversarial=False):
    # MPPPrefillInt4QMMTests.swift:19-60
    groups = k // 64
    W = ((np.arange(n * k // 2, dtype=np.uint64) * 37 + 0x29) & 0xFF).astype(np.uint8).reshape(n, k // 2)
    r, g = np.arange(n)[:, None], np.arange(groups)[None, :]
    if adversarial:
        sc = np.array([tfo.bf16_bits(0.001), tfo.bf16_bits(-0.0015), 0x0001, 0x8001], np.uint16)
        bi = np.array([tfo.bf16_bits(-0.01), tfo.bf16_bits(0.006), 0x0001, 0x8001], np.uint16)
        S, B = sc[(r + g) % 4], bi[(r * 3 + g) % 4]
    else:
        S = tfo.bf16_bits_array(np.float32(0.001) + ((r + g) % 5).astype(np.float32) * np.float32(0.00025)).reshape(n, groups)
        B = tfo.bf16_bits_array(np.float32(-0.01) + ((r * 3 + g) % 7).astype(np.float32) * np.float32(0.002)).reshape(n, groups)
    x = tfo.to_f16_bits(((np.arange(m * k) * 11) % 29 - 14).astype(np.float32) / np.float32(64.0))
    return W, np.ascontiguousarray(S), np.ascontiguousarray(B), x


@pytest.mark.parametrize("m,n,k,adv", [(64, 32, 64, False), (128, 64, 128, False), (33, 70, 192, True), (5, 40, 128, False),
                                       (32, 2112, 2816, False), (32, 2816, 2112, False), (100, 704, 2816, True), (32, 2816, 704, False),
                                       # scales are staged six groups at a time: rows of 1, 5, 6, 7 and 13 groups, and the shortest arrays taken
                                       (17, 8, 64, False), (40, 24, 320, True), (40, 33, 384, False), (70, 65, 448, True), (12, 31, 832, False), (9, 2, 192, False)])
def test_int4_qmm_on_matrix_cores(m, n, k, adv):
    # MPPPrefillInt4QMMTests.swift:183-200 (rel <= 1e-3 vs the fp32-fma CPU reference rounded to fp16) + production shapes
    W, S, B, x = mpp_inputs(m, n, k, adv)
    kk = ctx()
    y = zeros_bytes(m * n * 2 + 64, 0xEE)
    dW, dS, dB, dx = dev(W), dev(S), dev(B), dev(x)
    rc = kk.lib.tf_int4_qmm(kk.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0,
                            y.data_ptr(), 0, m, n, k, tfk.TF_BF16)
    assert rc == tfk.TF_OK, kk.last_error()
    got = tfo.from_f16_bits(host(y, np.uint16, m * n)).reshape(m, n)
    assert np.all(host(y, np.uint8)[m * n * 2:] == 0xEE)
    want = tfo.qmm_cpu_reference(W, S, B, x, m, n, k, threads=8)
    assert tfo.rel_error(got, want) <= 1e-3
    assert within_north_star(got, want)


@pytest.mark.parametrize("m,n,k,lo,hi,mixed", [(64, 128, 2816, 2e-6, 5e-5, False), (40, 96, 704, 1e-7, 3e-6, False), (33, 64, 2112, 3e-5, 9e-5, False),
                                                (48, 160, 1408, 1e-6, 4e-5, True)])
def test_int4_qmm_on_matrix_cores_with_scales_below_fp16_normal_range(m, n, k, lo, hi, mixed):
    # The reference's staged-affine path forms half(fma(float(q), scale, bias)) in fp32 (Metal/TensorCore/tensorops.metal:73-75), so a
    # bf16 scale of any size keeps its mantissa.  Scales of 1e-7 ... 9e-5 lie below or across the bottom of fp16's normal range
    # (6.1e-5): the matrix-core path carries every weight row times a power of two and must still meet the MPP tolerance.
    rng = np.random.default_rng(int(k + m))
    groups = k // 64
    W = rng.integers(0, 256, (n, k // 2), dtype=np.uint8)
    s = rng.uniform(lo, hi, (n, groups)).astype(np.float32)
    if mixed:   # every third row has ordinary scales: rows of both kinds share a wave, each is carried at its own power of two
        s[::3] = rng.uniform(0.004, 0.02, s[::3].shape).astype(np.float32)
    S = tfo.bf16_bits_array(s).reshape(n, groups)
    B = tfo.bf16_bits_array((-7.5 * s * rng.uniform(0.5, 1.5, (n, groups))).astype(np.float32)).reshape(n, groups)
    x = tfo.to_f16_bits(rng.standard_normal(m * k).astype(np.float32) * 4.0)
    kk = ctx()
    y = zeros_bytes(m * n * 2)
    dW, dS, dB, dx = dev(W), dev(S), dev(B), dev(x)
    assert kk.lib.tf_int4_qmm(kk.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0, y.data_ptr(), 0, m, n, k,
                              tfk.TF_BF16) == tfk.TF_OK
    got = tfo.from_f16_bits(host(y, np.uint16, m * n)).reshape(m, n).astype(np.float64)
    # fp64 reference from the fp32 weights float(q) * s + b (what every path approximates), beside the reference's own fp32 loop
    nib = np.stack([W & 0xF, W >> 4], axis=2).reshape(n, k).astype(np.float32)
    wf = (nib * np.repeat(tfo.bf16_array_to_float(S.ravel()).reshape(n, groups), 64, axis=1)
          + np.repeat(tfo.bf16_array_to_float(B.ravel()).reshape(n, groups), 64, axis=1)).astype(np.float64)
    exact = tfo.from_f16_bits(x).reshape(m, k).astype(np.float64) @ wf.T
    scale = np.max(np.abs(exact), axis=0)   # per weight row: a tiny row beside an ordinary one is held to its own size
    assert np.all(np.abs(got - exact) <= 1e-3 * scale[None, :]), float(np.max(np.abs(got - exact) / scale[None, :]))
    want = tfo.qmm_cpu_reference(W, S, B, x, m, n, k, threads=8)
    assert tfo.rel_error(got.astype(np.float32), want) <= 1e-3


def test_int4_qmm_unavailable_and_exact_variant():
    W, S, B, x = mpp_inputs(8, 64, 128)
    kk = ctx()
    y = zeros_bytes(8 * 64 * 2, 0xEE)
    dW, dS, dB, dx = dev(W, 2), dev(S), dev(B), dev(x)
    # k not a multiple of 64 / misaligned weights: Path.unavailable, nothing enqueued (MPPPrefillInt4QMM.swift:40-56)
    assert kk.lib.tf_int4_qmm(kk.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0, y.data_ptr(), 0, 8, 64, 96, tfk.TF_BF16) == tfk.TF_ERR_UNAVAILABLE
    assert kk.lib.tf_int4_qmm(kk.handle, None, dW.data_ptr(), 2, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0, y.data_ptr(), 0, 8, 64, 128, tfk.TF_BF16) == tfk.TF_ERR_UNAVAILABLE
    assert kk.lib.tf_int4_qmm(kk.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0, y.data_ptr(), 0, 0, 64, 128, tfk.TF_BF16) == tfk.TF_ERR_UNAVAILABLE
    # fewer than six scale values in the whole matrix: left to the exact kernel
    assert kk.lib.tf_int4_qmm(kk.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0, y.data_ptr(), 0, 8, 5, 64, tfk.TF_BF16) == tfk.TF_ERR_UNAVAILABLE
    torch.cuda.synchronize()
    assert np.all(host(y, np.uint8) == 0xEE)
    # the exact (fp32 weight) QMM equals repeated GEMV bit for bit, at the +2 weight offset too (PrefillAffineTests.swift:176-231)
    kk.check(kk.lib.tf_prefill_int4_qmm(kk.handle, None, dW.data_ptr(), 2, dS.data_ptr(), 0, dB.data_ptr(), 0, dx.data_ptr(), 0, y.data_ptr(), 0, 8, 64, 128, tfk.TF_BF16))
    got = host(y, np.uint16, 8 * 64).reshape(8, 64)
    for t in range(8):
        yr = zeros_bytes(64 * 2)
        kk.dequant_int4_gemv(dW, dS, dB, dev(x[t * 128:(t + 1) * 128]), yr, 64, 128, offsets=(2, 0, 0, 0, 0))
        assert np.array_equal(host(yr, np.uint16, 64), got[t])
    ref = tfo.qmm_cpu_reference(W, S, B, x, 8, 64, 128)
    assert np.max(np.abs(tfo.from_f16_bits(got.ravel()).reshape(8, 64) - ref)) <= 2e-4 + 5e-4 * np.max(np.abs(ref))

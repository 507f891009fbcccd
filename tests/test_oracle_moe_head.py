"""Pins the oracle's GELU, RMSNorm, router, routed/shared expert and lm_head references."""
import numpy as np
import torch

import refcases
from test_oracle_quant_gemv import np_dequant


def test_gelu_matches_torch_tanh_approximation_and_known_points(tfo):
    x = np.linspace(-8, 8, 4001, dtype=np.float32)
    want = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    assert np.max(np.abs(tfo.gelu_tanh(x) - want)) < 2e-6
    # MoEReferenceTests.swift:7-17
    y = tfo.gelu_tanh(np.array([0.0, 1.0, -1.0, 2.0], np.float32))
    assert abs(y[0]) < 1e-7
    assert abs(y[1] - 0.5 * (1 + np.tanh(0.7978845608028654 * (1 + 0.044715)))) < 1e-5
    assert y[1] > 0 and y[2] < 0 and y[3] > y[1]


def test_rmsnorm_matches_float64(tfo):
    # RMSNormReferenceTests.swift:28-43 shapes/seeds
    for d, seed in [(256, 0xA1), (512, 0xB2), (2816, 0xC3)]:
        rng = tfo.SeedTree(seed).key("rmsnorm-ref")
        x, w = rng.uniform_array(-1.0, 1.0, d), rng.uniform_array(0.5, 1.5, d)
        x64, w64 = x.astype(np.float64), w.astype(np.float64)
        want = x64 * w64 / np.sqrt(np.mean(x64 * x64) + 1e-6)
        assert tfo.rel_error(tfo.rmsnorm_ref(x, w, 1e-6), want.astype(np.float32)) < tfo.Tolerance.identity
    y = tfo.rmsnorm_ref(np.array([1e-4, -1e-4, 2e-4, -2e-4] * 2, np.float32), np.ones(8, np.float32), 1e-6)
    assert np.all(np.isfinite(y))


def _router_expect(tfo, weights, hidden, eff, expert_scale):
    """Independent float64 statement of RouterTopKTests.reference."""
    W, S, B = tfo.quantize_int8(weights)
    logits = np_dequant(W, S, B, 8, tfo).astype(np.float64) @ (hidden * eff).astype(np.float64)
    order = sorted(range(len(logits)), key=lambda e: (-logits[e], e))[:8]
    p = torch.softmax(torch.tensor(logits[order]), 0).numpy()
    return (W, S, B), np.array(order), p * expert_scale[order], logits


def test_router_reference_production_case(tfo):
    weights, hidden, eff, escale = refcases.router_case_production()
    (W, S, B), order, wts, logits = _router_expect(tfo, weights, hidden, eff, escale)
    idx, w, lg = tfo.router_reference(W, S, B, hidden, eff, escale)
    assert np.allclose(lg, logits, rtol=1e-5, atol=1e-6)
    assert list(idx) == list(order)
    assert np.max(np.abs(w - wts)) < 1e-6
    # experts carry a +0.01*e offset and hidden*eff has a positive mean: the high experts must win, best first
    assert list(idx) == sorted(idx, key=lambda e: -logits[e])


def test_router_reference_near_tie_known_answer(tfo):
    # RouterTopKTests.swift:46-70: gains 1.0,0.95,..0.70 then 0.5 (e7) vs 0.5*(1+1e-4) (e8) => e8 beats e7
    weights, hidden, eff, escale = refcases.router_case_near_tie()
    W, S, B = tfo.quantize_int8(weights)
    idx, w, lg = tfo.router_reference(W, S, B, hidden, eff, escale)
    assert list(idx) == [0, 1, 2, 3, 4, 5, 6, 8]
    assert abs(float(w.sum()) - 1.0) < 1e-6
    # kernel-order restatement (bf16 scales, fp16 hidden) must pick the same experts
    k_logits = tfo.k_router_logits(W, S, B, tfo.to_f16_bits(hidden), tfo.bf16_bits_array(eff))
    k_idx, k_w = tfo.k_router_topk(k_logits, tfo.bf16_bits_array(escale))
    assert list(k_idx) == [0, 1, 2, 3, 4, 5, 6, 8]
    assert np.max(np.abs(tfo.from_f16_bits(k_w) - w)) < 5e-3
    p_logits = tfo.k_router_logits(W, S, B, tfo.to_f16_bits(hidden), tfo.bf16_bits_array(eff), prefill_order=True)
    assert list(tfo.k_router_topk(p_logits, tfo.bf16_bits_array(escale))[0]) == [0, 1, 2, 3, 4, 5, 6, 8]


def test_router_exact_ties_prefer_lower_index(tfo):
    # moe.metal:157 — equal scores: lower expert index first
    logits = np.array([1.0, 3.0, 3.0, 0.5, 3.0, -1.0, 2.0, 2.0, 0.0, 2.0], np.float32)
    idx, w = tfo.k_router_topk(logits, tfo.bf16_bits_array(np.ones(10, np.float32)))
    assert list(idx) == [1, 2, 4, 6, 7, 9, 0, 3]
    want = torch.softmax(torch.tensor(logits[list(idx)].astype(np.float64)), 0).numpy()
    assert np.max(np.abs(tfo.from_f16_bits(w) - want)) < 1e-3
    W = np.zeros((10, 64), np.uint8)
    W[:, 0] = [1, 3, 3, 0, 3, 0, 2, 2, 0, 2]
    one, zero = np.full((10, 1), tfo.bf16_bits(1.0), np.uint16), np.zeros((10, 1), np.uint16)
    hidden = np.zeros(64, np.float32)
    hidden[0] = 1.0
    ridx, _, _ = tfo.router_reference(W, one, zero, hidden, np.ones(64, np.float32), np.ones(10, np.float32))
    assert list(ridx[:6]) == [1, 2, 4, 6, 7, 9]


def test_moe_reference_matches_float64_composition(tfo):
    c = refcases.moe_fused_case()
    d, f, off = c["d"], c["f"], c["off"]
    x = tfo.from_f16_bits(c["x_bits"])
    res = tfo.from_f16_bits(c["residual_bits"])
    rw = tfo.from_f16_bits(c["routing_w_bits"])
    y = tfo.moe_apply_streamed_routed(c["blobs"], off, x, res, rw, d, f)

    def mat(blob, w_off, s_off, b_off, rows, cols):
        W = blob[w_off:w_off + rows * cols // 2].reshape(rows, cols // 2)
        S = blob[s_off:s_off + rows * cols // 64 * 2].view("<u2").reshape(rows, cols // 64)
        B = blob[b_off:b_off + rows * cols // 64 * 2].view("<u2").reshape(rows, cols // 64)
        return np_dequant(W, S, B, 4, tfo).astype(np.float64)

    want = res.astype(np.float64)
    for slot, blob in enumerate(c["blobs"]):
        g = mat(blob, off.gate_W_off, off.gate_s_off, off.gate_b_off, f, d) @ x
        u = mat(blob, off.up_W_off, off.up_s_off, off.up_b_off, f, d) @ x
        act = torch.nn.functional.gelu(torch.from_numpy(g), approximate="tanh").numpy() * u
        want = want + rw[slot] * (mat(blob, off.down_W_off, off.down_s_off, off.down_b_off, d, f) @ act)
    assert tfo.rel_error(y, want.astype(np.float32)) < 2e-5
    assert np.array_equal(tfo.moe_apply_streamed_routed(c["blobs"], off, x, res, rw, d, f, threads=4), y)
    # kernel-order chain (fp16 acts, fp16 output) stays inside the reference's own budget (MoEFusedFFNTests.swift:157-158)
    acts = tfo.k_moe_phase1(c["blobs"], off, c["x_bits"], d, f)
    yk = tfo.from_f16_bits(tfo.k_moe_phase2(c["blobs"], off, acts, c["routing_w_bits"], c["residual_bits"], d, f))
    assert tfo.rel_error(yk, y) < tfo.Tolerance.fp16ChainedReduction


def test_shared_expert_reference(tfo):
    c = refcases.shared_expert_case()
    x = tfo.from_f16_bits(c["x_bits"])
    y = tfo.shared_expert_ref(c["gate"], c["up"], c["down"], x)
    g = np_dequant(*c["gate"], 4, tfo).astype(np.float64) @ x
    u = np_dequant(*c["up"], 4, tfo).astype(np.float64) @ x
    act = (torch.nn.functional.gelu(torch.from_numpy(g), approximate="tanh").numpy() * u).astype(np.float16).astype(np.float64)
    want = np_dequant(*c["down"], 4, tfo).astype(np.float64) @ act
    # fp16 rounding of act can flip by one ulp between the fp32 and fp64 routes: allow a few ulps of act through down
    assert tfo.rel_error(y, want.astype(np.float32)) < 1e-3
    # kernel-order: gate/up rounded to fp16 first (SharedExpertInt4.swift:61-99, utility.metal:6-18)
    gk = tfo.to_f16_bits(tfo.k_int4_gemv(*c["gate"], c["x_bits"]))
    uk = tfo.to_f16_bits(tfo.k_int4_gemv(*c["up"], c["x_bits"]))
    yk = tfo.k_int4_gemv(*c["down"], tfo.k_gelu_mul_fp16(gk, uk))
    assert tfo.rel_error(tfo.from_f16_bits(tfo.to_f16_bits(yk)), y) < tfo.Tolerance.quantInt4 * 4   # SharedExpertInt4Tests.swift:52


def test_lm_head_greedy_known_answers(tfo):
    d, v = 64, 1024
    one = tfo.bf16_bits_array(np.ones(d, np.float32))
    # ties resolve to the lowest index (LMHeadChainInt4Tests.swift:174-190)
    hidden = tfo.to_f16_bits(np.float32(0.2) + (np.arange(d) % 5).astype(np.float32) * np.float32(0.02))
    W, S, B = refcases.lm_head_constant_rows(d, v, [17, 311], hot=1.0, cold=-0.25)
    assert tfo.lm_head_cpu_greedy(hidden, one, W, S, B) == 17
    # all-NaN hidden: nothing beats -inf => token 0 (:136-150)
    W, S, B = tfo.quantize_int4(np.full((v, d), 0.25, np.float32))
    assert tfo.lm_head_cpu_greedy(np.full(d, 0x7E00, np.uint16), one, W, S, B) == 0
    # single hot row at v-3 for several vocab sizes (:152-172)
    for vv in (1024, 2048, 4096):
        hidden = tfo.to_f16_bits(np.float32(0.25) + (np.arange(d) % 7).astype(np.float32) * np.float32(0.01))
        W, S, B = refcases.lm_head_constant_rows(d, vv, [vv - 3])
        assert tfo.lm_head_cpu_greedy(hidden, one, W, S, B) == vv - 3


def test_lm_head_greedy_random_case_vs_float64(tfo):
    hidden_bits, norm_bits, W, S, B = refcases.lm_head_random_case()
    tok, logits = tfo.lm_head_cpu_greedy(hidden_bits, norm_bits, W, S, B, want_logits=True)
    h = tfo.from_f16_bits(hidden_bits).astype(np.float64)
    nw = tfo.bf16_array_to_float(norm_bits).astype(np.float64)
    normed = (h * nw / np.sqrt(np.mean(h * h) + 1e-6)).astype(np.float32).astype(np.float16).astype(np.float64)
    want = np_dequant(W, S, B, 4, tfo).astype(np.float64) @ normed
    assert tfo.rel_error(logits, want.astype(np.float32)) < 1e-3   # fp16 rounding of the normed vector may differ by an ulp
    top2 = np.sort(want)[-2:]
    assert top2[1] - top2[0] > 1e-3 and tok == int(np.argmax(want))
    assert tfo.lm_head_cpu_greedy(hidden_bits, norm_bits, W, S, B, threads=4) == tok

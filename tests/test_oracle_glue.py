"""Pins the CPU restatement of the two stages around the MoE block (fused_post_attn_setup, fused_layer_tail) by what the
arithmetic fixes: compositions of the already pinned RMSNorm reference, special cases with closed forms, and float64."""
import numpy as np

from oracle import tfo

D, EPS = 2816, 1e-6


def _draw(seed):
    rng = tfo.SplitMix64(seed)
    half = lambda: tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, D))
    weight = lambda: tfo.bf16_bits_array(rng.uniform_array(0.5, 1.5, D))
    return rng, half, weight


def test_layer_tail_kernel_order_follows_the_reference_tests_cpu_reference():
    # FusedLayerTailTests.swift:11-74: seed, draw order and the 4e-3 bound of the reference's own test
    rng, half, weight = _draw(0xC0DE7A11)
    h2, h1, hidden = half(), half(), half()
    w2, w = weight(), weight()
    scalar = rng.uniform(0.75, 1.25)
    got = tfo.from_f16_bits(tfo.k_layer_tail(h2, h1, hidden, w2, w, EPS, scalar))
    ref = tfo.layer_tail_ref(h2, h1, hidden, w2, w, EPS, scalar)
    assert np.max(np.abs(got - ref)) / max(float(np.max(np.abs(ref))), 1e-6) < 4e-3
    # float64 with the same fp16 stage boundaries
    f = lambda b: tfo.from_f16_bits(b).astype(np.float64)
    r16 = lambda v: v.astype(np.float16).astype(np.float64)
    wf = lambda b: tfo.bf16_array_to_float(b).astype(np.float64)
    n2 = r16(f(h2) / np.sqrt(np.mean(f(h2) ** 2) + EPS) * wf(w2))
    h12 = r16(f(h1) + n2)
    n12 = r16(h12 / np.sqrt(np.mean(h12 ** 2) + EPS) * wf(w))
    want = r16(r16(f(hidden) + n12) * float(np.float16(scalar)))
    assert np.max(np.abs(got - want)) <= 2 ** -9          # at most one fp16 ulp of values below 4 where a rounding flips


def test_layer_tail_special_cases():
    _, half, weight = _draw(0x7A11)
    h1, hidden = half(), half()
    ones = tfo.bf16_bits_array(np.ones(D, np.float32))
    zeros = np.zeros(D, np.uint16)
    # h2 = 0 -> its normalised branch vanishes: hidden' = (hidden + rmsnorm(h1)) * scalar
    got = tfo.from_f16_bits(tfo.k_layer_tail(zeros, h1, hidden, ones, ones, EPS, 1.0))
    n1 = tfo.from_f16_bits(tfo.k_rmsnorm_bf16w(h1, ones, EPS))
    want = (tfo.from_f16_bits(hidden) + n1).astype(np.float16).astype(np.float32)
    assert np.array_equal(got, want)
    # scalar 0 -> zeros; scalar 2 doubles exactly
    assert not np.any(tfo.from_f16_bits(tfo.k_layer_tail(zeros, h1, hidden, ones, ones, EPS, 0.0)))
    assert np.array_equal(tfo.from_f16_bits(tfo.k_layer_tail(zeros, h1, hidden, ones, ones, EPS, 2.0)), 2.0 * want)


def test_post_attn_setup_is_the_chain_of_standalone_kernels():
    # FusedPostAttentionSetupTests.swift:11-113 compares the fused kernel with rmsnorm_bf16w -> residual add -> rmsnorm:
    # the restatement must equal the chain built from the (separately pinned) rmsnorm restatement bit for bit
    _, half, weight = _draw(0x9057A77E)
    hidden, attn = half(), half()
    w_post, w_pre, w_pre2 = weight(), weight(), weight()
    h_out, dense, routed, router = tfo.k_post_attn_setup(hidden, attn, w_post, w_pre, w_pre2, EPS)
    an = tfo.k_rmsnorm_bf16w(attn, w_post, EPS)
    h_want = tfo.to_f16_bits(tfo.from_f16_bits(hidden) + tfo.from_f16_bits(an))
    assert np.array_equal(h_out, h_want)
    assert np.array_equal(dense, tfo.k_rmsnorm_bf16w(h_want, w_pre, EPS))
    assert np.array_equal(routed, tfo.k_rmsnorm_bf16w(h_want, w_pre2, EPS))
    assert np.array_equal(router, tfo.k_rmsnorm_bf16w(h_want, tfo.bf16_bits_array(np.ones(D, np.float32)), EPS))
    # and the fp32 RMSNorm reference within its fp16 output rounding
    ref = tfo.rmsnorm_ref(tfo.from_f16_bits(h_want), tfo.bf16_array_to_float(w_pre), EPS)
    assert np.max(np.abs(tfo.from_f16_bits(dense) - ref)) <= 2e-3 * float(np.max(np.abs(ref)))
    rms = np.sqrt(np.mean(tfo.from_f16_bits(router).astype(np.float64) ** 2))
    assert abs(rms - 1.0) < 2e-3                        # router_x is the unit-RMS view of hidden

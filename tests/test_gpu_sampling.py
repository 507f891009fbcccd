"""GPU parity of the output head's neighbours through the C ABI: embedding row lookup, soft-capped softmax, samplers.
Cases restate EmbedLookupTests, PrefillPrimitiveTests (embed block), LogitSoftcapSoftmaxTests, SampleTests and
SampleTopK64Tests of the reference; tokens are compared with the CPU oracle draw by draw."""
import numpy as np
import pytest

from gpu_helpers import ctx, dev, host, tfk, zeros_bytes
from oracle import tfo

pytestmark = pytest.mark.gpu


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16).view(np.uint16)


def gpu_sample(d_probs, v, temperature, top_k, top_p, seed, position=0, topk64=False):
    k = ctx()
    tok = zeros_bytes(4, 0xEE)
    if topk64:
        k.check(k.lib.tf_sample_topk64(k.handle, None, d_probs.data_ptr(), tok.data_ptr(), v, temperature, top_p, seed))
    else:
        k.check(k.lib.tf_sample(k.handle, None, d_probs.data_ptr(), tok.data_ptr(), v, temperature, top_k, top_p, seed, position))
    return int(host(tok, np.uint32, 1)[0])


@pytest.mark.parametrize("byte_off", [0, 2])
def test_embed_lookup_rows(byte_off):
    # EmbedLookupTests.swift:38-110 (V=16, D=128, token 9, sqrt(D) and unit scale) and the tied 2816-wide table
    for rows, d, token, seed in ((16, 128, 9, 0x131), (16, 128, 0, 0x132), (40, 2816, 39, 0x133)):
        rng = tfo.SeedTree(seed).key("embed-lookup-int4-table")
        W, S, B = tfo.quantize_int4(rng.uniform_array(-1.0, 1.0, rows * d).reshape(rows, d))
        k = ctx()
        dW, dS, dB = dev(W, byte_off), dev(S, byte_off), dev(B, byte_off)
        for scale in (float(np.sqrt(np.float32(d))), 1.0):
            out = dev(np.zeros(d + 8, np.uint16), byte_off)
            k.check(k.lib.tf_embed_lookup_int4(k.handle, None, dW.data_ptr(), byte_off, dS.data_ptr(), byte_off, dB.data_ptr(), byte_off,
                                               out.data_ptr(), byte_off, token, d, scale, rows))
            got = host(out, np.uint16, d + 8, byte_off)
            want = tfo.embed_lookup_int4(W, S, B, token, scale)
            assert np.array_equal(got[:d], f16(want)) and not np.any(got[d:])        # bit-exact: fp32 affine, one rounding to half
            assert tfo.rel_error(tfo.from_f16_bits(got[:d]), want) < 2e-3
        assert k.lib.tf_embed_lookup_int4(k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, out.data_ptr(), 0, rows, d, 1.0,
                                          rows) == tfk.TF_ERR_INVALID_ARGUMENT         # token outside the table
        assert k.lib.tf_embed_lookup_int4(k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, out.data_ptr(), 0, 0, 100, 1.0,
                                          rows) == tfk.TF_ERR_INVALID_ARGUMENT         # D % 64 (EmbedLookupInt4.swift:20)


def test_embed_lookup_block_equals_single_rows():
    rows, d = 50, 2816
    rng = tfo.SeedTree(0x134).key("embed-lookup-int4-table")
    W, S, B = tfo.quantize_int4(rng.uniform_array(-1.0, 1.0, rows * d).reshape(rows, d))
    tokens = np.array([3, 49, 0, 3, 17, 1000], np.uint32)         # the last one is outside the table: reads the last row
    k = ctx()
    dW, dS, dB, dT = dev(W), dev(S), dev(B), dev(tokens)
    out = zeros_bytes(tokens.size * d * 2)
    scale = float(np.sqrt(np.float32(d)))
    k.check(k.lib.tf_prefill_embed_lookup_int4_block(k.handle, None, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, dT.data_ptr(), 0,
                                                     out.data_ptr(), 0, tokens.size, d, scale, rows))
    got = host(out, np.uint16, tokens.size * d).reshape(tokens.size, d)
    for i, t in enumerate(tokens):
        assert np.array_equal(got[i], f16(tfo.embed_lookup_int4(W, S, B, min(int(t), rows - 1), scale))), i


@pytest.mark.parametrize("v,dtype", [(2048, "f16"), (2048, "f32"), (262144, "f16"), (1000, "f16"), (100, "f16")])
def test_softcap_softmax_matches_reference(v, dtype):
    # LogitSoftcapSoftmaxTests.swift:34-54 (random logits in +-50, bounded relative error with floor 1e-4, sum to one)
    rng = tfo.SeedTree(0x131).key("softcap-softmax-random")
    x16 = f16(rng.uniform_array(-50.0, 50.0, v))
    x = tfo.from_f16_bits(x16)
    k = ctx()
    d_in = dev(x16) if dtype == "f16" else dev(x)
    probs = zeros_bytes(v * 2 + 16, 0xEE)
    k.check(k.lib.tf_logit_softcap_softmax(k.handle, None, d_in.data_ptr(), probs.data_ptr(), v, 30.0, tfk.TF_FP16 if dtype == "f16" else tfk.TF_FP32))
    got = tfo.from_f16_bits(host(probs, np.uint16, v))
    assert np.all(host(probs, np.uint8)[v * 2:] == 0xEE)
    ref = tfo.logit_softcap_softmax_ref(x, 30.0)
    assert tfo.bounded_rel(got, ref, 1e-4) < tfo.Tolerance.fp16Reduction
    assert abs(float(got.astype(np.float64).sum()) - 1.0) < tfo.Tolerance.fp16Reduction
    assert int(np.argmax(got)) == int(np.argmax(ref)) or ref[int(np.argmax(got))] >= ref.max() * (1 - 2e-3)


def test_softcap_softmax_uniform_and_saturated_inputs():
    # LogitSoftcapSoftmaxTests.swift:56-89
    k = ctx()
    v = 2048
    probs = zeros_bytes(v * 2)
    flat = dev(np.full(v, tfo.f16_bits(0.1234), np.uint16))
    k.check(k.lib.tf_logit_softcap_softmax(k.handle, None, flat.data_ptr(), probs.data_ptr(), v, 30.0, tfk.TF_FP16))
    assert np.max(np.abs(tfo.from_f16_bits(host(probs, np.uint16, v)) - 1.0 / v)) < 5e-4
    spike = np.zeros(v, np.float32)
    spike[42] = 1000.0
    d_spike = dev(f16(spike))
    k.check(k.lib.tf_logit_softcap_softmax(k.handle, None, d_spike.data_ptr(), probs.data_ptr(), v, 5.0, tfk.TF_FP16))
    g = float(tfo.from_f16_bits(host(probs, np.uint16, v))[42])
    c = float(tfo.logit_softcap_softmax_ref(tfo.from_f16_bits(f16(spike)), 5.0)[42])
    assert c < 0.5 and abs(g - c) / c < tfo.Tolerance.fp16Reduction
    assert k.lib.tf_logit_softcap_softmax(k.handle, None, probs.data_ptr(), probs.data_ptr(), 0, 30.0, tfk.TF_FP16) == tfk.TF_ERR_INVALID_ARGUMENT


def test_greedy_sampling_picks_the_argmax():
    # SampleTests.swift:52-65, ties, and the production vocabulary
    values = np.full(2048, 0.01, np.float32)
    values[1337] = 5.0
    assert gpu_sample(dev(f16(values / values.sum())), 2048, 0.0, 0, 1.0, 1) == 1337
    tie = np.full(5000, 0.0001, np.float32)
    tie[[4100, 311, 2900]] = 0.2
    assert gpu_sample(dev(f16(tie)), 5000, 0.0, 0, 1.0, 1) == 311
    big = np.random.default_rng(5).random(262144).astype(np.float32) / 131072
    bits = f16(big)
    assert gpu_sample(dev(bits), 262144, 0.0, 64, 0.95, 9) == tfo.sample(bits, 0.0, 64, 0.95, 9)


def test_gumbel_sampling_equals_the_reference_draw_by_draw():
    # SampleTests.swift:67-123: determinism, in-range ids on a spread distribution, concentration on a peak
    rng = tfo.SeedTree(0x51A71004).key("sample-gumbel-spread")
    v = 4096
    spread = rng.uniform_array(0.5, 1.0, v)
    bits = f16(spread / spread.sum())
    d_probs = dev(bits)
    close = 0
    for t in range(16):
        seed = ((t + 1) * 0x9E3779B97F4A7C15) & ((1 << 64) - 1)
        got = gpu_sample(d_probs, v, 2.0, 0, 1.0, seed, position=t)
        assert got < v and got == gpu_sample(d_probs, v, 2.0, 0, 1.0, seed, position=t)
        close += got == tfo.sample(bits, 2.0, 0, 1.0, seed, position=t)
    assert close >= 15                   # log / tanh differ in the last bit between the CPU and GPU libraries: near-ties may flip
    peaked = np.full(v, 0.0001, np.float32)
    peaked[2049] = 0.9
    d_peak = dev(f16(peaked / peaked.sum()))
    hits = sum(gpu_sample(d_peak, v, 0.3, 0, 1.0, ((t + 1) * 0x9E3779B97F4A7C15) & ((1 << 64) - 1)) == 2049 for t in range(32))
    assert hits >= 31
    big = np.random.default_rng(6).random(262144).astype(np.float32) / 131072
    bits = f16(big)
    d_big = dev(bits)
    assert sum(gpu_sample(d_big, 262144, 0.9, 0, 1.0, s, position=3) == tfo.sample(bits, 0.9, 0, 1.0, s, position=3) for s in (1, 2, 3, 4)) >= 3


@pytest.mark.parametrize("v", [1003, 1024, 5000, 262144])
def test_truncating_samplers_equal_the_reference_draw_by_draw(v):
    # SampleTests.swift:125-157 and SampleTopK64Tests.swift:84-131
    if v == 262144:
        i = np.arange(v, dtype=np.uint64)
        mixed = i * np.uint64(6364136223846793005) + np.uint64(1442695040888963407)
        values = ((mixed >> np.uint64(40)).astype(np.float32) + 1.0) * np.float32(1.0 / 16777217.0)
    else:
        values = np.random.default_rng(v).random(v).astype(np.float32)
        values /= values.sum()
    bits = f16(values)
    d_probs = dev(bits)
    agree = total = 0
    for temperature in (0.7, 0.85, 1.0):
        for seed in (1, 2, 0x123456789ABCDEF0, (1 << 64) - 1):
            a = gpu_sample(d_probs, v, temperature, 64, 0.95, seed)
            b = gpu_sample(d_probs, v, temperature, 0, 0.95, seed, topk64=True)
            assert a == b                                                            # the two GPU samplers agree exactly
            agree += a == tfo.sample(bits, temperature, 64, 0.95, seed)
            total += 1
    assert agree >= total - 1            # pow differs in the last bit between libraries: a draw on a CDF boundary may move
    for top_k, top_p, temperature in ((4, 1.0, 1.0), (200, 0.5, 0.8), (0, 0.3, 1.3), (256, 0.999, 1.0)):
        for seed in (11, 12, 13):
            assert gpu_sample(d_probs, v, temperature, top_k, top_p, seed) == tfo.sample(bits, temperature, top_k, top_p, seed), (top_k, top_p, seed)


def test_top_k_keeps_only_the_top_and_ties_resolve_to_low_indices():
    values = np.full(1024, 0.0001, np.float32)
    top = [10, 200, 500, 900]
    values[top] = [0.40, 0.30, 0.20, 0.10]
    d_probs = dev(f16(values / values.sum()))
    for t in range(32):
        assert gpu_sample(d_probs, 1024, 1.0, 4, 1.0, ((t + 1) * 0x9E3779B97F4A7C15) & ((1 << 64) - 1)) in top
    ones = f16(np.ones(1003))
    d_ones = dev(ones)
    for seed in range(1, 9):
        got = gpu_sample(d_ones, 1003, 1.0, 0, 0.95, seed, topk64=True)
        assert got < 64 and got == tfo.sample_topk64(ones, 1.0, 0.95, seed)
    flat = f16(np.full(1003, 1.0 / 1003.0))
    d_flat = dev(flat)
    picks = [gpu_sample(d_flat, 1003, 1.0, 0, 0.95, s, topk64=True) for s in range(1, 65)]
    assert max(picks) < 64 and picks == [tfo.sample_topk64(flat, 1.0, 0.95, s) for s in range(1, 65)]
    k = ctx()
    assert k.lib.tf_sample_topk64(k.handle, None, d_flat.data_ptr(), d_flat.data_ptr(), 262145, 1.0, 0.95, 1) == tfk.TF_ERR_INVALID_ARGUMENT
    assert k.lib.tf_sample(k.handle, None, d_flat.data_ptr(), d_flat.data_ptr(), 0, 1.0, 0, 1.0, 1, 0) == tfk.TF_ERR_INVALID_ARGUMENT

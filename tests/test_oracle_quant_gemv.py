"""Pins the oracle's quantizer and GEMV references: the reference tests' known answers,
independent numpy bit-twiddling, float64 brute force and closed-form special cases."""
import numpy as np
import pytest

import refcases


def np_unpack_nibbles(W):
    """Independent unpack: element 2k = low nibble of byte k, 2k+1 = high nibble."""
    out = np.empty((W.shape[0], W.shape[1] * 2), np.uint8)
    out[:, 0::2] = W & 0x0F
    out[:, 1::2] = W >> 4
    return out


def np_dequant(W, S, B, bits, tfo):
    q = np_unpack_nibbles(W) if bits == 4 else W
    s = np.repeat(tfo.bf16_array_to_float(S).reshape(S.shape), 64, axis=1)
    b = np.repeat(tfo.bf16_array_to_float(B).reshape(B.shape), 64, axis=1)
    return q.astype(np.float32) * s + b      # product exact in fp32 => one rounding


def test_nibble_layout_low_even_high_odd(tfo):
    # QuantizationTests.swift:35-50
    row = (np.arange(64, dtype=np.float32) - np.float32(31.5))[None, :]
    W, S, B = tfo.quantize_int4(row)
    lo, hi = int(W[0, 0] & 0x0F), int(W[0, 0] >> 4)
    scale, bias = tfo.bf16_to_float(S[0, 0]), tfo.bf16_to_float(B[0, 0])
    assert abs(lo * scale + bias - row[0, 0]) <= scale + 1e-3
    assert abs(hi * scale + bias - row[0, 1]) <= scale + 1e-3
    # a monotone ramp over 64 elements with 16 levels: element k quantises to round(k*15/63)
    q = np_unpack_nibbles(W)[0]
    assert q[0] == 0 and q[-1] == 15 and np.all(np.diff(q.astype(int)) >= 0)
    assert (lo, hi) == (0, 0) and int(W[0, 31] >> 4) == 15


def test_literal_roundtrip_bounds(tfo):
    # QuantizationAffineTests.swift:7-29 (int4 < 0.025) and :31-46 (int8 < 0.008)
    row = np.concatenate([np.float32(0.10) + np.arange(64, dtype=np.float32) * np.float32(0.01),
                          np.float32(-0.50) - np.arange(64, dtype=np.float32) * np.float32(0.005)])[None, :]
    W, S, B = tfo.quantize_int4(row)
    assert W.shape == (1, 64) and S.shape == (1, 2) and B.shape == (1, 2)
    assert np.max(np.abs(tfo.dequantize_int4(W, S, B) - row)) < 0.025
    row8 = (np.float32(-0.3) + np.arange(64, dtype=np.float32) * np.float32(0.02))[None, :]
    W8, S8, B8 = tfo.quantize_int8(row8)
    assert W8.shape == (1, 64) and S8.shape == (1, 1)
    assert np.max(np.abs(tfo.dequantize_int8(W8, S8, B8) - row8)) < 0.008


def test_constant_group_is_exact_bf16(tfo):
    # QuantizationAffineTests.swift:61-73
    W, S, B = tfo.quantize_int4(np.full((1, 64), 0.42, np.float32))
    assert S[0, 0] == tfo.bf16_bits(1.0) and np.all(W == 0)
    want = tfo.bf16_to_float(tfo.bf16_bits(0.42))
    assert np.all(np.abs(tfo.dequantize_int4(W, S, B) - want) < 1e-6)


def test_positive_only_uses_full_codebook(tfo):
    # QuantizationAffineTests.swift:76-88
    row = (np.arange(64, dtype=np.float32) / np.float32(63.0) + np.float32(1.0))[None, :]
    q = np_unpack_nibbles(tfo.quantize_int4(row)[0])
    assert (q == 0).any() and (q == 15).any()


@pytest.mark.parametrize("n", [128, 256, 2816])
def test_roundtrip_within_one_step(tfo, n):
    # DequantInt4GEMVReferenceTests.swift:59-76
    raw = tfo.SeedTree(0xF5).key(f"int4-affine-roundtrip-n{n}").uniform_array(-1.0, 1.0, n)[None, :]
    W, S, B = tfo.quantize_int4(raw)
    rec = tfo.dequantize_int4(W, S, B)
    bound = np.repeat(tfo.bf16_array_to_float(S).reshape(S.shape), 64, axis=1) + 1e-4
    assert np.all(np.abs(rec - raw) <= bound)


def test_roundtrip_amax_bound(tfo):
    # QuantizationTests.swift:8-33
    row = tfo.SeedTree(0x51A71001).key("int4-affine-round-trip").uniform_array(-1.0, 1.0, 256)[None, :]
    W, S, B = tfo.quantize_int4(row)
    rec = tfo.dequantize_int4(W, S, B)
    amax = np.abs(row.reshape(4, 64)).max(axis=1)
    bound = np.repeat(amax / 7.0 + 1e-3, 64)
    assert np.all(np.abs(rec[0] - row[0]) <= bound)


def test_quantizer_rounds_half_away_and_clamps(tfo):
    # scale = 1 (group spans 0..15), so (w - bias) * inv is w itself: x.5 must round away from zero
    row = np.zeros((1, 64), np.float32)
    row[0, :16] = np.arange(16)
    row[0, 16:24] = [0.5, 1.5, 2.5, 3.5, 4.49, 14.5, 13.5, 7.5]
    W, S, B = tfo.quantize_int4(row)
    assert tfo.bf16_to_float(S[0, 0]) == 1.0 and tfo.bf16_to_float(B[0, 0]) == 0.0
    q = np_unpack_nibbles(W)[0]
    assert list(q[16:24]) == [1, 2, 3, 4, 4, 15, 14, 8]
    row8 = np.zeros((1, 64), np.float32)
    row8[0, 0], row8[0, 1], row8[0, 2] = 255.0, 0.5, 254.5
    W8, S8, _ = tfo.quantize_int8(row8)
    assert tfo.bf16_to_float(S8[0, 0]) == 1.0 and list(W8[0, :3]) == [255, 1, 255]


@pytest.mark.parametrize("bits", [4, 8])
def test_dequant_bitexact_vs_numpy_and_f64(tfo, bits):
    rng = np.random.default_rng(5 + bits)
    m, n = 37, 320
    W = rng.integers(0, 256, (m, n // 2 if bits == 4 else n), dtype=np.uint8)
    s = rng.uniform(-0.02, 0.02, (m, n // 64)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, (m, n // 64)).astype(np.float32)
    S, B = tfo.bf16_bits_array(s).reshape(s.shape), tfo.bf16_bits_array(b).reshape(b.shape)
    got = (tfo.dequantize_int4 if bits == 4 else tfo.dequantize_int8)(W, S, B)
    want = np_dequant(W, S, B, bits, tfo)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # float(q)*s is exact, so the fp32 result equals the correctly rounded double expression
    q = (np_unpack_nibbles(W) if bits == 4 else W).astype(np.float64)
    d64 = q * np.repeat(tfo.bf16_array_to_float(S).reshape(S.shape), 64, 1).astype(np.float64) \
        + np.repeat(tfo.bf16_array_to_float(B).reshape(B.shape), 64, 1).astype(np.float64)
    assert np.array_equal(got, d64.astype(np.float32))


@pytest.mark.parametrize("m,n,seed", [(4, 128, 0xF1), (8, 256, 0xF2), (16, 512, 0xF3), (32, 2816, 0xF4)])
def test_gemv_ref_matches_independent_sums(tfo, m, n, seed):
    # DequantInt4GEMVReferenceTests.swift:32-53 shapes/seeds; the fp32 reference must sit within
    # Tolerance.identity of an independently unpacked float64 sum.
    rng = tfo.SeedTree(seed).key(f"int4-gemv-ref-m{m}-n{n}")
    W, S, B = tfo.quantize_int4(rng.uniform_array(-1.0, 1.0, m * n).reshape(m, n))
    x = rng.uniform_array(-1.0, 1.0, n)
    ref = tfo.int4_gemv_ref(W, S, B, x)
    truth = np_dequant(W, S, B, 4, tfo).astype(np.float64) @ x.astype(np.float64)
    assert tfo.rel_error(ref, truth.astype(np.float32)) < tfo.Tolerance.identity
    assert np.allclose(tfo.int4_gemv_f64(W, S, B, x), truth, rtol=1e-12, atol=1e-12)
    assert np.array_equal(tfo.int4_gemv_ref(W, S, B, x, threads=4), ref)


def test_int8_gemv_ref_matches_independent_sums(tfo):
    rng = tfo.SeedTree(0xE1).key("int8-gemv-ref")
    m, n = 16, 512
    W, S, B = tfo.quantize_int8(rng.uniform_array(-1.0, 1.0, m * n).reshape(m, n))
    x = rng.uniform_array(-1.0, 1.0, n)
    truth = np_dequant(W, S, B, 8, tfo).astype(np.float64) @ x.astype(np.float64)
    assert tfo.rel_error(tfo.int8_gemv_ref(W, S, B, x), truth.astype(np.float32)) < tfo.Tolerance.identity
    assert np.allclose(tfo.int8_gemv_f64(W, S, B, x), truth, rtol=1e-12, atol=1e-12)


def test_gemv_all_equal_nibbles_closed_form(tfo):
    # every nibble of a row equal => y = sum_g (q*s_g + b_g) * sum(x_g)
    n, m = 256, 16
    W = np.repeat((np.arange(m, dtype=np.uint8) * 0x11)[:, None], n // 2, axis=1)
    rng = np.random.default_rng(3)
    S = tfo.bf16_bits_array(rng.uniform(0.005, 0.02, (m, 4)).astype(np.float32)).reshape(m, 4)
    B = tfo.bf16_bits_array(rng.uniform(-0.1, 0.1, (m, 4)).astype(np.float32)).reshape(m, 4)
    x = rng.standard_normal(n).astype(np.float32)
    w = np.arange(m, dtype=np.float64)[:, None] * tfo.bf16_array_to_float(S).reshape(m, 4).astype(np.float64) \
        + tfo.bf16_array_to_float(B).reshape(m, 4).astype(np.float64)
    want = (w * x.reshape(4, 64).astype(np.float64).sum(axis=1)[None, :]).sum(axis=1)
    assert np.allclose(tfo.int4_gemv_ref(W, S, B, x), want, rtol=1e-5, atol=1e-5)


def test_kernel_order_gemv_agrees_with_reference(tfo):
    # factored form s*sum(q x) + b*sum(x) == elementwise form (dequant_int4.metal:14-17)
    for m, n, seed in [(128, 128, 0xC1), (64, 64, 0xC3), (33, 704, 0x77), (16, 2816, 0x78)]:
        c = refcases.int4_gemv_case(m, n, seed)
        ref = tfo.int4_gemv_ref(c["W"], c["S"], c["B"], c["x_ref"])
        k = tfo.k_int4_gemv(c["W"], c["S"], c["B"], c["x_bits"])
        assert tfo.rel_error(k, ref) < 2e-5

"""Pins the oracle's scalar codecs and seeded streams against library routines,
published vectors and the reference tests' own known answers."""
import numpy as np
import torch


def test_bf16_encode_matches_torch_rne(tfo):
    rng = np.random.default_rng(1)
    x = np.concatenate([
        rng.standard_normal(200000).astype(np.float32),
        (rng.standard_normal(100000) * 1e-3).astype(np.float32),
        rng.integers(0, 0x7F7FFFFF, 200000, dtype=np.uint32).view(np.float32),   # finite positive patterns
        -rng.integers(0, 0x7F7FFFFF, 100000, dtype=np.uint32).view(np.float32),
        np.array([0.0, -0.0, 1.0, -1.0, 0.5, 1 / 3, 12345.0, 0.42, 65504.0, 1e-40], np.float32),
    ])
    want = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got_vec = tfo.bf16_bits_array(x)
    finite = np.isfinite(torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    assert np.array_equal(got_vec[finite], want[finite])
    # scalar C entry == vectorised formula
    for v in x[::4099]:
        assert tfo.bf16_bits(v) == int(tfo.bf16_bits_array(np.array([v], np.float32))[0])


def test_bf16_reference_known_values(tfo):
    # QuantizationAffineTests.swift:48-58 — rel error < 8e-3 on these literals
    for v in [0.0, 1.0, -1.0, 0.5, -0.5, 1.0 / 3.0, 12345.0]:
        back = tfo.bf16_to_float(tfo.bf16_bits(v))
        assert abs(back - v) / max(abs(v), 1e-6) < 8e-3
    assert tfo.bf16_bits(1.0) == 0x3F80 and tfo.bf16_bits(-0.5) == 0xBF00
    assert tfo.bf16_to_float(0x3F80) == 1.0
    # halfway cases round to even: 1 + 2^-8 is halfway between 0x3F80 and 0x3F81
    assert tfo.bf16_bits(np.float32(1.0 + 2.0 ** -8)) == 0x3F80
    assert tfo.bf16_bits(np.float32(1.0 + 3 * 2.0 ** -8)) == 0x3F82


def test_bf16_decode_is_shift(tfo):
    bits = np.arange(0, 65536, dtype=np.uint32).astype(np.uint16)
    want = (bits.astype(np.uint32) << 16).view(np.float32)
    got = np.array([tfo.bf16_to_float(int(b)) for b in bits[::7]], np.float32)
    ok = ~np.isnan(want[::7])      # NaN payloads do not survive the float->double->float trip through ctypes
    assert np.array_equal(got.view(np.uint32)[ok], want[::7].view(np.uint32)[ok])
    assert np.array_equal(tfo.bf16_array_to_float(bits).view(np.uint32), want.view(np.uint32))


def test_f16_decode_all_patterns_match_numpy(tfo):
    bits = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    want = bits.view(np.float16).astype(np.float32)
    got = np.array([tfo.f16_to_float(int(b)) for b in bits], np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_encode_matches_numpy_rne(tfo):
    rng = np.random.default_rng(2)
    x = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(20000) * 1e-5).astype(np.float32),      # subnormal range
        (rng.standard_normal(5000) * 3e4).astype(np.float32),        # overflow range
        rng.integers(0, 0x7F800000, 20000, dtype=np.uint32).view(np.float32),
        np.array([0.0, -0.0, 65504.0, 65519.99, 65520.0, 2.0 ** -24, 2.0 ** -25, 2.0 ** -25 * 1.0001,
                  2.0 ** -14, 2.0 ** -14 - 2.0 ** -25, np.inf, -np.inf], np.float32),
        # exact halfway points between adjacent halves
        (np.arange(0x3C00, 0x3C40, dtype=np.uint16).view(np.float16).astype(np.float32) + np.float32(2.0 ** -11)),
    ])
    with np.errstate(over="ignore"):
        want = x.astype(np.float16).view(np.uint16)
    got = np.array([tfo.f16_bits(v) for v in x], np.uint16)
    assert np.array_equal(got, want)


def test_splitmix64_published_vectors(tfo):
    g = tfo.SplitMix64(0)
    assert [g.next() for _ in range(3)] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    g = tfo.SplitMix64(1234567)   # Rosetta Code "Pseudo-random numbers/Splitmix64"
    assert [g.next() for _ in range(5)] == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                            4593380528125082431, 16408922859458223821]


def test_uniform_closed_form(tfo):
    # SplitMix64.swift:20-23: lo + (hi-lo) * Float(next >> 40) / 2^24, all in fp32
    a, b = tfo.SplitMix64(0xA5B61234), tfo.SplitMix64(0xA5B61234)
    for lo, hi in [(-0.05, 0.05), (-1.0, 1.0), (0.5, 1.5), (0.005, 0.02)]:
        for _ in range(50):
            u = np.float32(a.next() >> 40) / np.float32(1 << 24)
            want = np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u
            assert np.float32(b.uniform(lo, hi)) == want
    arr = tfo.SplitMix64(7).uniform_array(-1, 1, 1000)
    g = tfo.SplitMix64(7)
    assert np.array_equal(arr, np.array([g.uniform(-1, 1) for _ in range(1000)], np.float32))
    assert arr.min() >= -1 and arr.max() < 1


def test_seedtree_fnv1a_vectors(tfo):
    # FNV-1a 64 published test vectors (offset basis, "a", "foobar"); key = root ^ hash
    assert tfo.SeedTree(0).key_state("") == 0xCBF29CE484222325
    assert tfo.SeedTree(0).key_state("a") == 0xAF63DC4C8601EC8C
    assert tfo.SeedTree(0).key_state("foobar") == 0x85944171F73967E8
    assert tfo.SeedTree(0xFF).key_state("a") == 0xAF63DC4C8601EC8C ^ 0xFF
    # the stream DequantInt4GEMVTests.gemv_m1024_n2816 draws from
    assert tfo.SeedTree(0xC2).key_state("int4-gemv-kernel-m1024-n2816") == 0xA38BB6725F0AC119

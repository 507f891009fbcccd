"""Pins the CPU restatement of the output head's neighbours: embedding row lookup, soft-capped softmax and the samplers.
Known answers where the reference's tests give them, library routines (torch softmax / tanh), closed forms, and for the
samplers the statistics the mathematics fixes: draw frequencies must follow p^(1/T) restricted to the surviving set."""
import numpy as np
import torch

from oracle import tfo


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16).view(np.uint16)


def test_embed_lookup_is_the_dequantized_row_times_the_scale():
    # EmbedLookupTests.swift:16-77: V=16, D=128, token 9, scale sqrt(D); and scale 1 == raw dequant
    rng = tfo.SeedTree(0x131).key("embed-lookup-int4-table")
    W, S, B = tfo.quantize_int4(rng.uniform_array(-1.0, 1.0, 16 * 128).reshape(16, 128))
    full = tfo.dequantize_int4(W, S, B)
    assert np.array_equal(tfo.embed_lookup_int4(W, S, B, 9, 1.0), full[9])
    scale = float(np.sqrt(np.float32(128)))
    assert np.array_equal(tfo.embed_lookup_int4(W, S, B, 9, scale), (full[9] * np.float32(scale)).astype(np.float32))
    assert np.array_equal(tfo.embed_lookup_int4(W, S, B, 0, 1.0), full[0]) and np.array_equal(tfo.embed_lookup_int4(W, S, B, 15, 1.0), full[15])


def test_softcap_softmax_matches_torch_and_the_reference_tests_cases():
    # LogitSoftcapSoftmaxTests.swift:34-89
    rng = tfo.SeedTree(0x131).key("softcap-softmax-random")
    x = tfo.from_f16_bits(f16(rng.uniform_array(-50.0, 50.0, 2048)))
    got = tfo.logit_softcap_softmax_ref(x, 30.0)
    want = torch.softmax(30.0 * torch.tanh(torch.from_numpy(x).double() / 30.0), dim=0).numpy()
    assert np.max(np.abs(got - want)) < 1e-7 and abs(float(got.sum()) - 1.0) < 1e-5
    uniform = tfo.logit_softcap_softmax_ref(np.full(2048, np.float32(np.float16(0.1234))), 30.0)
    assert np.max(np.abs(uniform - 1.0 / 2048)) < 1e-9
    spike = np.zeros(2048, np.float32)
    spike[42] = 1000.0
    capped = tfo.logit_softcap_softmax_ref(spike, 5.0)
    closed = np.exp(5.0) / (np.exp(5.0) + 2047.0)        # tanh(200) == 1: the outlier sits exactly at the cap
    assert capped[42] < 0.5 and abs(capped[42] - closed) / closed < 1e-4


def test_generators_are_the_published_ones():
    # xorshift64* (Vigna): shifts 13/7/17 then the multiplier, checked against plain integer arithmetic
    mask = (1 << 64) - 1
    for seed in (1, 42, 0xDEADBEEFCAFEF00D, mask):
        s = seed
        s ^= (s << 13) & mask
        s ^= s >> 7
        s ^= (s << 17) & mask
        assert tfo.sampler_xorshift64(seed) == ((s * 2685821657736338717) & mask, s)
    # Gumbel noise: -log(-log(u)) with u strictly inside (0, 1): finite, mean = Euler-Mascheroni, variance = pi^2 / 6
    g = np.array([tfo.sampler_gumbel(0x1234, 3, r) for r in range(40000)])
    assert np.all(np.isfinite(g)) and abs(g.mean() - 0.5772) < 0.02 and abs(g.var() - np.pi ** 2 / 6) < 0.06
    assert tfo.sampler_gumbel(7, 0, 5) != tfo.sampler_gumbel(7, 1, 5) != tfo.sampler_gumbel(8, 1, 5)


def _frequencies(draw, n, v):
    counts = np.zeros(v)
    for t in range(n):
        counts[draw((t + 1) * 0x9E3779B97F4A7C15 & ((1 << 64) - 1))] += 1
    return counts / n


def test_greedy_and_known_answers_of_the_reference_tests():
    values = np.full(2048, 0.01, np.float32)
    values[1337] = 5.0
    probs = f16(values / values.sum())
    assert tfo.sample(probs, 0.0, 0, 1.0, 1) == 1337                                   # SampleTests.swift:52-65
    tie = f16(np.array([0.1, 0.4, 0.4, 0.1]))
    assert tfo.sample(tie, 0.0, 0, 1.0, 1) == 1                                        # lowest index among equals
    rng = tfo.SeedTree(0x51A71003).key("sample-seeded-determinism")
    p = f16(rng.uniform_array(0.0, 1.0, 1024) / 512.0)
    seed = 0xDEADBEEFCAFEF00D
    assert tfo.sample(p, 1.0, 0, 1.0, seed) == tfo.sample(p, 1.0, 0, 1.0, seed)         # :67-94
    assert len({tfo.sample(p, 1.0, 0, 1.0, s) for s in (42, 1337, 0xAABBCCDD, 0xFFFEDCBA)}) > 1


def test_truncating_sampler_draws_from_the_surviving_reweighted_set():
    p = np.array([0.05, 0.30, 0.02, 0.25, 0.20, 0.10, 0.08], np.float32)
    bits = f16(p)
    pf = tfo.from_f16_bits(bits).astype(np.float64)
    n = 6000
    # top-k 4 at T = 1: indices 1, 3, 4, 5 with their own masses renormalised
    freq = _frequencies(lambda s: tfo.sample(bits, 1.0, 4, 1.0, s), n, p.size)
    want = np.zeros(p.size)
    keep = [1, 3, 4, 5]
    want[keep] = pf[keep] / pf[keep].sum()
    assert np.all(freq[[0, 2, 6]] == 0) and np.max(np.abs(freq - want)) < 0.03
    # top-p 0.7 against the full distribution: 0.30 + 0.25 + 0.20 >= 0.7 -> three survivors; then T = 0.5 squares them
    freq = _frequencies(lambda s: tfo.sample(bits, 0.5, 0, 0.7, s), n, p.size)
    want = np.zeros(p.size)
    keep = [1, 3, 4]
    want[keep] = pf[keep] ** 2 / (pf[keep] ** 2).sum()
    assert np.max(np.abs(freq - want)) < 0.03
    # the top-64 sampler is the same chain with k = 64 (SampleTopK64Tests.swift:84-131)
    for seed in range(1, 40):
        assert tfo.sample_topk64(bits, 0.85, 0.95, seed) == tfo.sample(bits, 0.85, 64, 0.95, seed)
    ones = f16(np.ones(1003))
    assert all(tfo.sample_topk64(ones, 1.0, 0.95, s) < 64 for s in range(1, 9))        # ties resolve to the lowest indices
    flat = f16(np.full(1003, 1.0 / 1003.0))
    picks = [tfo.sample_topk64(flat, 1.0, 0.95, s) for s in range(1, 257)]
    assert max(picks) >= 61 and max(picks) < 64                                        # top-p uses the full-vocabulary mass (:113-131)


def test_gumbel_path_draws_from_p_to_the_one_over_t():
    p = np.array([0.05, 0.30, 0.02, 0.25, 0.20, 0.10, 0.08], np.float32)
    bits = f16(p)
    pf = tfo.from_f16_bits(bits).astype(np.float64)
    for temperature in (1.0, 0.5):
        freq = _frequencies(lambda s: tfo.sample(bits, temperature, 0, 1.0, s), 6000, p.size)
        want = pf ** (1.0 / temperature) / (pf ** (1.0 / temperature)).sum()
        assert np.max(np.abs(freq - want)) < 0.03
    with_zero = f16(np.array([0.0, 0.5, 0.5, 0.0]))
    assert all(tfo.sample(with_zero, 1.0, 0, 1.0, s) in (1, 2) for s in range(1, 50))   # p == 0 is never drawn
    assert tfo.sample(bits, 1.0, 0, 1.0, 5, position=0) == tfo.sample(bits, 1.0, 0, 1.0, 5, position=0)
    assert len({tfo.sample(bits, 1.0, 0, 1.0, 5, position=q) for q in range(40)}) > 1   # the position enters the noise

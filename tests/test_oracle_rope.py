"""Pins the RoPE / Q-K-V epilogue part of the oracle by what the mathematics fixes: a rotation preserves every pair's
norm, angle 0 is the identity, rotations compose additively in the position for the lowest frequency, untouched pairs
pass through, numpy's complex arithmetic gives the same numbers; the epilogue equals per-head RMSNorm followed by RoPE.
CPU only."""
import numpy as np
import pytest

from oracle import tfo


def rand(n, seed):
    return tfo.SeedTree(seed).key("rope").uniform_array(-1.0, 1.0, n)


@pytest.mark.parametrize("tokens,heads,d,pairs,position,theta", [(1, 16, 256, 128, 7, 1e4), (1, 16, 512, 64, 11, 1e6), (3, 2, 64, 10, 4097, 1e4)])
def test_rope_ref_equals_complex_rotation(tokens, heads, d, pairs, position, theta):
    x = rand(tokens * heads * d, 0xF1)
    got = tfo.rope_neox_ref(x, tokens, heads, d, pairs, position, theta).reshape(tokens * heads, d)
    xs = x.reshape(tokens * heads, d).astype(np.float64)
    z = xs[:, :d // 2] + 1j * xs[:, d // 2:]
    k = np.arange(d // 2)
    angle = position * np.power(float(theta), -2.0 * k / d)
    rot = np.where(k < pairs, np.exp(1j * angle), 1.0)
    want = z * rot
    assert np.allclose(got[:, :d // 2], want.real, atol=2e-6) and np.allclose(got[:, d // 2:], want.imag, atol=2e-6)
    # norms of pairs are preserved, untouched pairs are bit-identical
    assert np.allclose(got[:, :d // 2] ** 2 + got[:, d // 2:] ** 2, xs[:, :d // 2] ** 2 + xs[:, d // 2:] ** 2, atol=1e-5)
    assert np.array_equal(got[:, pairs:d // 2], x.reshape(-1, d)[:, pairs:d // 2])


def test_rope_identity_and_composition():
    d, heads = 64, 3
    x = rand(heads * d, 0xF2)
    assert np.array_equal(tfo.rope_neox_ref(x, 1, heads, d, d // 2, 0, 1e4), x)
    # pair 0 has frequency 1: position a then position b == position a + b
    once = tfo.rope_neox_ref(x, 1, heads, d, 1, 5, 1e4)
    twice = tfo.rope_neox_ref(tfo.rope_neox_ref(x, 1, heads, d, 1, 2, 1e4), 1, heads, d, 1, 3, 1e4)
    assert np.allclose(once, twice, atol=1e-6)


def test_kernel_order_rope_tracks_the_reference():
    # RoPETests.swift:7-46, 48-99: fp16 data, tolerance fp16Reduction
    for tokens, heads, d, pairs, position, theta, seed in ((1, 16, 256, 128, 7, 1e4, 0xF1), (1, 16, 512, 64, 11, 1e6, 0xF3)):
        bits = tfo.to_f16_bits(rand(tokens * heads * d, seed))
        got = tfo.from_f16_bits(tfo.k_rope_neox(bits, tokens, heads, d, pairs, position, theta))
        ref = tfo.rope_neox_ref(tfo.from_f16_bits(bits), tokens, heads, d, pairs, position, theta)
        assert tfo.rel_error(got, ref) < tfo.Tolerance.fp16Reduction
        assert np.array_equal(got.reshape(-1, d)[:, pairs:d // 2], tfo.from_f16_bits(bits).reshape(-1, d)[:, pairs:d // 2])


def test_epilogue_is_per_head_rmsnorm_then_rope():
    # FusedQKVEpilogueTests.swift:28-147 compares with the chain of separate kernels; here the chain is numpy + the rope restatement
    d, nq, nkv, pairs, position, theta, eps = 256, 16, 8, 128, 9, 1e4, 1e-6
    q, k, v = (tfo.to_f16_bits(rand(n * d, s)) for n, s in ((nq, 1), (nkv, 2), (nkv, 3)))
    wq = tfo.bf16_bits_array(1.0 + 0.1 * rand(d, 4))
    wk = tfo.bf16_bits_array(1.0 + 0.1 * rand(d, 5))
    gq, gk, gv = tfo.k_fused_qkv_epilogue(q, k, v, wq, wk, d, nq, nkv, position, theta, pairs, eps)

    def norm(bits, w):
        x = tfo.from_f16_bits(bits).reshape(-1, d).astype(np.float64)
        y = x / np.sqrt((x * x).mean(axis=1, keepdims=True) + eps)
        if w is not None:
            y = y * tfo.bf16_array_to_float(w).astype(np.float64)
        return y.astype(np.float32)
    for got, bits, w, heads in ((gq, q, wq, nq), (gk, k, wk, nkv)):
        chain = tfo.rope_neox_ref(tfo.from_f16_bits(tfo.to_f16_bits(norm(bits, w).reshape(-1))), 1, heads, d, pairs, position, theta)
        assert tfo.rel_error(tfo.from_f16_bits(got), chain) < tfo.Tolerance.fp16Reduction
    assert np.max(np.abs(tfo.from_f16_bits(gv) - norm(v, None).reshape(-1))) <= 2e-3      # one fp16 rounding of values below 4
    # a normalized head has unit mean square (v: exactly the definition)
    ms = (tfo.from_f16_bits(gv).reshape(nkv, d).astype(np.float64) ** 2).mean(axis=1)
    assert np.allclose(ms, 1.0, atol=2e-3)

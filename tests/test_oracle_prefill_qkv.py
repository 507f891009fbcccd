"""Pins of the oracle's row-grid RMSNorm restatement (rmsnorm_no_scale / *_perhead and their prefill block twins): closed
forms in float64, row independence, untouched padding (PrefillPerHeadNormTests.swift shapes)."""
import numpy as np
import pytest

from oracle import tfo

EPS = 1e-6


def block(tokens, heads, d, pad, seed):
    rng = np.random.default_rng(seed)
    stride = heads * d + pad
    x = tfo.to_f16_bits(rng.standard_normal(tokens * stride).astype(np.float32))
    w = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, d).astype(np.float32))
    return x, w, stride


def closed_form(x_bits, w_bits, tokens, heads, d, stride):
    """x / sqrt(mean(x^2) + eps) [* w] per head in float64."""
    x = tfo.from_f16_bits(x_bits).astype(np.float64).reshape(tokens, stride)[:, :heads * d].reshape(tokens, heads, d)
    inv = 1.0 / np.sqrt(np.mean(x * x, axis=2, keepdims=True) + EPS)
    y = x * inv
    if w_bits is not None:
        y = y * tfo.bf16_array_to_float(w_bits).astype(np.float64)
    return y


@pytest.mark.parametrize("tokens,heads,d,pad", [(3, 16, 256, 23), (3, 8, 256, 23), (2, 16, 512, 23), (2, 2, 512, 23), (1, 1, 2816, 0), (4, 3, 40, 1)])
@pytest.mark.parametrize("weighted", [True, False])
def test_rows_match_the_closed_form_and_leave_padding_alone(tokens, heads, d, pad, weighted):
    x, w, stride = block(tokens, heads, d, pad, 0xB500 + d + heads)
    out = tfo.k_rmsnorm_rows(x, w if weighted else None, EPS, tokens, heads, d, stride)
    got = tfo.from_f16_bits(out).reshape(tokens, stride)
    want = closed_form(x, w if weighted else None, tokens, heads, d, stride)
    used = got[:, :heads * d].reshape(tokens, heads, d)
    assert np.max(np.abs(used - want)) <= 2.0 ** -10 * max(1.0, float(np.max(np.abs(want))))      # one fp16 rounding of the exact value
    assert np.array_equal(out.reshape(tokens, stride)[:, heads * d:], x.reshape(tokens, stride)[:, heads * d:])


def test_rows_are_independent_and_equal_the_single_row_routine():
    tokens, heads, d, pad = 3, 4, 64, 5
    x, w, stride = block(tokens, heads, d, pad, 0xB510)
    out = tfo.k_rmsnorm_rows(x, w, EPS, tokens, heads, d, stride)
    for t in range(tokens):
        for h in range(heads):
            at = t * stride + h * d
            assert np.array_equal(out[at:at + d], tfo.k_rmsnorm_bf16w(x[at:at + d], w, EPS))
    # changing one head changes only that head
    x2 = x.copy()
    x2[stride + d:stride + 2 * d] = tfo.to_f16_bits(np.full(d, 3.0, np.float32))
    out2 = tfo.k_rmsnorm_rows(x2, w, EPS, tokens, heads, d, stride)
    same = np.ones(out.size, bool)
    same[stride + d:stride + 2 * d] = False
    assert np.array_equal(out[same], out2[same])


def test_known_answers_without_scale():
    # a constant head c normalises to sign(c) (eps negligible); a head of zeros stays zero; scaling the input by 2 changes nothing
    d = 128
    for c in (0.5, -3.0):
        out = tfo.from_f16_bits(tfo.k_rmsnorm_rows(tfo.to_f16_bits(np.full(d, c, np.float32)), None, EPS, 1, 1, d, d))
        assert np.allclose(out, np.sign(c), atol=2e-3)
    assert np.all(tfo.from_f16_bits(tfo.k_rmsnorm_rows(np.zeros(d, np.uint16), None, EPS, 1, 1, d, d)) == 0.0)
    rng = np.random.default_rng(7)
    x = rng.standard_normal(d).astype(np.float32)
    a = tfo.k_rmsnorm_rows(tfo.to_f16_bits(x), None, EPS, 1, 1, d, d)
    b = tfo.k_rmsnorm_rows(tfo.to_f16_bits(2.0 * x), None, EPS, 1, 1, d, d)      # doubling is exact in fp16
    assert np.max(np.abs(a.astype(np.int32) - b.astype(np.int32))) <= 1

"""GPU parity of RoPE and the fused Q/K/V epilogue through the C ABI against the oracle (RoPETests.swift,
FusedQKVEpilogueTests.swift shapes)."""
import numpy as np
import pytest

from gpu_helpers import ctx, dev, host, tfk
from oracle import tfo
from test_oracle_rope import rand

pytestmark = pytest.mark.gpu


def same_up_to_rounding(got_bits, want_bits, ulps=2, share=0.02):
    """The two sides evaluate pow / cos / sin with different libraries: a result may land on the neighbouring fp16 value."""
    a, b = tfo.from_f16_bits(got_bits).astype(np.float64), tfo.from_f16_bits(want_bits).astype(np.float64)
    step = np.maximum(np.abs(b), 1.0) * 2.0 ** -10        # a rotated value's error scales with the pair's size, not with its own
    diff = np.abs(a - b)
    assert np.all(diff <= ulps * step), float(np.max(diff / step))
    assert np.mean(diff > 0) <= share, float(np.mean(diff > 0))


@pytest.mark.parametrize("tokens,heads,d,pairs,position,theta,seed", [(1, 16, 256, None, 7, 1e4, 0xF1),       # defaultNeoxMatchesSWAReference
                                                                      (1, 16, 512, 64, 11, 1e6, 0xF3),      # proportionalNeoxMatchesFullAttentionReference
                                                                      (1, 2, 512, 64, 11, 1e6, 0xF4),
                                                                      (5, 3, 64, 10, 100003, 1e4, 0xF5),    # several tokens, a large position
                                                                      (1, 4, 128, 0, 3, 1e4, 0xF6)])        # nothing rotates
def test_rope_matches_the_reference(tokens, heads, d, pairs, position, theta, seed):
    bits = tfo.to_f16_bits(rand(tokens * heads * d, seed))
    k = ctx()
    data = dev(np.concatenate([np.zeros(3, np.uint16), bits]))         # a 6-byte offset
    if pairs is None:
        k.check(k.lib.tf_rope_default_neox(k.handle, None, data.data_ptr(), 6, position, d, heads, tokens, theta))
        pairs = d // 2
    else:
        k.check(k.lib.tf_rope_proportional_neox(k.handle, None, data.data_ptr(), 6, position, d, heads, tokens, pairs, theta))
    got = host(data, np.uint16)[3:]
    ref = tfo.rope_neox_ref(tfo.from_f16_bits(bits), tokens, heads, d, pairs, position, theta)
    if position < 4096:
        assert tfo.rel_error(tfo.from_f16_bits(got), ref) < tfo.Tolerance.fp16Reduction
        same_up_to_rounding(got, tfo.k_rope_neox(bits, tokens, heads, d, pairs, position, theta))
    else:
        # an fp32 angle near 1e5 carries 4e-3 rad of rounding (and one ulp of pow moves it by as much): both sides are
        # that far from the exact rotation, and from each other; what a rotation preserves must still hold exactly enough
        assert tfo.rel_error(tfo.from_f16_bits(got), ref) < tfo.Tolerance.fp16ChainedReduction
        g = tfo.from_f16_bits(got).reshape(-1, d).astype(np.float64)
        x = tfo.from_f16_bits(bits).reshape(-1, d).astype(np.float64)
        assert np.allclose(g[:, :d // 2] ** 2 + g[:, d // 2:] ** 2, x[:, :d // 2] ** 2 + x[:, d // 2:] ** 2, atol=4e-3)
    # what does not rotate is untouched (RoPETests.swift:88-98)
    assert np.array_equal(got.reshape(-1, d)[:, pairs:d // 2], bits.reshape(-1, d)[:, pairs:d // 2])
    assert np.array_equal(got.reshape(-1, d)[:, d // 2 + pairs:], bits.reshape(-1, d)[:, d // 2 + pairs:])


@pytest.mark.parametrize("d,nq,nkv,pairs,position,theta", [(256, 16, 8, 128, 9, 1e4), (512, 16, 2, 64, 1234, 1e6), (64, 4, 2, 7, 5, 1e4)])
def test_fused_qkv_epilogue(d, nq, nkv, pairs, position, theta):
    eps = 1e-6
    q, kk, v = (tfo.to_f16_bits(rand(n * d, s)) for n, s in ((nq, 11), (nkv, 12), (nkv, 13)))
    wq, wk = tfo.bf16_bits_array(1.0 + 0.1 * rand(d, 14)), tfo.bf16_bits_array(1.0 + 0.1 * rand(d, 15))
    k = ctx()
    t = dict(q=dev(q), k=dev(kk), v=dev(v), wq=dev(wq), wk=dev(wk))
    k.check(k.lib.tf_fused_qkv_epilogue(k.handle, None, t["q"].data_ptr(), 0, t["k"].data_ptr(), 0, t["v"].data_ptr(), 0, t["wq"].data_ptr(), 0,
                                        t["wk"].data_ptr(), 0, d, nq, nkv, position, theta, pairs, eps))
    want = tfo.k_fused_qkv_epilogue(q, kk, v, wq, wk, d, nq, nkv, position, theta, pairs, eps)
    for name, w in zip(("q", "k", "v"), want):
        got = host(t[name], np.uint16)
        assert tfo.rel_error(tfo.from_f16_bits(got), tfo.from_f16_bits(w)) < tfo.Tolerance.fp16Reduction, name
        same_up_to_rounding(got, w, ulps=2, share=0.05)


def test_contract():
    k = ctx()
    data = dev(np.zeros(512, np.uint16))
    bad = tfk.TF_ERR_INVALID_ARGUMENT
    assert k.lib.tf_rope_default_neox(k.handle, None, data.data_ptr(), 0, 1, 63, 1, 1, 1e4) == bad            # RoPE.swift:35
    assert k.lib.tf_rope_proportional_neox(k.handle, None, data.data_ptr(), 0, 1, 64, 1, 1, 33, 1e4) == bad   # :66-67
    assert k.lib.tf_rope_proportional_neox(k.handle, None, data.data_ptr(), 0, 1, 64, 1, 0, 8, 1e4) == tfk.TF_OK
    w = dev(np.zeros(1024, np.uint16))
    args = (data.data_ptr(), 0, data.data_ptr(), 0, data.data_ptr(), 0, w.data_ptr(), 0, w.data_ptr(), 0)
    assert k.lib.tf_fused_qkv_epilogue(k.handle, None, *args, 514, 1, 1, 0, 1e4, 4, 1e-6) == bad              # FusedQKVEpilogue.swift:60-61
    assert k.lib.tf_fused_qkv_epilogue(k.handle, None, *args, 64, 1, 1, 0, 1e4, 33, 1e-6) == bad              # :62-63

"""GPU parity: tied int4 output head (greedy argmax and logits) through the C ABI against the CPU oracle.
Cases restate Tests/TurboFieldfare/Core/Kernels/Fusions/LMHeadChainInt4Tests.swift."""
import numpy as np
import pytest

import refcases
from gpu_helpers import ctx, dev, host, tfk, within_north_star, zeros_bytes
from oracle import tfo

pytestmark = pytest.mark.gpu
ONE = lambda d: tfo.bf16_bits_array(np.ones(d, np.float32))


def gpu_greedy(hidden_bits, norm_bits, W, S, B, hidden_offset=0, w_off=0):
    v, d = W.shape[0], W.shape[1] * 2
    out = zeros_bytes(4, 0xEE)
    ctx().lm_head_greedy(dev(hidden_bits), dev(norm_bits), dev(W, w_off), dev(S), dev(B), out, d, v,
                         hidden_offset=hidden_offset, weights_offset=w_off)
    return int(host(out, np.uint32, 1)[0])


def test_raw_greedy_matches_cpu_reference():
    hidden_bits, norm_bits, W, S, B = refcases.lm_head_random_case()
    assert gpu_greedy(hidden_bits, norm_bits, W, S, B) == tfo.lm_head_cpu_greedy(hidden_bits, norm_bits, W, S, B)


def test_all_invalid_candidates_fall_back_to_zero():
    d, v = 64, 1024
    W, S, B = tfo.quantize_int4(np.full((v, d), 0.25, np.float32))
    assert gpu_greedy(np.full(d, 0x7E00, np.uint16), ONE(d), W, S, B) == 0


@pytest.mark.parametrize("v", [1024, 2048, 4096])
def test_greedy_matches_cpu_reference_across_vocab_sizes(v):
    d = 64
    hidden = tfo.to_f16_bits(np.float32(0.25) + (np.arange(d) % 7).astype(np.float32) * np.float32(0.01))
    W, S, B = refcases.lm_head_constant_rows(d, v, [v - 3])
    ref = tfo.lm_head_cpu_greedy(hidden, ONE(d), W, S, B)
    assert ref == v - 3 and gpu_greedy(hidden, ONE(d), W, S, B) == ref


def test_ties_resolve_to_lowest_index():
    d, v = 64, 1024
    hidden = tfo.to_f16_bits(np.float32(0.2) + (np.arange(d) % 5).astype(np.float32) * np.float32(0.02))
    W, S, B = refcases.lm_head_constant_rows(d, v, [17, 311], hot=1.0, cold=-0.25)
    assert gpu_greedy(hidden, ONE(d), W, S, B) == 17


def test_reads_selected_hidden_row():
    d, v, stride, sel, target = 64, 1024, 80, 3, 777
    rows = np.zeros(5 * stride, np.float32)
    for r in range(5):
        idx = np.arange(d)
        rows[r * stride:r * stride + d] = (0.25 + (idx % 7) * 0.01) if r == sel else (-0.4 - (idx % 5) * 0.01)
    W, S, B = refcases.lm_head_constant_rows(d, v, [target], hot=1.0, cold=-0.25)
    assert gpu_greedy(tfo.to_f16_bits(rows), ONE(d), W, S, B, hidden_offset=sel * stride * 2) == target


@pytest.mark.parametrize("v,w_off", [(4096, 0), (4099, 0), (3000, 2)])
def test_greedy_and_logits_at_production_width(v, w_off):
    # d = 2816 rows take the streaming kernel (16-byte aligned) or the 16-bit-load path (+2 offset)
    d = 2816
    W, S, B = refcases.synthetic_int4(v, d, 0x1ead + v)
    hidden_bits = refcases.normal_f16(d, 0x1ead)
    norm_bits = tfo.bf16_bits_array(np.random.default_rng(1).uniform(0.5, 1.5, d).astype(np.float32))
    tok_ref, logits_ref = tfo.lm_head_cpu_greedy(hidden_bits, norm_bits, W, S, B, threads=8, want_logits=True)
    assert gpu_greedy(hidden_bits, norm_bits, W, S, B, w_off=w_off) == tok_ref
    if w_off == 0:
        for od, np_dt in ((tfk.TF_FP32, np.float32), (tfk.TF_FP16, np.uint16)):
            out = zeros_bytes(v * 4)
            ctx().lm_head_logits(dev(hidden_bits), dev(norm_bits), dev(W), dev(S), dev(B), out, d, v, out_dtype=od)
            got = host(out, np_dt, v)
            got = got if od == tfk.TF_FP32 else tfo.from_f16_bits(got)
            assert tfo.rel_error(got, logits_ref) < tfo.Tolerance.fp16Reduction
            assert within_north_star(got, logits_ref, abs_=2e-3)


def test_ties_and_nonfinite_rows_at_production_width():
    d, v = 2816, 5000
    W, S, B = refcases.synthetic_int4(v, d, 0x7135)
    # rows 1234 and 4321 become identical copies of the current winner pattern: the lower index must win
    W[1234], S[1234], B[1234] = 0xFF, tfo.bf16_bits(0.02), tfo.bf16_bits(0.1)
    W[4321], S[4321], B[4321] = W[1234], S[1234], B[1234]
    hidden_bits = tfo.to_f16_bits(np.abs(tfo.from_f16_bits(refcases.normal_f16(d, 5))) + 0.1)   # all positive: all-15 rows win
    assert gpu_greedy(hidden_bits, ONE(d), W, S, B) == 1234
    assert tfo.lm_head_cpu_greedy(hidden_bits, ONE(d), W, S, B, threads=8) == 1234
    # a row whose scale is +inf produces a non-finite logit and must be skipped
    S2 = S.copy()
    S2[1234, 0] = 0x7F80
    assert gpu_greedy(hidden_bits, ONE(d), W, S2, B) == 4321


def test_head_rejects_bad_contract():
    d, v = 64, 128
    W, S, B = tfo.quantize_int4(np.zeros((v, d), np.float32))
    k = ctx()
    out = zeros_bytes(4)
    args = (dev(np.zeros(d, np.uint16)), dev(ONE(d)), dev(W, 1), dev(S), dev(B), out)
    assert k.lm_head_greedy(*args, d, v, weights_offset=1, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT   # LMHeadChainInt4.swift:74-75
    assert k.lm_head_greedy(*args, 96, v, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT                    # :71-72

"""GPU parity: dequantization (bit-exact) and the int4/int8 GEMV, through the C ABI, against the CPU oracle.
Cases restate Tests/TurboFieldfare/Core/Kernels/Quant/DequantInt4GEMVTests.swift plus the BASELINE shapes."""
import numpy as np
import pytest

import refcases
from gpu_helpers import ctx, dev, host, tfk, within_north_star, zeros_bytes
from oracle import tfo

pytestmark = pytest.mark.gpu


def run_gemv(W, S, B, x_bits, scale_dtype=tfk.TF_BF16, out_dtype=tfk.TF_FP16, w_off=0, bits=4, x_off=0):
    m = W.shape[0]
    n = W.shape[1] * (2 if bits == 4 else 1)
    dW, dS, dB, dx = dev(W, w_off), dev(S), dev(B), dev(x_bits, x_off)
    y = zeros_bytes(m * (2 if out_dtype == tfk.TF_FP16 else 4) + 64, 0xEE)
    ctx().dequant_int4_gemv(dW, dS, dB, dx, y, m, n, scale_dtype, out_dtype, offsets=(w_off, 0, 0, x_off, 0), bits=bits)
    if out_dtype == tfk.TF_FP16:
        out = tfo.from_f16_bits(host(y, np.uint16, m))
    else:
        out = host(y, np.float32, m)
    tail = host(y, np.uint8)[m * (2 if out_dtype == tfk.TF_FP16 else 4):]
    assert np.all(tail == 0xEE), "kernel wrote past y"
    return out


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("sd", ["bf16", "fp16"])
def test_dequantize_is_bit_exact(bits, sd):
    rng = np.random.default_rng(11 + bits)
    m, n = 67, 2816
    W = rng.integers(0, 256, (m, n // 2 if bits == 4 else n), dtype=np.uint8)
    s = rng.uniform(-0.02, 0.02, (m, n // 64)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, (m, n // 64)).astype(np.float32)
    if sd == "bf16":
        S, B = tfo.bf16_bits_array(s).reshape(s.shape), tfo.bf16_bits_array(b).reshape(b.shape)
        want = (tfo.dequantize_int4 if bits == 4 else tfo.dequantize_int8)(W, S, B)
    else:
        S, B = s.astype(np.float16).view(np.uint16), b.astype(np.float16).view(np.uint16)
        q = W.astype(np.float32)
        if bits == 4:
            q = np.empty((m, n), np.float32)
            q[:, 0::2], q[:, 1::2] = W & 0x0F, W >> 4
        want = q * np.repeat(S.view(np.float16).astype(np.float32), 64, 1) + np.repeat(B.view(np.float16).astype(np.float32), 64, 1)
    out = zeros_bytes(m * n * 4)
    # weights bound at an odd-word (+2) offset, as in the resident layout
    ctx().dequantize_int4(dev(W, 2), dev(S), dev(B), out, m, n, tfk.TF_BF16 if sd == "bf16" else tfk.TF_FP16, offsets=(2, 0, 0, 0), bits=bits)
    got = host(out, np.float32, m * n).reshape(m, n)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


def check_case(c, rel_tol=tfo.Tolerance.fp16Reduction, w_off=0):
    ref = tfo.int4_gemv_ref(c["W"], c["S"], c["B"], c["x_ref"])
    got16 = run_gemv(c["W"], c["S"], c["B"], c["x_bits"], w_off=w_off)
    assert tfo.rel_error(got16, ref) < rel_tol
    assert within_north_star(got16, ref)
    got32 = run_gemv(c["W"], c["S"], c["B"], c["x_bits"], out_dtype=tfk.TF_FP32, w_off=w_off)
    truth = tfo.int4_gemv_f64(c["W"], c["S"], c["B"], c["x_ref"])
    # fp32 accumulation, exact products: only summation-order noise separates the device from the double sum
    assert np.max(np.abs(got32 - truth)) <= 2e-5 * max(1.0, float(np.max(np.abs(truth))))
    # rounding the fp32 result to fp16 is what the fp16 entry returns
    assert np.array_equal(tfo.to_f16_bits(got32), tfo.to_f16_bits(got16))


def test_gemv_d128_n128():
    check_case(refcases.int4_gemv_case(128, 128, 0xC1))


def test_gemv_m1024_n2816():
    check_case(refcases.int4_gemv_case(1024, 2816, 0xC2))


def test_gemv_m64_n64():
    check_case(refcases.int4_gemv_case(64, 64, 0xC3))


def test_gemv_weights_at_2_aligned_not_4_aligned_offset():
    # DequantInt4GEMVTests.swift:113-121
    check_case(refcases.int4_gemv_case(128, 2816, 0xC4, weight_byte_offset=2), w_off=2)


@pytest.mark.parametrize("m", [64, 65, 128, 129])
@pytest.mark.parametrize("n", [64, 128, 192, 256, 320, 512])
def test_gemv_sweep(m, n):
    # DequantInt4GEMVTests.swift:123-128
    check_case(refcases.int4_gemv_case(m, n, (m * 0x9E37 + n) & 0xFFFFFFFFFFFFFFFF))


@pytest.mark.parametrize("m,n", [(33, 704), (7, 1024), (129, 1088), (50, 1536), (131, 2112), (9, 2816), (66, 4096), (35, 8192), (5, 8256)])
def test_gemv_production_and_ragged_shapes(m, n):
    check_case(refcases.int4_gemv_case(m, n, 0xD00 + m + n))


def test_gemv_unaligned_activation_falls_back():
    c = refcases.int4_gemv_case(70, 2816, 0xD5)
    ref = tfo.int4_gemv_ref(c["W"], c["S"], c["B"], c["x_ref"])
    got = run_gemv(c["W"], c["S"], c["B"], c["x_bits"], x_off=6)
    assert tfo.rel_error(got, ref) < tfo.Tolerance.fp16Reduction


@pytest.mark.parametrize("sd", ["bf16", "fp16"])
def test_baseline_config0_int4_gemv_2112x2816(sd):
    # BASELINE config 0: N=2112 x K=2816, uniform nibbles, scale U(0.005,0.02), bias U(-0.1,0.1), x ~ N(0,1) fp16
    W, S, B = refcases.synthetic_int4(2112, 2816, 0xB0, scale_dtype=sd)
    x_bits = refcases.normal_f16(2816, 0xB0)
    x = tfo.from_f16_bits(x_bits)
    if sd == "bf16":
        ref = tfo.int4_gemv_ref(W, S, B, x)
    else:
        q = np.empty((2112, 2816), np.float32)
        q[:, 0::2], q[:, 1::2] = W & 0x0F, W >> 4
        w = q * np.repeat(S.view(np.float16).astype(np.float32), 64, 1) + np.repeat(B.view(np.float16).astype(np.float32), 64, 1)
        ref = (w.astype(np.float64) @ x.astype(np.float64)).astype(np.float32)
    got = run_gemv(W, S, B, x_bits, scale_dtype=tfk.TF_BF16 if sd == "bf16" else tfk.TF_FP16)
    assert within_north_star(got, ref)
    assert tfo.rel_error(got, ref) < tfo.Tolerance.fp16Reduction


@pytest.mark.parametrize("m,n,off", [(16, 128, 0), (128, 2816, 0), (37, 512, 0), (128, 2816, 3), (40, 2112, 0)])
def test_int8_gemv(m, n, off):
    rng = tfo.SeedTree(0xE8).key(f"int8-gemv-{m}-{n}")
    W, S, B = tfo.quantize_int8(rng.uniform_array(-0.5, 0.5, m * n).reshape(m, n))
    x_bits = tfo.to_f16_bits(rng.uniform_array(-1, 1, n))
    ref = tfo.int8_gemv_ref(W, S, B, tfo.from_f16_bits(x_bits))
    got = run_gemv(W, S, B, x_bits, bits=8, w_off=off)
    assert tfo.rel_error(got, ref) < tfo.Tolerance.fp16Reduction
    assert within_north_star(got, ref)


def test_gelu_mul_and_rmsnorm_match_kernel_order_oracle():
    rng = np.random.default_rng(3)
    g = rng.standard_normal(2112).astype(np.float16).view(np.uint16)
    u = rng.standard_normal(2112).astype(np.float16).view(np.uint16)
    out = zeros_bytes(2112 * 2)
    ctx().gelu_mul_fp16(dev(g), dev(u), out, 2112)
    got = tfo.from_f16_bits(host(out, np.uint16, 2112))
    want = tfo.from_f16_bits(tfo.k_gelu_mul_fp16(g, u))
    assert np.max(np.abs(got - want)) <= 2e-3 and tfo.rel_error(got, want) < 1e-3
    for d in (64, 2816):
        x = (rng.standard_normal(d) * 3).astype(np.float16).view(np.uint16)
        w = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, d).astype(np.float32))
        out = zeros_bytes(d * 2)
        ctx().rmsnorm_bf16w(dev(x), dev(w), out, d, 1e-6)
        got = tfo.from_f16_bits(host(out, np.uint16, d))
        want = tfo.rmsnorm_ref(tfo.from_f16_bits(x), tfo.bf16_array_to_float(w), 1e-6)
        assert tfo.rel_error(got, want) < tfo.Tolerance.fp16Reduction


def test_contract_violations_return_status_and_enqueue_nothing():
    c = refcases.int4_gemv_case(64, 128, 1)
    dW, dS, dB, dx = dev(c["W"], 3), dev(c["S"]), dev(c["B"]), dev(c["x_bits"])
    y = zeros_bytes(256, 0xEE)
    k = ctx()
    # N not a multiple of 64 (DequantInt4GEMV.swift:57-58)
    assert k.dequant_int4_gemv(dW, dS, dB, dx, y, 64, 96, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT
    # odd weightsOffset (DequantInt4GEMV.swift:61-62)
    assert k.dequant_int4_gemv(dW, dS, dB, dx, y, 64, 128, offsets=(3, 0, 0, 0, 0), raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT
    assert "2-aligned weightsOffset" in k.last_error()
    assert k.dequant_int4_gemv(dW, dS, dB, dx, y, 0, 128, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT
    assert k.dequant_int4_gemv(None, dS, dB, dx, y, 64, 128, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT
    k.synchronize()
    assert np.all(host(y, np.uint8) == 0xEE)


@pytest.mark.parametrize("q_rows,kv_rows,n,w_off,seed", [(64, 32, 128, 0, 0x51564745), (128, 64, 2816, 2, 0x51564746), (128, 64, 2816, 0, 0x51564746),
                                                        (4096, 2048, 2816, 0, 7), (8192, 1024, 2816, 0, 8), (33, 7, 2112, 0, 9)])
def test_fused_qkv_gemv_equals_three_gemvs(q_rows, kv_rows, n, w_off, seed):
    # FusedQKVGEMVTests.swift:8-127 (one launch == the three projections, also at a +2 weight offset) + the decode shapes
    rng = tfo.SplitMix64(seed)
    mats = []
    for rows in (q_rows, kv_rows, kv_rows):
        if rows * n <= 1 << 20:
            mats.append(tfo.quantize_int4(rng.uniform_array(-0.5, 0.5, rows * n).reshape(rows, n)))
        else:
            mats.append(refcases.synthetic_int4(rows, n, seed + rows))
    x_bits = tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, n))
    k = ctx()
    d = [(dev(W, w_off), dev(S), dev(B)) for W, S, B in mats]
    dx = dev(x_bits)
    fused = [zeros_bytes(r * 2 + 16, 0xEE) for r in (q_rows, kv_rows, kv_rows)]
    args = []
    for W, S, B in d:
        args += [W.data_ptr(), w_off, S.data_ptr(), 0, B.data_ptr(), 0]
    outs = []
    for o in fused:
        outs += [o.data_ptr(), 0]
    k.check(k.lib.tf_fused_qkv_gemv(k.handle, None, *args, dx.data_ptr(), *outs, q_rows, kv_rows, n, tfk.TF_BF16))
    for (W, S, B), (dW, dS, dB), o, rows in zip(mats, d, fused, (q_rows, kv_rows, kv_rows)):
        single = zeros_bytes(rows * 2)
        k.dequant_int4_gemv(dW, dS, dB, dx, single, rows, n, offsets=(w_off, 0, 0, 0, 0))
        got = host(o, np.uint16, rows)
        assert np.array_equal(got, host(single, np.uint16, rows))
        assert np.all(host(o, np.uint8)[rows * 2:] == 0xEE)
        ref = tfo.int4_gemv_ref(W, S, B, tfo.from_f16_bits(x_bits), threads=8)
        assert within_north_star(tfo.from_f16_bits(got), ref, abs_=1e-3 * max(1.0, float(np.max(np.abs(ref)))))
    bad = list(args)
    bad[1] = 1                                     # odd q weights offset (FusedQKVGEMV.swift:60-63)
    assert k.lib.tf_fused_qkv_gemv(k.handle, None, *bad, dx.data_ptr(), *outs, q_rows, kv_rows, n, tfk.TF_BF16) == tfk.TF_ERR_INVALID_ARGUMENT

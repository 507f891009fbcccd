"""Input generators shared by the oracle tests and the GPU parity tests.

Each builder restates how one of the reference's test suites draws its inputs
(same seeds, labels, ranges and draw order), so a case here is the same case the
reference runs on Metal.  Test infrastructure: uses the CPU oracle's quantizer.
"""
import numpy as np

from oracle import tfo


def int4_gemv_case(m, n, seed, weight_byte_offset=0, lo=-0.5, hi=0.5, label_prefix="int4-gemv-kernel"):
    """Tests/TurboFieldfare/Core/Kernels/Quant/DequantInt4GEMVTests.swift:41-62."""
    base = f"{label_prefix}-m{m}-n{n}"
    key = base if weight_byte_offset == 0 else f"{base}-off{weight_byte_offset}"
    rng = tfo.SeedTree(seed).key(key)
    raw = rng.uniform_array(lo, hi, m * n).reshape(m, n)
    W, S, B = tfo.quantize_int4(raw)
    x32 = rng.uniform_array(-1.0, 1.0, n)
    x_bits = tfo.to_f16_bits(x32)
    return dict(W=W, S=S, B=B, x_bits=x_bits, x_ref=tfo.from_f16_bits(x_bits), raw=raw)


def synthetic_int4(m, n, seed, label="synthetic-int4", scale_dtype="bf16"):
    """BASELINE-style weights: uniform nibbles, scale ~U(0.005,0.02), bias ~U(-0.1,0.1)."""
    rng = np.random.default_rng(tfo.SeedTree(seed).key_state(label) & 0xFFFFFFFF)
    W = rng.integers(0, 256, (m, n // 2), dtype=np.uint8)
    s = rng.uniform(0.005, 0.02, (m, n // 64)).astype(np.float32)
    b = rng.uniform(-0.1, 0.1, (m, n // 64)).astype(np.float32)
    if scale_dtype == "bf16":
        return W, tfo.bf16_bits_array(s).reshape(s.shape), tfo.bf16_bits_array(b).reshape(b.shape)
    return W, s.astype(np.float16).view(np.uint16), b.astype(np.float16).view(np.uint16)


def synthetic_int8(m, n, seed, label="synthetic-int8"):
    rng = np.random.default_rng(tfo.SeedTree(seed).key_state(label) & 0xFFFFFFFF)
    W = rng.integers(0, 256, (m, n), dtype=np.uint8)
    s = rng.uniform(0.0002, 0.0008, (m, n // 64)).astype(np.float32)
    b = rng.uniform(-0.1, 0.0, (m, n // 64)).astype(np.float32)
    return W, tfo.bf16_bits_array(s).reshape(s.shape), tfo.bf16_bits_array(b).reshape(b.shape)


def normal_f16(n, seed, label="activation"):
    rng = np.random.default_rng(tfo.SeedTree(seed).key_state(label) & 0xFFFFFFFF)
    return rng.standard_normal(n).astype(np.float32).astype(np.float16).view(np.uint16)


def router_case_production(experts=16, d=128):
    """Tests/.../Kernels/MoE/RouterTopKTests.swift:22-33."""
    rng = tfo.SplitMix64(0xA5B61234)
    weights = np.empty((experts, d), np.float32)
    for e in range(experts):
        weights[e] = rng.uniform_array(-0.05, 0.05, d) + np.float32(e) * np.float32(0.01)
    hidden = rng.uniform_array(-1.0, 1.0, d)
    inv_sqrt_d = np.float32(1.0) / np.sqrt(np.float32(d))
    eff = rng.uniform_array(0.5, 1.5, d) * inv_sqrt_d
    expert_scale = rng.uniform_array(0.6, 1.4, experts)
    return weights, hidden, eff, expert_scale


def router_case_near_tie(experts=16, d=128):
    """Tests/.../Kernels/MoE/RouterTopKTests.swift:46-63."""
    rng = tfo.SplitMix64(0x71E0F4A)
    pattern = rng.uniform_array(0.2, 1.0, d)
    hidden = rng.uniform_array(0.5, 1.5, d)
    gains = np.zeros(experts, np.float32)
    for e in range(7):
        gains[e] = np.float32(1.0) - np.float32(e) * np.float32(0.05)
    gains[7] = 0.5
    gains[8] = np.float32(0.5) * (np.float32(1.0) + np.float32(1e-4))
    for e in range(9, experts):
        gains[e] = np.float32(0.4) - np.float32(e - 9) * np.float32(0.02)
    weights = gains[:, None] * pattern[None, :]
    return weights.astype(np.float32), hidden, np.ones(d, np.float32), np.ones(experts, np.float32)


def moe_fused_case(d=128, f=64, top_k=8):
    """Tests/.../Kernels/MoE/MoEFusedFFNTests.swift:17-58 (draw order: per expert gate, up, down; then x, residual)."""
    rng = tfo.SeedTree(0x2D3).key("production-routed-moe")
    blobs, off = [], None
    for _ in range(top_k):
        gate = tfo.quantize_int4(rng.uniform_array(-0.4, 0.4, f * d).reshape(f, d))
        up = tfo.quantize_int4(rng.uniform_array(-0.4, 0.4, f * d).reshape(f, d))
        down = tfo.quantize_int4(rng.uniform_array(-0.4, 0.4, d * f).reshape(d, f))
        blob, off = tfo.make_blob(gate, up, down)
        blobs.append(blob)
    x_bits = tfo.to_f16_bits(rng.uniform_array(-0.5, 0.5, d))
    res_bits = tfo.to_f16_bits(rng.uniform_array(-0.5, 0.5, d))
    w_bits = tfo.to_f16_bits(np.float32(0.04) + np.arange(top_k, dtype=np.float32) * np.float32(0.015))
    return dict(blobs=blobs, off=off, x_bits=x_bits, residual_bits=res_bits, routing_w_bits=w_bits, d=d, f=f)


def shared_expert_case(d=128, f=64):
    """Tests/.../Kernels/MoE/SharedExpertInt4Tests.swift:15-23."""
    rng = tfo.SeedTree(0x604).key("shared-expert-int4")
    x = rng.uniform_array(-0.4, 0.4, d)
    gate = tfo.quantize_int4(rng.uniform_array(-0.4, 0.4, f * d).reshape(f, d))
    up = tfo.quantize_int4(rng.uniform_array(-0.4, 0.4, f * d).reshape(f, d))
    down = tfo.quantize_int4(rng.uniform_array(-0.4, 0.4, d * f).reshape(d, f))
    return dict(x_bits=tfo.to_f16_bits(x), gate=gate, up=up, down=down, d=d, f=f)


def lm_head_random_case(d=64, v=1024):
    """Tests/.../Kernels/Fusions/LMHeadChainInt4Tests.swift:113-121."""
    rng = tfo.SplitMix64(0x1A4E4EAD20260603)
    hidden_bits = tfo.to_f16_bits(rng.uniform_array(-1, 1, d))
    norm_bits = tfo.bf16_bits_array(rng.uniform_array(0.5, 1.5, d))
    W, S, B = tfo.quantize_int4(rng.uniform_array(-1, 1, v * d).reshape(v, d))
    return hidden_bits, norm_bits, W, S, B


def lm_head_constant_rows(d, v, hot_rows, hot=1.0, cold=-0.5):
    rows = np.full((v, d), cold, np.float32)
    for r in hot_rows:
        rows[r] = hot
    return tfo.quantize_int4(rows)


def synthetic_expert_pool(num_experts, d, f):
    """Tests/.../Kernels/Prefill/PrefillGroupedRoutedMoETests.swift:109-216."""
    def rows(r, c, expert, role):
        rr = ((np.arange(r) % 7) - 3).astype(np.float32)[:, None]
        cc = ((np.arange(c) % 11) - 5).astype(np.float32)[None, :]
        return (np.float32(expert + 1) * np.float32(0.001) + np.float32(role + 1) * np.float32(0.003)
                + rr * np.float32(0.0004) + cc * np.float32(0.0002)).astype(np.float32)
    blobs, off = [], None
    for e in range(num_experts):
        blob, off = tfo.make_blob(tfo.quantize_int4(rows(f, d, e, 0)), tfo.quantize_int4(rows(f, d, e, 1)),
                                  tfo.quantize_int4(rows(d, f, e, 2)))
        blobs.append(blob)
    stride = blobs[0].size
    return np.concatenate(blobs), off, stride

"""Writes the small input/output fixtures kept beside this script (`*.npz`, plain arrays, no pickled objects).

Every case draws its inputs the way one of the reference's own test suites does (seed, label, range and draw order
are cited per case) and records what the CPU restatement of the reference computes for them.  The fixtures are data
only; nothing of the reference is executed or stored.  Run from the repository root:

    python tests/golden/make_golden.py

The CPU tests check that the oracle still reproduces every file bit for bit; the GPU tests run the HIP library on
the stored inputs and compare with the stored outputs, without importing the oracle.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

import refcases  # noqa: E402
from oracle import tfo  # noqa: E402


def offsets_array(off):
    return np.array([getattr(off, name) for name, _ in off._fields_], np.uint32)


def raw16(records):
    """16-byte pair records (token, expert, rank, weight bits, padding) as a [n, 16] byte matrix."""
    return np.ascontiguousarray(records).view(np.uint8).reshape(-1, 16)


def prng_streams():
    """Validation/Support/PRNG/SplitMix64.swift:11-23, SeedTree.swift:12-19 with the seeds/labels the kernel tests use."""
    out = {}
    for seed in (0, 1234567, 0xA5B61234, 0x71E0F4A, 0x1A4E4EAD20260603):
        g = tfo.SplitMix64(seed)
        out[f"next_{seed:x}"] = np.array([g.next() for _ in range(8)], np.uint64)
        out[f"uniform_{seed:x}"] = tfo.SplitMix64(seed).uniform_array(-1.0, 1.0, 8)
    for seed, label in ((0x2D3, "production-routed-moe"), (0x604, "shared-expert-int4"), (0x1D4, "int4-gemv-kernel-m64-n128")):
        out[f"tree_{seed:x}_{label}"] = np.array([tfo.SeedTree(seed).key_state(label)], np.uint64)
        out[f"tree_uniform_{seed:x}_{label}"] = tfo.SeedTree(seed).key(label).uniform_array(-0.5, 0.5, 8)
    return out


def gemv_int4():
    """Tests/TurboFieldfare/Core/Kernels/Quant/DequantInt4GEMVTests.swift:41-62 at M=64, K=128."""
    c = refcases.int4_gemv_case(64, 128, 0x1D4)
    return dict(W=c["W"], S=c["S"], B=c["B"], x_bits=c["x_bits"], raw=c["raw"],
                dequantized=tfo.dequantize_int4(c["W"], c["S"], c["B"]),
                y_ref=tfo.int4_gemv_ref(c["W"], c["S"], c["B"], c["x_ref"]),
                y_kernel_order=tfo.k_int4_gemv(c["W"], c["S"], c["B"], c["x_bits"]))


def gemv_int8():
    """Validation/Support/Reference/Quant/DequantInt8Gemv.swift over a 16 x 128 router-like matrix."""
    rng = tfo.SeedTree(0x1D8).key("int8-gemv-kernel-m16-n128")
    raw = rng.uniform_array(-0.05, 0.05, 16 * 128).reshape(16, 128)
    W, S, B = tfo.quantize_int8(raw)
    x_bits = tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, 128))
    return dict(W=W, S=S, B=B, x_bits=x_bits, dequantized=tfo.dequantize_int8(W, S, B),
                y_ref=tfo.int8_gemv_ref(W, S, B, tfo.from_f16_bits(x_bits)))


def router():
    """Tests/.../Kernels/MoE/RouterTopKTests.swift:22-70: the production-like draw and the near-tie case, E=16, D=128."""
    out = {}
    for name, case in (("prod", refcases.router_case_production()), ("tie", refcases.router_case_near_tie())):
        weights, hidden, eff, escale = case
        W, S, B = tfo.quantize_int8(weights)
        hidden_bits, eff_bits, pes_bits = tfo.to_f16_bits(hidden), tfo.bf16_bits_array(eff), tfo.bf16_bits_array(escale)
        idx, wts, logits = tfo.router_reference(W, S, B, tfo.from_f16_bits(hidden_bits), tfo.bf16_array_to_float(eff_bits),
                                                  tfo.bf16_array_to_float(pes_bits))
        out.update({f"{name}_W": W, f"{name}_S": S, f"{name}_B": B, f"{name}_hidden_bits": hidden_bits, f"{name}_eff_bits": eff_bits,
                    f"{name}_per_expert_bits": pes_bits, f"{name}_indices": np.asarray(idx, np.uint32),
                    f"{name}_weights": np.asarray(wts, np.float32), f"{name}_logits": np.asarray(logits, np.float32)})
    return out


def moe():
    """Tests/.../Kernels/MoE/MoEFusedFFNTests.swift:17-58: D=128, F=64, eight experts, fp16 routing weights."""
    c = refcases.moe_fused_case()
    x, res, rw = (tfo.from_f16_bits(c[k]) for k in ("x_bits", "residual_bits", "routing_w_bits"))
    y = tfo.moe_apply_streamed_routed(c["blobs"], c["off"], x, res, rw, c["d"], c["f"])
    acts = tfo.k_moe_phase1(c["blobs"], c["off"], c["x_bits"], c["d"], c["f"])
    return dict(blobs=np.stack(c["blobs"]), offsets=offsets_array(c["off"]), x_bits=c["x_bits"], residual_bits=c["residual_bits"],
                routing_w_bits=c["routing_w_bits"], y_ref=y, acts_kernel_order=acts,
                expert0_ffn=tfo.moe_run_ffn(c["blobs"][0], c["off"], x, c["d"], c["f"]))


def shared_expert():
    """Tests/.../Kernels/MoE/SharedExpertInt4Tests.swift:15-28: D=128, F=64."""
    c = refcases.shared_expert_case()
    y = tfo.shared_expert_ref(c["gate"], c["up"], c["down"], tfo.from_f16_bits(c["x_bits"]))
    out = dict(x_bits=c["x_bits"], y_ref=y)
    for name in ("gate", "up", "down"):
        for part, a in zip("WSB", c[name]):
            out[f"{name}_{part}"] = a
    return out


def lm_head():
    """Tests/.../Kernels/Fusions/LMHeadChainInt4Tests.swift:10-39,113-193: random head D=64, V=1024, and the tie / target rows."""
    hidden_bits, norm_bits, W, S, B = refcases.lm_head_random_case()
    token, logits = tfo.lm_head_cpu_greedy(hidden_bits, norm_bits, W, S, B, want_logits=True)
    out = dict(hidden_bits=hidden_bits, norm_bits=norm_bits, W=W, S=S, B=B, token=np.array([token], np.uint32),
               logits=np.asarray(logits, np.float32))
    d, v = 64, 1024
    ones_hidden, ones_norm = tfo.to_f16_bits(np.ones(d, np.float32)), tfo.bf16_bits_array(np.ones(d, np.float32))
    for name, rows in (("tie", (17, 311)), ("target", (v - 3,))):
        Wc, Sc, Bc = refcases.lm_head_constant_rows(d, v, rows)
        tok = tfo.lm_head_cpu_greedy(ones_hidden, ones_norm, Wc, Sc, Bc)
        out.update({f"{name}_W": Wc, f"{name}_S": Sc, f"{name}_B": Bc, f"{name}_token": np.array([tok], np.uint32)})
    out["ones_hidden_bits"], out["ones_norm_bits"] = ones_hidden, ones_norm
    return out


def rmsnorm_gelu():
    """Validation/Support/Reference/Primitives/RmsNorm.swift and Reference/MoE/Moe.swift:84-85 (tanh GELU) on 256 values."""
    rng = tfo.SeedTree(0x9E1).key("rmsnorm-gelu")
    x_bits = tfo.to_f16_bits(rng.uniform_array(-2.0, 2.0, 256))
    w_bits = tfo.bf16_bits_array(rng.uniform_array(0.5, 1.5, 256))
    gate_bits = tfo.to_f16_bits(rng.uniform_array(-3.0, 3.0, 256))
    up_bits = tfo.to_f16_bits(rng.uniform_array(-2.0, 2.0, 256))
    return dict(x_bits=x_bits, w_bits=w_bits, gate_bits=gate_bits, up_bits=up_bits,
                rmsnorm_ref=tfo.rmsnorm_ref(tfo.from_f16_bits(x_bits), tfo.bf16_array_to_float(w_bits), 1e-6),
                rmsnorm_kernel_bits=tfo.k_rmsnorm_bf16w(x_bits, w_bits, 1e-6),
                gelu_points=tfo.gelu_tanh(np.array([0.0, 1.0, -1.0, 2.0], np.float32)),
                gelu_mul_kernel_bits=tfo.k_gelu_mul_fp16(gate_bits, up_bits))


def prefill():
    """Tests/.../Kernels/Prefill/PrefillGroupedRoutedMoETests.swift:109-303: synthetic pool (closed-form rows), 6 experts,
    D=128, F=64, five tokens with top-2 routes; grouping per Kernels/Prefill/MoE/PrefillMoEGrouping.swift:90-193."""
    d, f, ne, t, top_k = 128, 64, 6, 5, 2
    pool, off, stride = refcases.synthetic_expert_pool(ne, d, f)
    rng = tfo.SeedTree(0x6F1).key("prefill-grouped-golden")
    hidden_bits = tfo.to_f16_bits(rng.uniform_array(-0.5, 0.5, t * d))
    indices = np.array([[4, 1], [1, 5], [0, 4], [4, 2], [1, 0]], np.uint32)
    weights_bits = tfo.to_f16_bits(np.array([[0.6, 0.4], [0.7, 0.3], [0.55, 0.45], [0.8, 0.2], [0.5, 0.5]], np.float32).ravel())
    pairs = tfo.make_pairs(indices.ravel(), weights_bits, t, top_k)
    g = tfo.group_pairs(pairs, t, top_k, ne)
    partials = tfo.prefill_route_partials(g["sorted_pairs"], t, hidden_bits, d, pool, stride, off, top_k, d, f)
    reduced = tfo.prefill_reduce_token_major(partials, weights_bits, t, top_k, d)
    return dict(pool=pool, offsets=offsets_array(off), stride=np.array([stride], np.uint64), hidden_bits=hidden_bits, indices=indices,
                weights_bits=weights_bits, pairs_bytes=raw16(pairs), sorted_pairs_bytes=raw16(g["sorted_pairs"]),
                expert_offsets=np.asarray(g["per_expert_offsets"], np.uint32), expert_counts=np.asarray(g["per_expert_counts"], np.uint32),
                route_partials_bits=np.asarray(partials), reduced_bits=np.asarray(reduced))


def qmm():
    """Tests/.../Kernels/TensorCore/MPPPrefillInt4QMMTests.swift:80-105: Y[M,N] = X[M,K] . dequant(W[N,K])^T at M=8, N=64, K=128."""
    m, n, k = 8, 64, 128
    rng = tfo.SeedTree(0x3A7).key("int4-qmm-golden")
    W, S, B = tfo.quantize_int4(rng.uniform_array(-0.5, 0.5, n * k).reshape(n, k))
    x_bits = tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, m * k))
    return dict(W=W, S=S, B=B, x_bits=x_bits, y_ref=np.asarray(tfo.qmm_cpu_reference(W, S, B, x_bits, m, n, k), np.float32).reshape(m, n))


def layer_glue():
    """Tests/.../Kernels/Fusions/FusedLayerTailTests.swift:11-20 and FusedPostAttentionSetupTests.swift:11-17 at D = 2816."""
    d, eps = 2816, 1e-6
    rng = tfo.SplitMix64(0xC0DE7A11)
    half = lambda r: tfo.to_f16_bits(r.uniform_array(-1.0, 1.0, d))
    weight = lambda r: tfo.bf16_bits_array(r.uniform_array(0.5, 1.5, d))
    h2, h1, hidden = half(rng), half(rng), half(rng)
    w2, w = weight(rng), weight(rng)
    scalar = rng.uniform(0.75, 1.25)
    out = dict(tail_h2=h2, tail_h1=h1, tail_hidden=hidden, tail_w_postffn2=w2, tail_w_postffn=w, tail_scalar=np.array([scalar], np.float32),
               tail_hidden_out=tfo.k_layer_tail(h2, h1, hidden, w2, w, eps, scalar), tail_ref=tfo.layer_tail_ref(h2, h1, hidden, w2, w, eps, scalar))
    rng = tfo.SplitMix64(0x9057A77E)
    hidden, attn = half(rng), half(rng)
    w_post, w_pre, w_pre2 = weight(rng), weight(rng), weight(rng)
    h_out, dense, routed, router = tfo.k_post_attn_setup(hidden, attn, w_post, w_pre, w_pre2, eps)
    out.update(setup_hidden=hidden, setup_attn=attn, setup_w_post=w_post, setup_w_pre=w_pre, setup_w_pre2=w_pre2, setup_hidden_out=h_out,
               setup_dense=dense, setup_routed=routed, setup_router=router)
    return out


def head_neighbours():
    """EmbedLookupTests.swift:16-77 (V=16, D=128), LogitSoftcapSoftmaxTests.swift:34-54 (2048 logits in +-50), and sampler draws
    on a 1003-entry distribution (SampleTopK64Tests.swift:101-131 shapes) with the tokens the restated sampler returns."""
    rng = tfo.SeedTree(0x131).key("embed-lookup-int4-table")
    W, S, B = tfo.quantize_int4(rng.uniform_array(-1.0, 1.0, 16 * 128).reshape(16, 128))
    scale = float(np.sqrt(np.float32(128)))
    out = dict(embed_W=W, embed_S=S, embed_B=B, embed_scale=np.array([scale], np.float32),
               embed_row9=tfo.embed_lookup_int4(W, S, B, 9, scale))
    rng = tfo.SeedTree(0x131).key("softcap-softmax-random")
    logits = tfo.to_f16_bits(rng.uniform_array(-50.0, 50.0, 2048))
    out.update(softmax_logits=logits, softmax_probs=tfo.logit_softcap_softmax_ref(tfo.from_f16_bits(logits), 30.0))
    p = np.random.default_rng(1003).random(1003).astype(np.float32)
    probs = tfo.to_f16_bits(p / p.sum())
    seeds = np.array([1, 2, 3, 0x123456789ABCDEF0, 0xFFFFFFFFFFFFFFFF], np.uint64)
    out.update(sample_probs=probs, sample_seeds=seeds,
               sample_greedy=np.array([tfo.sample(probs, 0.0, 0, 1.0, 1)], np.uint32),
               sample_top4=np.array([tfo.sample(probs, 1.0, 4, 1.0, int(s)) for s in seeds], np.uint32),
               sample_top64_p95_t085=np.array([tfo.sample_topk64(probs, 0.85, 0.95, int(s)) for s in seeds], np.uint32),
               sample_nucleus_p30=np.array([tfo.sample(probs, 1.3, 0, 0.3, int(s)) for s in seeds], np.uint32))
    return out


CASES = dict(prng_streams=prng_streams, gemv_int4_m64_k128=gemv_int4, gemv_int8_m16_k128=gemv_int8, router_e16_d128=router,
             moe_d128_f64_top8=moe, shared_expert_d128_f64=shared_expert, lm_head_d64_v1024=lm_head, rmsnorm_gelu_256=rmsnorm_gelu,
             prefill_grouped_e6_d128_f64=prefill, int4_qmm_m8_n64_k128=qmm, layer_glue_d2816=layer_glue, head_neighbours=head_neighbours)


def generate(name):
    return {k: np.ascontiguousarray(v) for k, v in CASES[name]().items()}


if __name__ == "__main__":
    for case in CASES:
        arrays = generate(case)
        path = os.path.join(HERE, case + ".npz")
        np.savez_compressed(path, **arrays)
        print(f"{case}: {len(arrays)} arrays, {os.path.getsize(path)} bytes")

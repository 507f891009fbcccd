"""GPU parity against the committed fixtures under tests/golden/: the HIP library, called through its C ABI, on the
stored inputs, compared with the stored outputs.  Nothing here imports the CPU oracle, so these checks hold even where
only the fixtures travelled.  Tolerances: dequantized weights, indices, tokens and the pair order are exact; matmul
outputs are within 1e-3 absolute + 1e-2 relative of the fp32 reference (and much closer in practice)."""
import ctypes as C
import os

import numpy as np
import pytest

from gpu_helpers import ctx, dev, host, tfk, within_north_star, zeros_bytes

pytestmark = pytest.mark.gpu
GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(case):
    with np.load(os.path.join(GOLDEN, case + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def f16(bits):
    return np.asarray(bits, np.uint16).view(np.float16).astype(np.float32)


def test_int4_dequant_and_gemv_fixture():
    z = load("gemv_int4_m64_k128")
    k = ctx()
    W, S, B, x = dev(z["W"]), dev(z["S"]), dev(z["B"]), dev(z["x_bits"])
    out = zeros_bytes(64 * 128 * 4)
    k.dequantize_int4(W, S, B, out, 64, 128)
    assert host(out, np.float32, 64 * 128).tobytes() == z["dequantized"].tobytes()        # bit-exact unpack + affine
    y16, y32 = zeros_bytes(64 * 2), zeros_bytes(64 * 4)
    k.dequant_int4_gemv(W, S, B, x, y16, 64, 128)
    k.dequant_int4_gemv(W, S, B, x, y32, 64, 128, out_dtype=tfk.TF_FP32)
    assert within_north_star(host(y32, np.float32, 64), z["y_ref"]) and np.max(np.abs(host(y32, np.float32, 64) - z["y_ref"])) < 1e-4
    assert np.max(np.abs(f16(host(y16, np.uint16, 64)) - z["y_ref"])) <= 4e-3


def test_int8_dequant_and_gemv_fixture():
    z = load("gemv_int8_m16_k128")
    k = ctx()
    W, S, B, x = dev(z["W"]), dev(z["S"]), dev(z["B"]), dev(z["x_bits"])
    out = zeros_bytes(16 * 128 * 4)
    k.dequantize_int4(W, S, B, out, 16, 128, bits=8)
    assert host(out, np.float32, 16 * 128).tobytes() == z["dequantized"].tobytes()
    y32 = zeros_bytes(16 * 4)
    k.dequant_int4_gemv(W, S, B, x, y32, 16, 128, out_dtype=tfk.TF_FP32, bits=8)
    assert np.max(np.abs(host(y32, np.float32, 16) - z["y_ref"])) < 1e-4


@pytest.mark.parametrize("name", ["prod", "tie"])
def test_router_fixture(name):
    z = load("router_e16_d128")
    k = ctx()
    idx, wts = zeros_bytes(32), zeros_bytes(16)
    k.router_gemma4(dev(z[f"{name}_W"]), dev(z[f"{name}_S"]), dev(z[f"{name}_B"]), dev(z[f"{name}_hidden_bits"]),
                    dev(z[f"{name}_eff_bits"]), dev(z[f"{name}_per_expert_bits"]), idx, wts, 16, 128)
    assert list(host(idx, np.uint32, 8)) == list(z[f"{name}_indices"])
    assert np.max(np.abs(f16(host(wts, np.uint16, 8)) - z[f"{name}_weights"])) < 5e-4


def test_routed_moe_fixture():
    z = load("moe_d128_f64_top8")
    k = ctx()
    d, f = 128, 64
    blobs = [dev(b) for b in z["blobs"]]
    routed = k.routed_from_pointers([b.data_ptr() for b in blobs])
    off = tfk.ExpertOffsets(*[int(v) for v in z["offsets"]])
    acts, y = zeros_bytes(8 * f * 4), zeros_bytes(d * 2)
    x, rw, res = dev(z["x_bits"]), dev(z["routing_w_bits"]), dev(z["residual_bits"])
    k.moe_phase1(routed, off, x, acts, d, f)
    k.moe_phase2(routed, off, acts, rw, res, y, d, f)
    got = f16(host(y, np.uint16, d))
    assert within_north_star(got, z["y_ref"]) and np.max(np.abs(got - z["y_ref"])) < 3e-3


def test_shared_expert_fixture():
    z = load("shared_expert_d128_f64")
    k = ctx()
    d, f = 128, 64
    t = {n: dev(z[n]) for n in z if n != "y_ref"}
    proj = {n: tfk.projection(t[f"{n}_W"], t[f"{n}_S"], t[f"{n}_B"], *(r_c)) for n, r_c in (("gate", (f, d)), ("up", (f, d)), ("down", (d, f)))}
    y, sg, su, sa = zeros_bytes(d * 2), zeros_bytes(f * 2), zeros_bytes(f * 2), zeros_bytes(f * 2)
    k.shared_expert_int4(t["x_bits"], proj["gate"], proj["up"], proj["down"], y, sg, su, sa)
    got = f16(host(y, np.uint16, d))
    assert within_north_star(got, z["y_ref"]) and np.max(np.abs(got - z["y_ref"])) < 3e-3


def test_lm_head_fixture():
    z = load("lm_head_d64_v1024")
    k = ctx()
    tok = zeros_bytes(4, 0xFF)
    k.lm_head_greedy(dev(z["hidden_bits"]), dev(z["norm_bits"]), dev(z["W"]), dev(z["S"]), dev(z["B"]), tok, 64, 1024)
    assert int(host(tok, np.uint32, 1)[0]) == int(z["token"][0])
    logits = zeros_bytes(1024 * 4)
    k.lm_head_logits(dev(z["hidden_bits"]), dev(z["norm_bits"]), dev(z["W"]), dev(z["S"]), dev(z["B"]), logits, 64, 1024, out_dtype=tfk.TF_FP32)
    got = host(logits, np.float32, 1024)
    assert within_north_star(got, z["logits"], rel=1e-2, abs_=2e-2)          # the head reads the fp16-rounded normalised row
    for name in ("tie", "target"):
        k.lm_head_greedy(dev(z["ones_hidden_bits"]), dev(z["ones_norm_bits"]), dev(z[f"{name}_W"]), dev(z[f"{name}_S"]), dev(z[f"{name}_B"]), tok, 64, 1024)
        assert int(host(tok, np.uint32, 1)[0]) == int(z[f"{name}_token"][0])


def test_rmsnorm_and_gelu_mul_fixture():
    z = load("rmsnorm_gelu_256")
    k = ctx()
    out = zeros_bytes(256 * 2)
    k.rmsnorm_bf16w(dev(z["x_bits"]), dev(z["w_bits"]), out, 256, 1e-6)
    got = host(out, np.uint16, 256)
    assert np.max(np.abs(f16(got) - z["rmsnorm_ref"])) <= 2e-3 * max(1.0, float(np.max(np.abs(z["rmsnorm_ref"]))))
    assert np.max(np.abs(got.astype(np.int32) - z["rmsnorm_kernel_bits"].astype(np.int32))) <= 1      # within one fp16 ulp of the kernel-order restatement
    k.gelu_mul_fp16(dev(z["gate_bits"]), dev(z["up_bits"]), out, 256)
    got = host(out, np.uint16, 256)
    assert np.max(np.abs(f16(got) - f16(z["gelu_mul_kernel_bits"]))) <= 4e-3


def test_prefill_grouping_experts_and_reduce_fixture():
    z = load("prefill_grouped_e6_d128_f64")
    k = ctx()
    d, f, E, T, top_k = 128, 64, 6, 5, 2
    n = T * top_k
    idx, w = dev(z["indices"]), dev(z["weights_bits"])
    cap = E + n // 128 + 1
    sp, offs, cnts, chunks, nch = zeros_bytes(n * 16), zeros_bytes(E * 4), zeros_bytes(E * 4), zeros_bytes(cap * 12), zeros_bytes(4)
    k.check(k.lib.tf_prefill_group_pairs_device(k.handle, None, idx.data_ptr(), w.data_ptr(), T, top_k, E, sp.data_ptr(), offs.data_ptr(),
                                                cnts.data_ptr(), chunks.data_ptr(), nch.data_ptr()))
    assert host(sp, np.uint8, n * 16).tobytes() == z["sorted_pairs_bytes"].tobytes()
    assert list(host(cnts, np.uint32, E)) == list(z["expert_counts"])
    present = z["expert_counts"] > 0
    assert list(host(offs, np.uint32, E)[present]) == list(z["expert_offsets"][present])
    off = tfk.ExpertOffsets(*[int(v) for v in z["offsets"]])
    pool, hidden = dev(z["pool"]), dev(z["hidden_bits"])
    acts, partials, h2 = zeros_bytes(n * f * 2), zeros_bytes(n * d * 2), zeros_bytes(T * d * 2)
    k.check(k.lib.tf_prefill_grouped_routed_moe_resident(k.handle, None, hidden.data_ptr(), 0, d, sp.data_ptr(), chunks.data_ptr(), nch.data_ptr(),
                                                         cap, n, pool.data_ptr(), int(z["stride"][0]), E, C.byref(off), acts.data_ptr(),
                                                         partials.data_ptr(), d, f, top_k, tfk.TF_BF16))
    k.check(k.lib.tf_prefill_moe_reduce_token_major(k.handle, None, partials.data_ptr(), 0, w.data_ptr(), 0, h2.data_ptr(), 0, T, top_k, d))
    assert np.max(np.abs(f16(host(partials, np.uint16, n * d)) - f16(z["route_partials_bits"]))) <= 0.0015   # the reference test's bound
    assert np.max(np.abs(f16(host(h2, np.uint16, T * d)) - f16(z["reduced_bits"]))) <= 0.0015


def test_int4_qmm_fixture():
    z = load("int4_qmm_m8_n64_k128")
    k = ctx()
    m, n, kk = 8, 64, 128
    W, S, B, x = dev(z["W"]), dev(z["S"]), dev(z["B"]), dev(z["x_bits"])
    for entry in ("tf_int4_qmm", "tf_prefill_int4_qmm"):
        y = zeros_bytes(m * n * 2)
        k.check(getattr(k.lib, entry)(k.handle, None, W.data_ptr(), 0, S.data_ptr(), 0, B.data_ptr(), 0, x.data_ptr(), 0, y.data_ptr(), 0,
                                      m, n, kk, tfk.TF_BF16))
        got = f16(host(y, np.uint16, m * n)).reshape(m, n)
        assert within_north_star(got, z["y_ref"]), entry


def test_layer_glue_fixture():
    z = load("layer_glue_d2816")
    k = ctx()
    d = 2816
    t = {n: dev(z[n]) for n in z if z[n].dtype == np.uint16 and z[n].size == d}       # keeps every operand alive until the results are read
    k.check(k.lib.tf_fused_layer_tail(k.handle, None, t["tail_h2"].data_ptr(), t["tail_h1"].data_ptr(), t["tail_hidden"].data_ptr(),
                                      t["tail_w_postffn2"].data_ptr(), 0, t["tail_w_postffn"].data_ptr(), 0, d, 1e-6, float(z["tail_scalar"][0])))
    got = host(t["tail_hidden"], np.uint16, d)
    assert np.count_nonzero(got != z["tail_hidden_out"]) <= 14 and np.max(np.abs(f16(got) - f16(z["tail_hidden_out"]))) <= 2.0 ** -9
    assert np.max(np.abs(f16(got) - z["tail_ref"])) / float(np.max(np.abs(z["tail_ref"]))) < 4e-3       # FusedLayerTailTests.swift:72
    dense, routed, router = zeros_bytes(d * 2), zeros_bytes(d * 2), zeros_bytes(d * 2)
    k.check(k.lib.tf_fused_post_attn_setup(k.handle, None, t["setup_hidden"].data_ptr(), t["setup_attn"].data_ptr(), dense.data_ptr(), routed.data_ptr(),
                                           router.data_ptr(), t["setup_w_post"].data_ptr(), 0, t["setup_w_pre"].data_ptr(), 0,
                                           t["setup_w_pre2"].data_ptr(), 0, d, 1e-6))
    for buf, name in ((t["setup_hidden"], "setup_hidden_out"), (dense, "setup_dense"), (routed, "setup_routed"), (router, "setup_router")):
        got = host(buf, np.uint16, d)
        assert np.count_nonzero(got != z[name]) <= 14 and np.max(np.abs(f16(got) - f16(z[name]))) <= 2.0 ** -9, name


def test_head_neighbours_fixture():
    z = load("head_neighbours")
    k = ctx()
    out = zeros_bytes(128 * 2)
    eW, eS, eB, logits = dev(z["embed_W"]), dev(z["embed_S"]), dev(z["embed_B"]), dev(z["softmax_logits"])
    k.check(k.lib.tf_embed_lookup_int4(k.handle, None, eW.data_ptr(), 0, eS.data_ptr(), 0, eB.data_ptr(), 0,
                                       out.data_ptr(), 0, 9, 128, float(z["embed_scale"][0]), 16))
    assert np.array_equal(host(out, np.uint16, 128), z["embed_row9"].astype(np.float16).view(np.uint16))
    probs = zeros_bytes(2048 * 2)
    k.check(k.lib.tf_logit_softcap_softmax(k.handle, None, logits.data_ptr(), probs.data_ptr(), 2048, 30.0, tfk.TF_FP16))
    got, ref = f16(host(probs, np.uint16, 2048)), z["softmax_probs"]
    assert np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1e-4)) < 5e-3        # LogitSoftcapSoftmaxTests.swift:46-49
    d_probs, tok = dev(z["sample_probs"]), zeros_bytes(4)

    def draw(*args, topk64=False):
        fn = k.lib.tf_sample_topk64 if topk64 else k.lib.tf_sample
        k.check(fn(k.handle, None, d_probs.data_ptr(), tok.data_ptr(), 1003, *args))
        return int(host(tok, np.uint32, 1)[0])

    assert draw(0.0, 0, 1.0, 1, 0) == int(z["sample_greedy"][0])
    for i, seed in enumerate(int(s) for s in z["sample_seeds"]):
        assert draw(1.0, 4, 1.0, seed, 0) == int(z["sample_top4"][i])
        assert draw(0.85, 0.95, seed, topk64=True) == int(z["sample_top64_p95_t085"][i])
        assert draw(1.3, 0, 0.3, seed, 0) == int(z["sample_nucleus_p30"][i])

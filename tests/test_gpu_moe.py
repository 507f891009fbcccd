"""GPU parity: router, routed experts (phase 1 / subset / phase 2), shared expert — through the C ABI, against the
CPU oracle.  Cases restate RouterTopKTests, MoEFusedFFNTests and SharedExpertInt4Tests of the reference."""
import numpy as np
import torch
import pytest

import refcases
from gpu_helpers import ctx, dev, device_view, host, tfk, within_north_star, zeros_bytes
from oracle import tfo

pytestmark = pytest.mark.gpu


def _router_tensors(weights, hidden, eff, escale, w_off=0):
    W, S, B = tfo.quantize_int8(weights)
    return W, S, B, dict(W=dev(W, w_off), S=dev(S), B=dev(B), h=dev(tfo.to_f16_bits(hidden)), eff=dev(tfo.bf16_bits_array(eff)),
                         pes=dev(tfo.bf16_bits_array(escale)), idx=zeros_bytes(32), wts=zeros_bytes(16))


def router_gpu(weights, hidden, eff, escale, w_off=0):
    W, S, B, t = _router_tensors(weights, hidden, eff, escale, w_off)
    e, d = W.shape
    k = ctx()
    k.check(k.lib.tf_router_gemma4(k.handle, None, t["W"].data_ptr(), w_off, t["S"].data_ptr(), 0, t["B"].data_ptr(), 0,
                                   t["h"].data_ptr(), t["eff"].data_ptr(), 0, t["pes"].data_ptr(), 0, t["idx"].data_ptr(),
                                   t["wts"].data_ptr(), e, d, 8))
    import torch
    torch.cuda.synchronize()
    return (W, S, B), host(t["idx"], np.uint32, 8), tfo.from_f16_bits(host(t["wts"], np.uint16, 8))


@pytest.mark.parametrize("w_off", [0, 1])
def test_production_router_matches_reference(w_off):
    weights, hidden, eff, escale = refcases.router_case_production()
    (W, S, B), idx, wts = router_gpu(weights, hidden, eff, escale, w_off)
    ref_idx, ref_w, _ = tfo.router_reference(W, S, B, hidden, eff, escale)
    assert list(idx) == list(ref_idx)
    assert np.max(np.abs(wts - ref_w)) < 5e-3


def test_production_router_resolves_near_tie_like_reference():
    weights, hidden, eff, escale = refcases.router_case_near_tie()
    (W, S, B), idx, _ = router_gpu(weights, hidden, eff, escale)
    assert list(idx) == [0, 1, 2, 3, 4, 5, 6, 8]
    assert list(idx) == list(tfo.router_reference(W, S, B, hidden, eff, escale)[0])


def test_router_at_production_shape_and_back_to_back_calls():
    # 128 experts x 2816, the shape BASELINE config 1 routes with; two calls in a row check the ticket counter resets
    rng = np.random.default_rng(0xA11)
    W, S, B = refcases.synthetic_int8(128, 2816, 0xA11)
    k = ctx()
    for trial in range(2):
        hidden_bits = refcases.normal_f16(2816, 0xA11 + trial)
        eff = rng.uniform(0.5, 1.5, 2816).astype(np.float32) / np.float32(np.sqrt(2816.0))
        escale = rng.uniform(0.6, 1.4, 128).astype(np.float32)
        eff_bits, pes_bits = tfo.bf16_bits_array(eff), tfo.bf16_bits_array(escale)
        idx, wts = zeros_bytes(32), zeros_bytes(16)
        k.router_gemma4(dev(W), dev(S), dev(B), dev(hidden_bits), dev(eff_bits), dev(pes_bits), idx, wts, 128, 2816)
        got_idx, got_w = host(idx, np.uint32, 8), tfo.from_f16_bits(host(wts, np.uint16, 8))
        ref_idx, ref_w, ref_logits = tfo.router_reference(W, S, B, tfo.from_f16_bits(hidden_bits), tfo.bf16_array_to_float(eff_bits),
                                                          tfo.bf16_array_to_float(pes_bits))
        logits = device_view(k.router_logits_ptr(), 128, "<f4")
        assert tfo.rel_error(logits, ref_logits) < 1e-4
        srt = np.sort(ref_logits)[::-1]
        if np.min(srt[:8] - srt[1:9]) > 1e-4 * np.max(np.abs(srt)):   # no near tie in the reference: order is pinned
            assert list(got_idx) == list(ref_idx)
            assert np.max(np.abs(got_w - ref_w)) < 5e-3
        assert abs(float(got_w.sum() / np.sum(tfo.bf16_array_to_float(pes_bits)[got_idx] * ref_w / tfo.bf16_array_to_float(pes_bits)[ref_idx])) - 1) < 0.2


def test_router_rejects_bad_contract():
    weights, hidden, eff, escale = refcases.router_case_production()
    W, S, B, t = _router_tensors(weights, hidden, eff, escale)
    k = ctx()
    def call(e, d, topk):
        return k.lib.tf_router_gemma4(k.handle, None, t["W"].data_ptr(), 0, t["S"].data_ptr(), 0, t["B"].data_ptr(), 0, t["h"].data_ptr(),
                                      t["eff"].data_ptr(), 0, t["pes"].data_ptr(), 0, t["idx"].data_ptr(), t["wts"].data_ptr(), e, d, topk)
    assert call(16, 128, 4) == tfk.TF_ERR_INVALID_ARGUMENT      # topK must be 8 (MoE.swift:123)
    assert call(257, 128, 8) == tfk.TF_ERR_INVALID_ARGUMENT     # numExperts <= 256 (MoE.swift:122)
    assert call(16, 100, 8) == tfk.TF_ERR_INVALID_ARGUMENT      # d % 64 (MoE.swift:121)


def _moe_buffers(c, blob_prefix=None):
    blobs = [dev(b, 0 if blob_prefix is None else blob_prefix(i)) for i, b in enumerate(c["blobs"])]
    ptrs = [t.data_ptr() + (0 if blob_prefix is None else blob_prefix(i)) for i, t in enumerate(blobs)]
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    return blobs, ptrs, off


def run_moe(c, split=False, blob_prefix=None, pool_mode=False):
    d, f = c["d"], c["f"]
    k = ctx()
    blobs, ptrs, off = _moe_buffers(c, blob_prefix)
    x, res, rw = dev(c["x_bits"]), dev(c["residual_bits"]), dev(c["routing_w_bits"])
    acts, y = zeros_bytes(8 * f * 2), zeros_bytes(d * 2 + 32, 0xEE)
    if pool_mode:
        stride = (c["blobs"][0].size + 63) // 64 * 64
        pool_np = np.zeros(16 * stride, np.uint8)
        perm = [5, 11, 2, 7, 0, 15, 9, 3]
        for slot, e in enumerate(perm):
            pool_np[e * stride:e * stride + c["blobs"][slot].size] = c["blobs"][slot]
        pool, d_perm = dev(pool_np), dev(np.array(perm, np.uint32))
        routed = k.routed_from_pool(pool, stride, d_perm, 16)
        keep = (pool, d_perm)
    else:
        routed = k.routed_from_pointers(ptrs)
        keep = blobs
    if split:
        for slots in ([0, 1, 2, 3], [4, 5, 6, 7]):
            d_slots = dev(np.array(slots, np.uint32))
            k.moe_phase1(routed, off, x, acts, d, f, active_slots=d_slots, active_count=4)
    else:
        k.moe_phase1(routed, off, x, acts, d, f)
    k.moe_phase2(routed, off, acts, rw, res, y, d, f)
    out = host(y, np.uint16, d)
    assert np.all(host(y, np.uint8)[d * 2:] == 0xEE)
    del keep
    return out, host(acts, np.uint16, 8 * f)


def test_production_routed_pipeline_and_hit_split_match_reference():
    # MoEFusedFFNTests.swift:17-159
    c = refcases.moe_fused_case()
    d, f = c["d"], c["f"]
    full, acts = run_moe(c)
    split, acts_split = run_moe(c, split=True)
    assert np.array_equal(full, split) and np.array_equal(acts, acts_split)     # bitwise
    expected = tfo.moe_apply_streamed_routed(c["blobs"], c["off"], tfo.from_f16_bits(c["x_bits"]), tfo.from_f16_bits(c["residual_bits"]),
                                             tfo.from_f16_bits(c["routing_w_bits"]), d, f)
    got = tfo.from_f16_bits(full)
    assert tfo.rel_error(got, expected) < tfo.Tolerance.fp16ChainedReduction
    assert within_north_star(got, expected)
    # against the kernel-order restatement the device may differ only by summation order: a couple of fp16 ulps
    k_acts = tfo.k_moe_phase1(c["blobs"], c["off"], c["x_bits"], d, f)
    assert np.max(np.abs(tfo.from_f16_bits(acts) - tfo.from_f16_bits(k_acts))) < 2e-3
    k_y = tfo.from_f16_bits(tfo.k_moe_phase2(c["blobs"], c["off"], acts, c["routing_w_bits"], c["residual_bits"], d, f))
    assert np.max(np.abs(got - k_y)) < 2e-3


def test_routed_pipeline_pool_indirection_and_unaligned_blobs_agree():
    c = refcases.moe_fused_case()
    full, acts = run_moe(c)
    pooled, acts_pool = run_moe(c, pool_mode=True)
    assert np.array_equal(full, pooled) and np.array_equal(acts, acts_pool)
    # blobs bound at 2-aligned, non-16-aligned bases take the 16-bit-load path: same sums up to order
    odd, _ = run_moe(c, blob_prefix=lambda i: 2 + 4 * i)
    assert np.max(np.abs(tfo.from_f16_bits(odd) - tfo.from_f16_bits(full))) < 2e-3


@pytest.mark.parametrize("d,f", [(2816, 704), (2816, 64), (704, 128)])
def test_routed_pipeline_production_shape(d, f):
    # BASELINE config 1 expert shape (gate/up 704 x 2816, down 2816 x 704), synthetic nibbles/scales
    rng = np.random.default_rng(d + f)
    blobs, off = [], None
    for e in range(8):
        blob, off = tfo.make_blob(refcases.synthetic_int4(f, d, 0x100 + e, "gate"), refcases.synthetic_int4(f, d, 0x100 + e, "up"),
                                  refcases.synthetic_int4(d, f, 0x100 + e, "down"))
        blobs.append(blob)
    c = dict(blobs=blobs, off=off, d=d, f=f, x_bits=refcases.normal_f16(d, 0x77),
             residual_bits=np.zeros(d, np.uint16),
             routing_w_bits=tfo.to_f16_bits(rng.dirichlet(np.ones(8)).astype(np.float32)))
    full, acts = run_moe(c)
    expected = tfo.moe_apply_streamed_routed(blobs, off, tfo.from_f16_bits(c["x_bits"]), np.zeros(d, np.float32),
                                             tfo.from_f16_bits(c["routing_w_bits"]), d, f, threads=8)
    got = tfo.from_f16_bits(full)
    assert tfo.rel_error(got, expected) < tfo.Tolerance.fp16ChainedReduction
    assert within_north_star(got, expected, abs_=1e-3 * max(1.0, float(np.max(np.abs(expected)))))
    split, _ = run_moe(c, split=True)
    assert np.array_equal(full, split)


def test_moe_rejects_bad_contract():
    c = refcases.moe_fused_case()
    k = ctx()
    blobs, ptrs, off = _moe_buffers(c)
    x, acts = dev(c["x_bits"]), zeros_bytes(8 * 64 * 2, 0xEE)
    routed = k.routed_from_pointers(ptrs)
    assert k.moe_phase1(routed, off, x, acts, 128, 64, top_k=4, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT   # MoE.swift:298
    missing = k.routed_from_pointers(ptrs[:7])
    assert k.moe_phase1(missing, off, x, acts, 128, 64, raise_on_error=False) == tfk.TF_ERR_INVALID_ARGUMENT          # MoE.swift:299
    # activeCount == 0: nothing is enqueued (MoE.swift:231)
    assert k.moe_phase1(routed, off, x, acts, 128, 64, active_slots=dev(np.zeros(1, np.uint32)), active_count=0) == tfk.TF_OK
    assert np.all(host(acts, np.uint8) == 0xEE)


def _proj(dW, dS, dB, rows, cols):
    return tfk.projection(dW, dS, dB, rows, cols)


def run_shared(c, scratch_halves=None, weight_bits=4):
    d, f = c["d"], c["f"]
    k = ctx()
    t = {n: [dev(a) for a in c[n]] for n in ("gate", "up", "down")}
    x, y = dev(c["x_bits"]), zeros_bytes(d * 2)
    n_s = (scratch_halves if scratch_halves is not None else f) * 2
    sg, su, sa = zeros_bytes(n_s), zeros_bytes(n_s), zeros_bytes(n_s)
    rc = k.shared_expert_int4(x, _proj(*t["gate"], f, d), _proj(*t["up"], f, d), _proj(*t["down"], d, f), y, sg, su, sa,
                              weight_bits=weight_bits, raise_on_error=False)
    return rc, host(y, np.uint16, d), (host(sg, np.uint16), host(su, np.uint16), host(sa, np.uint16))


def test_shared_expert_int4_matches_affine_reference():
    # SharedExpertInt4Tests.swift:11-53
    c = refcases.shared_expert_case()
    rc, y, (sg, su, sa) = run_shared(c)
    assert rc == tfk.TF_OK
    ref = tfo.shared_expert_ref(c["gate"], c["up"], c["down"], tfo.from_f16_bits(c["x_bits"]))
    assert tfo.rel_error(tfo.from_f16_bits(y), ref) < tfo.Tolerance.quantInt4 * 4
    # stage boundaries: gate/up are fp16-rounded GEMV outputs, act = gelu_mul_fp16 of those
    assert tfo.rel_error(tfo.from_f16_bits(sg), tfo.int4_gemv_ref(*c["gate"], tfo.from_f16_bits(c["x_bits"]))) < tfo.Tolerance.fp16Reduction
    want_act = tfo.from_f16_bits(tfo.k_gelu_mul_fp16(sg, su))
    assert np.max(np.abs(tfo.from_f16_bits(sa) - want_act)) <= 1e-3


def test_shared_expert_production_shape_fused_gate_up():
    # shared expert of the production model: gate/up 2112 x 2816, down 2816 x 2112
    d, f = 2816, 2112
    c = dict(d=d, f=f, x_bits=refcases.normal_f16(d, 0x5E), gate=refcases.synthetic_int4(f, d, 0x5E, "g"),
             up=refcases.synthetic_int4(f, d, 0x5E, "u"), down=refcases.synthetic_int4(d, f, 0x5E, "d"))
    rc, y, (sg, su, sa) = run_shared(c)
    assert rc == tfk.TF_OK
    x = tfo.from_f16_bits(c["x_bits"])
    g_ref, u_ref = tfo.int4_gemv_ref(*c["gate"], x, threads=8), tfo.int4_gemv_ref(*c["up"], x, threads=8)
    assert tfo.rel_error(tfo.from_f16_bits(sg), g_ref) < tfo.Tolerance.fp16Reduction
    assert tfo.rel_error(tfo.from_f16_bits(su), u_ref) < tfo.Tolerance.fp16Reduction
    want_act = tfo.from_f16_bits(tfo.k_gelu_mul_fp16(sg, su))
    assert tfo.rel_error(tfo.from_f16_bits(sa), want_act) < 2e-3
    y_ref = tfo.int4_gemv_ref(*c["down"], tfo.from_f16_bits(sa), threads=8)
    assert tfo.rel_error(tfo.from_f16_bits(y), y_ref) < tfo.Tolerance.fp16Reduction
    full_ref = tfo.shared_expert_ref(c["gate"], c["up"], c["down"], x, threads=8)
    assert tfo.rel_error(tfo.from_f16_bits(y), full_ref) < tfo.Tolerance.fp16ChainedReduction


def test_shared_expert_errors():
    c = refcases.shared_expert_case()
    assert run_shared(c, weight_bits=3)[0] == tfk.TF_ERR_UNSUPPORTED_BITS        # SharedExpertInt4.swift:110
    assert run_shared(c, weight_bits=16)[0] == tfk.TF_ERR_UNSUPPORTED_BITS
    assert run_shared(c, scratch_halves=c["f"] - 1)[0] == tfk.TF_ERR_SCRATCH_TOO_SMALL   # :46-50
    bad = dict(c)
    bad["down"] = c["gate"]
    k = ctx()
    t = {n: [dev(a) for a in c[n]] for n in ("gate", "up")}
    x, y, s = dev(c["x_bits"]), zeros_bytes(256), zeros_bytes(128)
    rc = k.shared_expert_int4(x, _proj(*t["gate"], 64, 128), _proj(*t["up"], 64, 128), _proj(*t["gate"], 64, 128), y, s, s, s, raise_on_error=False)
    assert rc == tfk.TF_ERR_DIMENSION_MISMATCH                                    # :41-45


# ---------------------------------------------------------------------------------------------------- shared expert, 8-bit
def _int8_case(d, f, seed, weight_range=0.4):
    rng = np.random.default_rng(seed)
    mats = {name: tfo.quantize_int8(rng.uniform(-weight_range, weight_range, shape).astype(np.float32))       # SharedExpertInt8Tests.swift:50-60
            for name, shape in (("gate", (f, d)), ("up", (f, d)), ("down", (d, f)))}
    return dict(d=d, f=f, x_bits=tfo.to_f16_bits(rng.uniform(-0.4, 0.4, d).astype(np.float32)), **mats)


def _gelu64(g):
    g = g.astype(np.float64)
    return 0.5 * g * (1.0 + np.tanh(0.7978845608028654 * (g + 0.044715 * g ** 3)))


def _int8_reference(c):
    # SharedExpertInt8Tests.swift:61-70: the reference GEMVs, the activation rounded through fp16 once, the down GEMV
    x = tfo.from_f16_bits(c["x_bits"])
    g, u = tfo.int8_gemv_ref(*c["gate"], x, threads=8), tfo.int8_gemv_ref(*c["up"], x, threads=8)
    act = tfo.from_f16_bits(tfo.to_f16_bits((_gelu64(g) * u).astype(np.float32)))
    return g, u, tfo.int8_gemv_ref(*c["down"], act, threads=8)


def _run_int8(c, through_runtime, pad=0):
    k = ctx()
    d, f = c["d"], c["f"]
    t = {name: tuple(dev(np.concatenate([np.zeros(pad, np.uint8), np.ascontiguousarray(a).view(np.uint8).ravel()])) for a in c[name])
         for name in ("gate", "up", "down")}
    def proj(name, rows, cols):
        w, s_, b = t[name]
        return tfk.Projection(w.data_ptr(), pad, s_.data_ptr(), pad, b.data_ptr(), pad, rows, cols)
    x, y, sa = dev(c["x_bits"]), zeros_bytes(d * 2), zeros_bytes(f * 2)
    g, u, dn = proj("gate", f, d), proj("up", f, d), proj("down", d, f)
    import ctypes as C
    if through_runtime:      # SharedExpertRuntime with weightBits 8: the scratch of gate and up is not used
        sg = zeros_bytes(2)
        rc = k.lib.tf_shared_expert_int4(k.handle, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(u), C.byref(dn), y.data_ptr(), 0, d * 2,
                                         sg.data_ptr(), 0, 2, sg.data_ptr(), 0, 2, sa.data_ptr(), 0, f * 2, 8, tfk.TF_BF16)
    else:
        rc = k.lib.tf_shared_expert_int8(k.handle, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(u), C.byref(dn), y.data_ptr(), 0, d * 2,
                                         sa.data_ptr(), 0, f * 2, tfk.TF_BF16)
    return rc, host(y, np.uint16, d), host(sa, np.uint16, f), (t, x, y, sa, g, u, dn)


@pytest.mark.parametrize("d,f,pad", [(256, 128, 0), (2816, 2112, 0), (5120, 64, 0), (256, 128, 2)])     # small, production, long rows, unaligned weights
@pytest.mark.parametrize("through_runtime", [False, True])
def test_shared_expert_int8_matches_reference(d, f, pad, through_runtime):
    c = _int8_case(d, f, 0x601 + d + f)
    rc, y, act, _ = _run_int8(c, through_runtime, pad)
    assert rc == tfk.TF_OK
    g_ref, u_ref, y_ref = _int8_reference(c)
    assert tfo.rel_error(tfo.from_f16_bits(y), y_ref) < tfo.Tolerance.quantInt8 * 4                 # SharedExpertInt8Tests.swift:110
    # stage boundary: act = gelu_mul_fp16 of the fp16-rounded gate and up sums (dequant_int8.metal:152-156)
    want_act = tfo.from_f16_bits(tfo.k_gelu_mul_fp16(tfo.to_f16_bits(g_ref), tfo.to_f16_bits(u_ref)))
    assert np.max(np.abs(tfo.from_f16_bits(act) - want_act)) <= 2e-3 * max(1.0, float(np.max(np.abs(want_act))))
    assert tfo.rel_error(tfo.from_f16_bits(y), tfo.int8_gemv_ref(*c["down"], tfo.from_f16_bits(act), threads=8)) < tfo.Tolerance.fp16Reduction


def test_shared_expert_int8_phases_and_contract():
    import ctypes as C
    c = _int8_case(256, 128, 0x602)
    rc, y, act, (t, x, yb, sa, g, u, dn) = _run_int8(c, False)
    assert rc == tfk.TF_OK
    k = ctx()
    lib, h = k.lib, k.handle
    d, f = 256, 128
    # encodePhase1 + encodeDown give what encode gives
    y2, sa2 = zeros_bytes(d * 2), zeros_bytes(f * 2)
    k.check(lib.tf_shared_expert_int8_phase1(h, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(u), sa2.data_ptr(), 0, f * 2, tfk.TF_BF16))
    k.check(lib.tf_shared_expert_int8_down(h, None, C.byref(dn), y2.data_ptr(), 0, d * 2, sa2.data_ptr(), 0, f * 2, tfk.TF_BF16))
    assert np.array_equal(host(y2, np.uint16, d), y) and np.array_equal(host(sa2, np.uint16, f), act)
    # SharedExpertInt8.swift:75-97
    assert lib.tf_shared_expert_int8(h, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(dn), C.byref(dn), yb.data_ptr(), 0, d * 2,
                                     sa.data_ptr(), 0, f * 2, tfk.TF_BF16) == tfk.TF_ERR_DIMENSION_MISMATCH        # gate/up shapes differ
    assert lib.tf_shared_expert_int8(h, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(u), C.byref(g), yb.data_ptr(), 0, d * 2,
                                     sa.data_ptr(), 0, f * 2, tfk.TF_BF16) == tfk.TF_ERR_DIMENSION_MISMATCH        # down is not the transpose shape
    assert lib.tf_shared_expert_int8(h, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(u), C.byref(dn), yb.data_ptr(), 0, d * 2,
                                     sa.data_ptr(), 0, f * 2 - 2, tfk.TF_BF16) == tfk.TF_ERR_SCRATCH_TOO_SMALL
    assert lib.tf_shared_expert_int8(h, None, x.data_ptr(), 2, d * 2, C.byref(g), C.byref(u), C.byref(dn), yb.data_ptr(), 0, d * 2,
                                     sa.data_ptr(), 0, f * 2, tfk.TF_BF16) == tfk.TF_ERR_SCRATCH_TOO_SMALL         # x range exceeds its buffer
    assert lib.tf_shared_expert_int8(h, None, x.data_ptr(), 0, d * 2, C.byref(g), C.byref(u), C.byref(dn), yb.data_ptr(), 2, d * 2,
                                     sa.data_ptr(), 0, f * 2, tfk.TF_BF16) == tfk.TF_ERR_SCRATCH_TOO_SMALL         # y range exceeds its buffer


@pytest.mark.parametrize("d,f,rows,pad", [(256, 128, 3, 8), (2816, 2112, 13, 0), (256, 128, 5, 3), (1024, 64, 1, 0), (2816, 2112, 37, 0),
                                         (256, 128, 40, 8), (256, 128, 33, 5)])
def test_prefill_shared_expert_block_with_8_bit_weights_is_the_row_chain(d, f, rows, pad):
    # PrefillSharedExpert(weightBits: 8) (PrefillSharedExpert.swift:7-8).  Fewer than 16 rows: every row as the 8-bit single-row
    # chain leaves it, bit for bit - rows in groups against each weight row where the operands are aligned, one by one otherwise
    # (odd stride, one row).  From 16 aligned rows on: weights expanded to fp16 and multiplied on the matrix cores, within the
    # 8-bit shared expert's tolerance of the row chain.
    import ctypes as C
    c = _int8_case(d, f, 0x603 + d)
    _, _, _, (t, _, _, sa, g, u, dn) = _run_int8(c, False)
    k = ctx()
    stride = d + pad
    rng = np.random.default_rng(0x603)
    xs = tfo.to_f16_bits(rng.uniform(-0.4, 0.4, rows * stride).astype(np.float32))
    x, y = dev(xs), dev(np.full(rows * stride, 0x7BFF, np.uint16))
    sg = zeros_bytes(f * 2)
    k.check(k.lib.tf_prefill_shared_expert_int4_block(k.handle, None, x.data_ptr(), 0, y.data_ptr(), 0, C.byref(g), C.byref(u), C.byref(dn),
                                                      sg.data_ptr(), 0, f * 2, sg.data_ptr(), 0, f * 2, sa.data_ptr(), 0, f * 2, rows, d, f,
                                                      stride, stride, 8, tfk.TF_BF16))
    got = host(y, np.uint16).reshape(rows, stride)
    assert np.all(got[:, d:] == 0x7BFF)
    for r in range(rows):
        y1 = zeros_bytes(d * 2)
        k.check(k.lib.tf_shared_expert_int8(k.handle, None, x.data_ptr(), r * stride * 2, (r * stride + d) * 2, C.byref(g), C.byref(u), C.byref(dn),
                                            y1.data_ptr(), 0, d * 2, sa.data_ptr(), 0, f * 2, tfk.TF_BF16))
        row_chain = host(y1, np.uint16, d)
        if rows >= 16 and stride % 8 == 0:
            assert tfo.rel_error(tfo.from_f16_bits(got[r, :d]), tfo.from_f16_bits(row_chain)) < tfo.Tolerance.quantInt8 * 4
        else:
            assert np.array_equal(row_chain, got[r, :d])



def test_8_bit_block_on_matrix_cores_with_small_scales():
    # From 16 rows on the 8-bit block rounds every weight to fp16 (half(q s + b), the reference's staged-affine rounding point,
    # tensorops.metal:57-94) while the row chain keeps q s + b in fp32.  Weights of magnitude 1e-3 and less have scales near
    # 8e-6, far below fp16's normal range: converted to fp16 directly they would lose mantissa bits (0.7 % error measured), so
    # the kernel carries a scale as mantissa and power of two.  The block must stay within the 8-bit shared expert's tolerance
    # of the row chain.
    import ctypes as C
    d, f, rows = 1024, 256, 32
    c = _int8_case(d, f, 0x6A1, weight_range=1e-3)
    _, _, _, (t, _, _, sa, g, u, dn) = _run_int8(c, False)
    k = ctx()
    rng = np.random.default_rng(0x6A1)
    xs = tfo.to_f16_bits(rng.uniform(-200.0, 200.0, rows * d).astype(np.float32))      # large activations keep the sums in fp16's normal range
    x, y = dev(xs), zeros_bytes(rows * d * 2)
    sg = zeros_bytes(f * 2)
    k.check(k.lib.tf_prefill_shared_expert_int4_block(k.handle, None, x.data_ptr(), 0, y.data_ptr(), 0, C.byref(g), C.byref(u), C.byref(dn),
                                                      sg.data_ptr(), 0, f * 2, sg.data_ptr(), 0, f * 2, sa.data_ptr(), 0, f * 2, rows, d, f,
                                                      d, d, 8, tfk.TF_BF16))
    got = tfo.from_f16_bits(host(y, np.uint16).reshape(rows, d))
    assert float(np.max(np.abs(got))) > 1e-3          # the case is not degenerate
    for r in range(rows):
        y1 = zeros_bytes(d * 2)
        k.check(k.lib.tf_shared_expert_int8(k.handle, None, x.data_ptr(), r * d * 2, (r + 1) * d * 2, C.byref(g), C.byref(u), C.byref(dn),
                                            y1.data_ptr(), 0, d * 2, sa.data_ptr(), 0, f * 2, tfk.TF_BF16))
        assert tfo.rel_error(got[r], tfo.from_f16_bits(host(y1, np.uint16, d))) < tfo.Tolerance.quantInt8 * 4


# ---------------------------------------------------------------------------------------------------- shared expert, block of rows
def _shared_block_case(rows, d, f, seed):
    c = dict(d=d, f=f, gate=refcases.synthetic_int4(f, d, seed, "g"), up=refcases.synthetic_int4(f, d, seed, "u"),
             down=refcases.synthetic_int4(d, f, seed, "d"))
    c["x_bits"] = refcases.normal_f16(rows * d, seed).reshape(rows, d)
    return c


SENTINEL = np.float16(-7.25).view(np.uint16)   # PrefillSharedExpertTests.swift:13


def run_shared_block(c, rows, x_stride, y_stride, weight_bits=4, scratch_halves=None):
    d, f = c["d"], c["f"]
    k = ctx()
    t = {n: [dev(a) for a in c[n]] for n in ("gate", "up", "down")}
    x_host = np.full((max(rows, 1), max(x_stride, d)), SENTINEL, np.uint16)   # a too-small stride is refused before any read
    x_host[:rows, :d] = c["x_bits"][:rows]
    keep = dict(x=dev(x_host), y=dev(np.full((max(rows, 1), max(y_stride, d)), SENTINEL, np.uint16)))
    n_s = (scratch_halves if scratch_halves is not None else f) * 2
    sg, su, sa = zeros_bytes(n_s), zeros_bytes(n_s), zeros_bytes(n_s)
    rc = k.prefill_shared_expert_block(keep["x"], _proj(*t["gate"], f, d), _proj(*t["up"], f, d), _proj(*t["down"], d, f), keep["y"],
                                       sg, su, sa, rows, d, f, x_stride=x_stride, y_stride=y_stride, weight_bits=weight_bits,
                                       raise_on_error=False)
    return rc, host(keep["y"], np.uint16).reshape(max(rows, 1), max(y_stride, d))


def _repeated_rows(c, rows):
    out = []
    for r in range(rows):
        one = dict(c)
        one["x_bits"] = c["x_bits"][r]
        rc, y, _ = run_shared(one)
        assert rc == tfk.TF_OK
        out.append(y)
    return np.stack(out)


def test_prefill_shared_expert_block_equals_repeated_rows_bit_for_bit():
    # PrefillSharedExpertTests.swift:8-13,178-243: 4 rows, d 128, f 64, x stride 144, y stride 137, sentinel padding
    rows, d, f = 4, 128, 64
    c = _shared_block_case(rows, d, f, 0xC0FFEE)
    rc, y = run_shared_block(c, rows, 144, 137)
    assert rc == tfk.TF_OK
    assert np.array_equal(y[:, :d], _repeated_rows(c, rows))
    assert np.all(y[:, d:] == SENTINEL)


@pytest.mark.parametrize("rows,d,f,x_stride,y_stride", [(8, 128, 64, 144, 136), (40, 128, 64, 128, 137), (133, 256, 192, 264, 256),
                                                       (200, 2816, 2112, 2816, 2816)])
def test_prefill_shared_expert_block_on_matrix_cores(rows, d, f, x_stride, y_stride):
    c = _shared_block_case(rows, d, f, 0x5B + rows)
    rc, y = run_shared_block(c, rows, x_stride, y_stride)
    assert rc == tfk.TF_OK
    assert np.all(y[:, d:] == SENTINEL)
    check = range(rows) if rows <= 40 else [0, 1, 31, 32, 127, 128, rows - 2, rows - 1]
    for r in check:
        ref = tfo.shared_expert_ref(c["gate"], c["up"], c["down"], tfo.from_f16_bits(c["x_bits"][r]), threads=8)
        assert tfo.rel_error(tfo.from_f16_bits(y[r, :d]), ref) < 6e-3, r       # SharedExpertInt4Tests.swift:52
    # and against the single-row chain of the same library (fp32 weights there, fp16-rounded weights here)
    chain = _repeated_rows(c, min(rows, 3))
    for r in range(min(rows, 3)):
        assert tfo.rel_error(tfo.from_f16_bits(y[r, :d]), tfo.from_f16_bits(chain[r])) < 6e-3


def test_prefill_shared_expert_block_with_gate_and_up_scales_far_apart_takes_the_row_chain():
    # the fused gate / up tiles address the scale arrays of both matrices through one 32-bit-offset descriptor; arrays more than
    # 2 GiB apart are outside it, and the rows go one by one through the single-row chain instead (bit-identical to it)
    rows, d, f = 16, 128, 64
    c = _shared_block_case(rows, d, f, 0xFA2)
    k = ctx()
    spacer_bytes = (1 << 31) + (1 << 20)
    arena = torch.empty(spacer_bytes + (1 << 16), dtype=torch.uint8, device="cuda")      # one allocation: gate scales at its start, up scales past 2 GiB
    gate_s, up_s = c["gate"][1], c["up"][1]
    arena[:gate_s.nbytes] = torch.from_numpy(np.ascontiguousarray(gate_s).view(np.uint8).ravel()).cuda()
    arena[spacer_bytes:spacer_bytes + up_s.nbytes] = torch.from_numpy(np.ascontiguousarray(up_s).view(np.uint8).ravel()).cuda()
    t = {n: [dev(a) for a in c[n]] for n in ("gate", "up", "down")}
    pg, pu = _proj(*t["gate"], f, d), _proj(*t["up"], f, d)
    pg.scales, pg.scales_offset = arena.data_ptr(), 0
    pu.scales, pu.scales_offset = arena.data_ptr(), spacer_bytes
    x, y = dev(c["x_bits"]), dev(np.full((rows, d), SENTINEL, np.uint16))
    sg, su, sa = zeros_bytes(f * 2), zeros_bytes(f * 2), zeros_bytes(f * 2)
    rc = k.prefill_shared_expert_block(x, pg, pu, _proj(*t["down"], d, f), y, sg, su, sa, rows, d, f, raise_on_error=False)
    assert rc == tfk.TF_OK, k.last_error()
    assert np.array_equal(host(y, np.uint16).reshape(rows, d), _repeated_rows(c, rows))
    del arena


def test_prefill_shared_expert_block_contract():
    c = _shared_block_case(4, 128, 64, 7)
    assert run_shared_block(c, 0, 128, 128)[0] == tfk.TF_OK                       # queryCount 0: nothing to do
    assert np.all(run_shared_block(c, 0, 128, 128)[1] == SENTINEL)
    assert run_shared_block(c, 4, 127, 128)[0] == tfk.TF_ERR_INVALID_ARGUMENT     # PrefillSharedExpert.swift:35
    assert run_shared_block(c, 4, 128, 127)[0] == tfk.TF_ERR_INVALID_ARGUMENT     # :36
    assert run_shared_block(c, 4, 128, 128, weight_bits=16)[0] == tfk.TF_ERR_UNSUPPORTED_BITS
    assert run_shared_block(c, 4, 128, 128, scratch_halves=63)[0] == tfk.TF_ERR_SCRATCH_TOO_SMALL
    big = _shared_block_case(16, 128, 64, 7)
    assert run_shared_block(big, 16, 128, 128, scratch_halves=63)[0] == tfk.TF_ERR_SCRATCH_TOO_SMALL
    k = ctx()
    t = {n: [dev(a) for a in c[n]] for n in ("gate", "up")}
    x, y, s = dev(c["x_bits"]), zeros_bytes(4 * 256), zeros_bytes(128)
    rc = k.prefill_shared_expert_block(x, _proj(*t["gate"], 64, 128), _proj(*t["up"], 64, 128), _proj(*t["gate"], 64, 128), y, s, s, s,
                                       4, 128, 64, raise_on_error=False)
    assert rc == tfk.TF_ERR_DIMENSION_MISMATCH                                   # :37-42


# ---------------------------------------------------------------------------------------------------- decode step
def _decode_step_case(d, f, num_experts, seed):
    rng = np.random.default_rng(seed)
    blobs, off = [], None
    for e in range(num_experts):
        blob, off = tfo.make_blob(refcases.synthetic_int4(f, d, seed + e, "gate"), refcases.synthetic_int4(f, d, seed + e, "up"),
                                  refcases.synthetic_int4(d, f, seed + e, "down"))
        blobs.append(blob)
    stride = (blobs[0].size + 63) // 64 * 64
    pool = np.zeros(num_experts * stride, np.uint8)
    for e, blob in enumerate(blobs):
        pool[e * stride:e * stride + blob.size] = blob
    rW, rS, rB = refcases.synthetic_int8(num_experts, d, seed)
    eff = rng.uniform(0.5, 1.5, d).astype(np.float32) / np.float32(np.sqrt(d))
    gain = rng.uniform(0.6, 1.4, num_experts).astype(np.float32)
    return dict(blobs=blobs, off=off, stride=stride, pool=pool, rW=rW, rS=rS, rB=rB, eff_bits=tfo.bf16_bits_array(eff),
                gain_bits=tfo.bf16_bits_array(gain), x_bits=refcases.normal_f16(d, seed + 7),
                residual_bits=refcases.normal_f16(d, seed + 9))


def _decode_step_call(k, t, c, d, f, num_experts, outs, scale_dtype=tfk.TF_BF16):
    idx, wts, acts, y = outs
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    return k.lib.tf_moe_decode_step(k.handle, None, t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0, t["x"].data_ptr(),
                                    t["eff"].data_ptr(), 0, t["gain"].data_ptr(), 0, t["pool"].data_ptr(), c["stride"], num_experts,
                                    off, t["x"].data_ptr(), acts.data_ptr(), t["res"].data_ptr(), y.data_ptr(), idx.data_ptr(),
                                    wts.data_ptr(), d, f, 8, scale_dtype)


def _decode_step_tensors(c):
    return dict(pool=dev(c["pool"]), rW=dev(c["rW"]), rS=dev(c["rS"]), rB=dev(c["rB"]), eff=dev(c["eff_bits"]), gain=dev(c["gain_bits"]),
                x=dev(c["x_bits"]), res=dev(c["residual_bits"]))


def _fresh_outs(d, f):
    return zeros_bytes(32), zeros_bytes(16), zeros_bytes(8 * f * 2), zeros_bytes(d * 2)


def _read_outs(outs, d, f):
    idx, wts, acts, y = outs
    return host(idx, np.uint32, 8), host(wts, np.uint16, 8), host(acts, np.uint16, 8 * f), host(y, np.uint16, d)


# (2816, 704, 128) is the production shape
@pytest.mark.parametrize("d,f,num_experts", [(2816, 704, 128), (2816, 704, 16), (3072, 128, 200), (2816, 128, 128), (704, 128, 16)])
@pytest.mark.parametrize("mode", ["default", "timed"])
def test_decode_step_equals_router_then_phases_and_the_reference(d, f, num_experts, mode):
    # one call (selection repeated inside phase 1 when the vector path applies) against the three wrapper calls of the
    # reference runner (RealForwardRunner.swift:1462-1685): bitwise the same indices, weights, activations and output;
    # "timed" also brackets the three launches with events
    import torch
    c = _decode_step_case(d, f, num_experts, 0x5EED + d + f)
    k = ctx()
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    t = _decode_step_tensors(c)
    outs = []
    for fused in (True, False):
        o = _fresh_outs(d, f)
        idx, wts, acts, y = o
        if fused:
            k.set_step_timing(mode == "timed")
            k.check(_decode_step_call(k, t, c, d, f, num_experts, o))
            if mode == "timed":
                times = k.last_step_timing()
                assert len(times) == 4 and all(0.0 <= v < 5e4 for v in times) and min(times[:3]) > 0.0
            k.set_step_timing(False)
            k.synchronize()
        else:
            k.router_gemma4(t["rW"], t["rS"], t["rB"], t["x"], t["eff"], t["gain"], idx, wts, num_experts, d)
            routed = k.routed_from_pool(t["pool"], c["stride"], idx, num_experts)
            k.moe_phase1(routed, off, t["x"], acts, d, f)
            k.moe_phase2(routed, off, acts, wts, t["res"], y, d, f)
        torch.cuda.synchronize()
        outs.append(_read_outs(o, d, f))
    for a, b in zip(outs[0], outs[1]):
        assert np.array_equal(a, b)
    got_idx, got_w_bits, _, got_y = outs[0]
    ref_idx, ref_w, _ = tfo.router_reference(c["rW"], c["rS"], c["rB"], tfo.from_f16_bits(c["x_bits"]),
                                             tfo.bf16_array_to_float(c["eff_bits"]), tfo.bf16_array_to_float(c["gain_bits"]))
    assert sorted(got_idx) == sorted(ref_idx)
    expected = tfo.moe_apply_streamed_routed([c["blobs"][e] for e in got_idx], c["off"], tfo.from_f16_bits(c["x_bits"]),
                                             tfo.from_f16_bits(c["residual_bits"]), tfo.from_f16_bits(got_w_bits), d, f, threads=8)
    assert within_north_star(tfo.from_f16_bits(got_y), expected, abs_=1e-3 * max(1.0, float(np.max(np.abs(expected)))))
    logits = device_view(k.router_logits_ptr(), num_experts, "<f4")
    assert tfo.rel_error(logits, tfo.router_reference(c["rW"], c["rS"], c["rB"], tfo.from_f16_bits(c["x_bits"]),
                                                      tfo.bf16_array_to_float(c["eff_bits"]), tfo.bf16_array_to_float(c["gain_bits"]))[2]) < 1e-4


def test_decode_steps_back_to_back_and_replayed_from_a_graph():
    # many steps in a row on one stream with changing activations and no host wait in between: every step must see its own
    # router result (logits and indices pass through device memory); then the same from a captured graph, replayed
    import torch
    d, f, num_experts, steps = 2816, 704, 128, 12
    c = _decode_step_case(d, f, num_experts, 0xBEE5)
    k = ctx()
    t = _decode_step_tensors(c)
    rng = np.random.default_rng(0xBEE5)
    xs = [dev(rng.standard_normal(d).astype(np.float16).view(np.uint16)) for _ in range(steps)]
    want = []
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    for i in range(steps):          # expected: the three wrapper calls, one step at a time
        o = _fresh_outs(d, f)
        idx, wts, acts, y = o
        k.router_gemma4(t["rW"], t["rS"], t["rB"], xs[i], t["eff"], t["gain"], idx, wts, num_experts, d)
        routed = k.routed_from_pool(t["pool"], c["stride"], idx, num_experts)
        k.moe_phase1(routed, off, xs[i], acts, d, f)
        k.moe_phase2(routed, off, acts, wts, t["res"], y, d, f)
        want.append(_read_outs(o, d, f))
    outs = [_fresh_outs(d, f) for _ in range(steps)]
    for i in range(steps):
        t["x"] = xs[i]
        k.check(_decode_step_call(k, t, c, d, f, num_experts, outs[i]))
    k.synchronize()
    for i in range(steps):
        for a, b in zip(_read_outs(outs[i], d, f), want[i]):
            assert np.array_equal(a, b), i
    assert len({tuple(w[0]) for w in want}) > 1      # the steps really chose different experts
    # graph: capture 4 steps on a side stream, replay three times with eager work between the replays
    side = torch.cuda.Stream()
    gouts = [_fresh_outs(d, f) for _ in range(4)]
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            for i in range(4):
                t["x"] = xs[i]
                idx, wts, acts, y = gouts[i]
                off = tfk.ExpertOffsets(*c["off"].as_tuple())
                k.check(k.lib.tf_moe_decode_step(k.handle, side.cuda_stream, t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0,
                                                 t["x"].data_ptr(), t["eff"].data_ptr(), 0, t["gain"].data_ptr(), 0, t["pool"].data_ptr(),
                                                 c["stride"], num_experts, off, t["x"].data_ptr(), acts.data_ptr(), t["res"].data_ptr(),
                                                 y.data_ptr(), idx.data_ptr(), wts.data_ptr(), d, f, 8, tfk.TF_BF16))
    for replay in range(3):
        for o in gouts:
            for buf in o:
                buf.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        for i in range(4):
            for a, b in zip(_read_outs(gouts[i], d, f), want[i]):
                assert np.array_equal(a, b), (replay, i)
        t["x"] = xs[5 + replay]                       # an eager step between the replays
        o = _fresh_outs(d, f)
        k.check(_decode_step_call(k, t, c, d, f, num_experts, o))
        k.synchronize()
        for a, b in zip(_read_outs(o, d, f), want[5 + replay]):
            assert np.array_equal(a, b)


def test_step_timing_needs_a_recorded_step():
    k = ctx()
    k.set_step_timing(True)
    import ctypes as C
    out = (C.c_float * 4)()
    assert k.lib.tf_ctx_last_step_timing(k.handle, out) == tfk.TF_ERR_UNAVAILABLE
    k.set_step_timing(False)

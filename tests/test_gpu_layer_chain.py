"""One decode step of a whole sliding-window decoder layer, enqueued through the C ABI with no host step in between, at the
production widths (d 2816, 16 query heads on 8 kv heads of 256, shared expert 2112, routed experts 704 wide; 16 experts to
keep the CPU side short).  Every stage reads what the previous stage left on the device, K and V land in their cache row
through offsets.  Each stage's output is checked against the oracle applied to that stage's own device inputs, so a
near-tie that tips differently upstream cannot hide or fake a defect downstream; when both sides pick the same experts the
end result is also compared with the oracle's chain run from the start."""
import ctypes as C

import numpy as np
import pytest

import refcases
import test_gpu_moe as M
from gpu_helpers import ctx, dev, host, tfk, zeros_bytes
from oracle import tfo

pytestmark = pytest.mark.gpu

D, HD, NQ, NKV = 2816, 256, 16, 8
F_SHARED, F_MOE, E = 2112, 704, 16
WINDOW, THETA, EPS, PAIRS, ATTN_SCALE, LAYER_SCALAR = 1024, 1e4, 1e-6, HD // 2, 1.0, 0.75
TOL = tfo.Tolerance.fp16ChainedReduction


def gemv(wsb, x_bits):
    """The GEMV kernels' arithmetic on the CPU, rounded to fp16 as they store it."""
    return tfo.to_f16_bits(tfo.k_int4_gemv(*wsb, x_bits))


def norm_weight(seed):
    return tfo.bf16_bits_array(1.0 + 0.1 * np.random.default_rng(seed).standard_normal(D).astype(np.float32))


def build_layer(seed):
    L = dict(q=refcases.synthetic_int4(NQ * HD, D, seed, "q"), k=refcases.synthetic_int4(NKV * HD, D, seed, "k"),
             v=refcases.synthetic_int4(NKV * HD, D, seed, "v"), o=refcases.synthetic_int4(D, NQ * HD, seed, "o"),
             gate=refcases.synthetic_int4(F_SHARED, D, seed, "sg"), up=refcases.synthetic_int4(F_SHARED, D, seed, "su"),
             down=refcases.synthetic_int4(D, F_SHARED, seed, "sd"))
    for i, name in enumerate(("input_norm", "post_attn", "pre_ffn", "pre_ffn2", "post_ffn1", "post_ffn2", "post_ffn")):
        L[name] = norm_weight(seed * 31 + i)
    rng = np.random.default_rng(seed + 5)
    L["q_norm"] = tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(HD).astype(np.float32))
    L["k_norm"] = tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(HD).astype(np.float32))
    L["moe"] = M._decode_step_case(D, F_MOE, E, seed + 11)
    return L


def test_decode_step_of_a_sliding_window_layer():
    L = build_layer(0x1A7E)
    position = 37                                            # rows 0..36 of the cache are history
    rng = np.random.default_rng(3)
    hidden0 = (rng.standard_normal(D) * 0.5).astype(np.float32).astype(np.float16).view(np.uint16)
    cache_rows = 64
    k_cache0 = (rng.uniform(-1, 1, cache_rows * NKV * HD)).astype(np.float32).astype(np.float16).view(np.uint16)
    v_cache0 = (rng.uniform(-1, 1, cache_rows * NKV * HD)).astype(np.float32).astype(np.float16).view(np.uint16)
    k = ctx()
    lib, h = k.lib, k.handle
    t = {name: [dev(a) for a in L[name]] for name in ("q", "k", "v", "o", "gate", "up", "down")}
    w = {name: dev(L[name]) for name in ("input_norm", "post_attn", "pre_ffn", "pre_ffn2", "post_ffn1", "post_ffn2", "post_ffn", "q_norm", "k_norm")}
    mt = M._decode_step_tensors(L["moe"])
    b = dict(hidden=dev(hidden0), x_norm=zeros_bytes(D * 2), q=zeros_bytes(NQ * HD * 2), k_cache=dev(k_cache0), v_cache=dev(v_cache0),
             attn=zeros_bytes(NQ * HD * 2), o=zeros_bytes(D * 2), dense_x=zeros_bytes(D * 2), routed_x=zeros_bytes(D * 2),
             router_x=zeros_bytes(D * 2), shared=zeros_bytes(D * 2), h1=zeros_bytes(D * 2), h2=zeros_bytes(D * 2),
             sg=zeros_bytes(F_SHARED * 2), su=zeros_bytes(F_SHARED * 2), sa=zeros_bytes(F_SHARED * 2), zero=zeros_bytes(D * 2),
             idx=zeros_bytes(32), wts=zeros_bytes(16), acts=zeros_bytes(8 * F_MOE * 2))
    row_bytes = NKV * HD * 2
    kv_off = position * row_bytes                             # the new K and V rows are written straight into the cache
    p = lambda name: b[name].data_ptr()
    snap = {}

    def grab(*names):
        for n in names:
            snap[n] = host(b[n], np.uint16).copy()

    # 1. input norm, q / k / v projections in one launch, per-head norm + RoPE in place (k, v inside the cache)
    k.check(lib.tf_rmsnorm_bf16w(h, None, p("hidden"), 0, w["input_norm"].data_ptr(), 0, p("x_norm"), 0, D, EPS))
    qkv = []
    for name in ("q", "k", "v"):
        qkv += [t[name][0].data_ptr(), 0, t[name][1].data_ptr(), 0, t[name][2].data_ptr(), 0]
    k.check(lib.tf_fused_qkv_gemv(h, None, *qkv, p("x_norm"), p("q"), 0, p("k_cache"), kv_off, p("v_cache"), kv_off, NQ * HD, NKV * HD, D, tfk.TF_BF16))
    grab("x_norm", "q", "k_cache", "v_cache")
    raw_q, raw_k, raw_v = snap["q"].copy(), snap["k_cache"].copy(), snap["v_cache"].copy()
    k.check(lib.tf_fused_qkv_epilogue(h, None, p("q"), 0, p("k_cache"), kv_off, p("v_cache"), kv_off, w["q_norm"].data_ptr(), 0,
                                      w["k_norm"].data_ptr(), 0, HD, NQ, NKV, position, THETA, PAIRS, EPS))
    grab("q", "k_cache", "v_cache")
    # 2. attention over rows [0, position], output projection
    seq_len = position + 1
    k.check(lib.tf_attention_swa(h, None, p("q"), 0, p("k_cache"), 0, p("v_cache"), 0, p("attn"), 0, HD, NQ, NKV, seq_len, WINDOW, ATTN_SCALE, 0))
    k.check(lib.tf_dequant_int4_gemv(h, None, t["o"][0].data_ptr(), 0, t["o"][1].data_ptr(), 0, t["o"][2].data_ptr(), 0, p("attn"), 0, p("o"), 0,
                                     D, NQ * HD, tfk.TF_BF16, tfk.TF_FP16))
    grab("attn", "o")
    hidden_before_setup = host(b["hidden"], np.uint16).copy()
    # 3. residual + the three inputs of the FFN sandwich
    k.check(lib.tf_fused_post_attn_setup(h, None, p("hidden"), p("o"), p("dense_x"), p("routed_x"), p("router_x"), w["post_attn"].data_ptr(), 0,
                                         w["pre_ffn"].data_ptr(), 0, w["pre_ffn2"].data_ptr(), 0, D, EPS))
    grab("hidden", "dense_x", "routed_x", "router_x")
    hidden_after_setup = snap["hidden"].copy()
    # 4. shared expert + its output norm; routed experts (router, gate/up, down) on the resident pool
    gate, up, down = (tfk.projection(*t[n], r, c) for n, r, c in (("gate", F_SHARED, D), ("up", F_SHARED, D), ("down", D, F_SHARED)))
    k.shared_expert_int4(b["dense_x"], gate, up, down, b["shared"], b["sg"], b["su"], b["sa"])
    k.check(lib.tf_rmsnorm_bf16w(h, None, p("shared"), 0, w["post_ffn1"].data_ptr(), 0, p("h1"), 0, D, EPS))
    off = tfk.ExpertOffsets(*L["moe"]["off"].as_tuple())
    k.check(lib.tf_moe_decode_step(h, None, mt["rW"].data_ptr(), 0, mt["rS"].data_ptr(), 0, mt["rB"].data_ptr(), 0, p("router_x"),
                                   mt["eff"].data_ptr(), 0, mt["gain"].data_ptr(), 0, mt["pool"].data_ptr(), L["moe"]["stride"], E, off,
                                   p("routed_x"), p("acts"), p("zero"), p("h2"), p("idx"), p("wts"), D, F_MOE, 8, tfk.TF_BF16))
    grab("shared", "h1", "h2", "acts")
    idx, wts = host(b["idx"], np.uint32, 8), host(b["wts"], np.uint16, 8)
    # 5. both branches folded back into the residual stream
    k.check(lib.tf_fused_layer_tail(h, None, p("h2"), p("h1"), p("hidden"), w["post_ffn2"].data_ptr(), 0, w["post_ffn"].data_ptr(), 0, D, EPS, LAYER_SCALAR))
    hidden_out = host(b["hidden"], np.uint16)

    f = tfo.from_f16_bits
    close = lambda got, want, tol=TOL: tfo.rel_error(f(got), f(want)) < tol
    # ---- stage by stage, each against the oracle on the device's own inputs
    assert close(snap["x_norm"], tfo.k_rmsnorm_bf16w(hidden0, L["input_norm"], EPS))
    assert close(raw_q, gemv(L["q"], snap["x_norm"]))
    new_row = slice(position * NKV * HD, (position + 1) * NKV * HD)
    assert close(raw_k[new_row], gemv(L["k"], snap["x_norm"]))
    assert close(raw_v[new_row], gemv(L["v"], snap["x_norm"]))
    untouched = np.ones(cache_rows * NKV * HD, bool)
    untouched[new_row] = False
    assert np.array_equal(snap["k_cache"][untouched], k_cache0[untouched]) and np.array_equal(snap["v_cache"][untouched], v_cache0[untouched])
    eq, ek, ev = tfo.k_fused_qkv_epilogue(raw_q, raw_k[new_row], raw_v[new_row], L["q_norm"], L["k_norm"], HD, NQ, NKV, position, THETA, PAIRS, EPS)
    assert close(snap["q"], eq) and close(snap["k_cache"][new_row], ek) and close(snap["v_cache"][new_row], ev)
    rows = seq_len * NKV * HD
    attn_ref = tfo.attention_ref(f(snap["q"]), f(snap["k_cache"][:rows]), f(snap["v_cache"][:rows]), HD, NQ, NKV, seq_len, WINDOW, ATTN_SCALE)
    assert tfo.rel_error(f(snap["attn"]), attn_ref) < TOL
    assert close(snap["o"], gemv(L["o"], snap["attn"]))
    want_hidden, want_dense, want_routed, want_router = tfo.k_post_attn_setup(hidden_before_setup, snap["o"], L["post_attn"], L["pre_ffn"], L["pre_ffn2"], EPS)
    for got, want in ((hidden_after_setup, want_hidden), (snap["dense_x"], want_dense), (snap["routed_x"], want_routed), (snap["router_x"], want_router)):
        assert close(got, want, tfo.Tolerance.fp16Reduction)
    shared_ref = tfo.shared_expert_ref(L["gate"], L["up"], L["down"], f(snap["dense_x"]), threads=8)
    assert tfo.rel_error(f(snap["shared"]), shared_ref) < 6e-3
    assert close(snap["h1"], tfo.k_rmsnorm_bf16w(snap["shared"], L["post_ffn1"], EPS))
    mo = L["moe"]
    logits = tfo.k_router_logits(mo["rW"], mo["rS"], mo["rB"], snap["router_x"], mo["eff_bits"])
    want_idx, want_wts = tfo.k_router_topk(logits, mo["gain_bits"])
    assert np.array_equal(idx, want_idx)
    assert np.max(np.abs(f(wts) - f(want_wts))) < 5e-3
    blobs = [mo["blobs"][int(e)] for e in idx]
    want_acts = tfo.k_moe_phase1(blobs, mo["off"], snap["routed_x"], D, F_MOE)
    assert close(snap["acts"], want_acts)
    assert close(snap["h2"], tfo.k_moe_phase2(blobs, mo["off"], snap["acts"], wts, np.zeros(D, np.uint16), D, F_MOE))
    assert close(hidden_out, tfo.k_layer_tail(snap["h2"], snap["h1"], hidden_after_setup, L["post_ffn2"], L["post_ffn"], EPS, LAYER_SCALAR),
                 tfo.Tolerance.fp16Reduction)

    # ---- the oracle's own chain from the start; comparable end to end when it picks the same experts
    x_norm = tfo.k_rmsnorm_bf16w(hidden0, L["input_norm"], EPS)
    oq, ok, ov = (gemv(L[n], x_norm) for n in ("q", "k", "v"))
    oq, ok, ov = tfo.k_fused_qkv_epilogue(oq, ok, ov, L["q_norm"], L["k_norm"], HD, NQ, NKV, position, THETA, PAIRS, EPS)
    kc, vc = k_cache0.copy(), v_cache0.copy()
    kc[new_row], vc[new_row] = ok, ov
    geo = tfo.attention_split_geometry(NQ, NKV, seq_len, 0, True)
    oattn = tfo.k_attention_split(oq, kc, vc, HD, NQ, NKV, seq_len, 0, geo["chunkLength"], geo["numChunks"], ATTN_SCALE)
    oo = gemv(L["o"], oattn)
    ohid, odense, orouted, orouter = tfo.k_post_attn_setup(hidden0, oo, L["post_attn"], L["pre_ffn"], L["pre_ffn2"], EPS)
    og = gemv(L["gate"], odense)
    ou = gemv(L["up"], odense)
    oshared = gemv(L["down"], tfo.k_gelu_mul_fp16(og, ou))
    oh1 = tfo.k_rmsnorm_bf16w(oshared, L["post_ffn1"], EPS)
    oidx, owts = tfo.k_router_topk(tfo.k_router_logits(mo["rW"], mo["rS"], mo["rB"], orouter, mo["eff_bits"]), mo["gain_bits"])
    if np.array_equal(oidx, idx):
        oblobs = [mo["blobs"][int(e)] for e in oidx]
        oacts = tfo.k_moe_phase1(oblobs, mo["off"], orouted, D, F_MOE)
        oh2 = tfo.k_moe_phase2(oblobs, mo["off"], oacts, owts, np.zeros(D, np.uint16), D, F_MOE)
        ofinal = tfo.k_layer_tail(oh2, oh1, ohid, L["post_ffn2"], L["post_ffn"], EPS, LAYER_SCALAR)
        assert tfo.rel_error(f(hidden_out), f(ofinal)) < 2 * TOL


@pytest.mark.parametrize("n,q_rows,kv_rows", [(D, NQ * HD, NKV * HD), (512, 96, 64), (4096, 130, 66)])
def test_norm_inside_the_qkv_launch_equals_norm_then_qkv(n, q_rows, kv_rows):
    # tf_fused_norm_qkv_gemv = tf_rmsnorm_bf16w + tf_fused_qkv_gemv: one launch at the production width (every block normalises
    # the row on its way into LDS), the two steps through the context's one-row buffer where the one-launch kernel does not apply
    # (rows of at most 1024 values); bit for bit in both cases
    rng = np.random.default_rng(n)
    mats = [refcases.synthetic_int4(r, n, 0x77 + i, "qkv"[i]) for i, r in enumerate((q_rows, kv_rows, kv_rows))]
    hidden = (rng.standard_normal(n) * 0.7).astype(np.float32).astype(np.float16).view(np.uint16)
    nw = tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(n).astype(np.float32))
    k = ctx()
    lib, h = k.lib, k.handle
    t = [[dev(a) for a in m] for m in mats]
    d_hidden, d_nw, x_norm = dev(hidden), dev(nw), zeros_bytes(n * 2)
    qkv = []
    for m in t:
        qkv += [m[0].data_ptr(), 0, m[1].data_ptr(), 0, m[2].data_ptr(), 0]
    outs = [[dev(np.full(r, 0x7BFF, np.uint16)) for r in (q_rows, kv_rows, kv_rows)] for _ in range(2)]
    k.check(lib.tf_rmsnorm_bf16w(h, None, d_hidden.data_ptr(), 0, d_nw.data_ptr(), 0, x_norm.data_ptr(), 0, n, EPS))
    k.check(lib.tf_fused_qkv_gemv(h, None, *qkv, x_norm.data_ptr(), outs[0][0].data_ptr(), 0, outs[0][1].data_ptr(), 0, outs[0][2].data_ptr(), 0,
                                  q_rows, kv_rows, n, tfk.TF_BF16))
    k.check(lib.tf_fused_norm_qkv_gemv(h, None, d_nw.data_ptr(), 0, EPS, *qkv, d_hidden.data_ptr(), outs[1][0].data_ptr(), 0,
                                       outs[1][1].data_ptr(), 0, outs[1][2].data_ptr(), 0, q_rows, kv_rows, n, tfk.TF_BF16))
    for a, b_, m in zip(outs[0], outs[1], mats):
        assert np.array_equal(host(a, np.uint16), host(b_, np.uint16))
        want = gemv(m, tfo.k_rmsnorm_bf16w(hidden, nw, EPS))
        assert tfo.rel_error(tfo.from_f16_bits(host(b_, np.uint16)), tfo.from_f16_bits(want)) < TOL
    assert lib.tf_fused_norm_qkv_gemv(h, None, None, 0, EPS, *qkv, d_hidden.data_ptr(), outs[1][0].data_ptr(), 0, outs[1][1].data_ptr(), 0,
                                      outs[1][2].data_ptr(), 0, q_rows, kv_rows, n, tfk.TF_BF16) == tfk.TF_ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("d", [D, 1000, 4096])
def test_shared_norm_inside_the_layer_tail_equals_norm_then_tail(d):
    # tf_fused_layer_tail_shared_norm = tf_rmsnorm_bf16w(shared, post_ffn1) + tf_fused_layer_tail: the squares of the shared
    # expert's output are summed in another order, so 1/rms may differ in its last bit and move an fp16 rounding that sits on
    # a tie: at most 0.5 % of the elements, each by one fp16 step of h1; and within the reference test's tolerance of the oracle
    rng = np.random.default_rng(d)
    bits = lambda a: a.astype(np.float32).astype(np.float16).view(np.uint16)
    h2, shared, hidden = bits(rng.standard_normal(d) * 0.3), bits(rng.standard_normal(d) * 2.0), bits(rng.standard_normal(d))
    w1, w2, w3 = (tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(d).astype(np.float32)) for _ in range(3))
    k = ctx()
    lib, h = k.lib, k.handle
    d_h2, d_sh, d_w1, d_w2, d_w3 = dev(h2), dev(shared), dev(w1), dev(w2), dev(w3)
    hid_a, hid_b, h1 = dev(hidden), dev(hidden), zeros_bytes(d * 2)
    k.check(lib.tf_rmsnorm_bf16w(h, None, d_sh.data_ptr(), 0, d_w1.data_ptr(), 0, h1.data_ptr(), 0, d, EPS))
    k.check(lib.tf_fused_layer_tail(h, None, d_h2.data_ptr(), h1.data_ptr(), hid_a.data_ptr(), d_w2.data_ptr(), 0, d_w3.data_ptr(), 0, d, EPS, LAYER_SCALAR))
    k.check(lib.tf_fused_layer_tail_shared_norm(h, None, d_h2.data_ptr(), d_sh.data_ptr(), hid_b.data_ptr(), d_w1.data_ptr(), 0, d_w2.data_ptr(), 0,
                                                d_w3.data_ptr(), 0, d, EPS, LAYER_SCALAR))
    a, b_ = tfo.from_f16_bits(host(hid_a, np.uint16)), tfo.from_f16_bits(host(hid_b, np.uint16))
    differ = a != b_
    assert differ.mean() <= 0.005
    assert np.max(np.abs(a - b_)) <= 2.0 ** -8 * max(1.0, float(np.max(np.abs(a))))
    want = tfo.k_layer_tail(h2, tfo.k_rmsnorm_bf16w(shared, w1, EPS), hidden, w2, w3, EPS, LAYER_SCALAR)
    assert tfo.rel_error(b_, tfo.from_f16_bits(want)) < tfo.Tolerance.fp16Reduction
    assert lib.tf_fused_layer_tail_shared_norm(h, None, d_h2.data_ptr(), d_sh.data_ptr(), hid_b.data_ptr(), None, 0, d_w2.data_ptr(), 0,
                                               d_w3.data_ptr(), 0, d, EPS, LAYER_SCALAR) == tfk.TF_ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("d,f,fs,misalign,sd", [(D, F_MOE, F_SHARED, 0, tfk.TF_BF16), (D, F_MOE, F_SHARED, 0, tfk.TF_FP16), (D, F_MOE, F_SHARED, 2, tfk.TF_BF16),
                                                (256, 128, 192, 0, tfk.TF_BF16), (2816, 704, 1088, 0, tfk.TF_BF16)])
def test_decode_step_with_the_shared_expert_riding_along_equals_the_two_calls(d, f, fs, misalign, sd):
    # tf_moe_decode_step_shared = tf_shared_expert_int4 + tf_moe_decode_step, every output of both bit for bit: at the production
    # widths the shared expert's rows are extra blocks of the step's first two launches; with a misaligned shared input, rows too
    # short for the row streamers or a width that takes another tile shape (1088 -> one-row tiles) it runs as its own launches
    # first.  With TF_FP16 the same bits are read as fp16 scales and biases: other numbers, the same equality.
    c = M._decode_step_case(d, f, E, 0x5AE + d + fs)
    shared = dict(gate=refcases.synthetic_int4(fs, d, 0x51, "sg"), up=refcases.synthetic_int4(fs, d, 0x52, "su"),
                  down=refcases.synthetic_int4(d, fs, 0x53, "sd"))
    dense_x = refcases.normal_f16(d, 0x54)
    k = ctx()
    lib, h = k.lib, k.handle
    t = M._decode_step_tensors(c)
    st = {n: [dev(a) for a in shared[n]] for n in shared}
    gate, up, down = (tfk.projection(*st[n], r, cc) for n, r, cc in (("gate", fs, d), ("up", fs, d), ("down", d, fs)))
    d_x = dev(np.concatenate([np.zeros(misalign // 2, np.uint16), dense_x]))
    x_ptr = d_x.data_ptr() + misalign
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    results = []
    for fused in (False, True):
        outs = M._fresh_outs(d, f)
        idx, wts, acts, y = outs
        sy, sg, su, sa = (dev(np.full(n, 0x7BFF, np.uint16)) for n in (d, fs, fs, fs))
        if fused:
            k.check(lib.tf_moe_decode_step_shared(h, None, t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0, t["x"].data_ptr(),
                                                  t["eff"].data_ptr(), 0, t["gain"].data_ptr(), 0, t["pool"].data_ptr(), c["stride"], E, off,
                                                  t["x"].data_ptr(), acts.data_ptr(), t["res"].data_ptr(), y.data_ptr(), idx.data_ptr(),
                                                  wts.data_ptr(), d, f, 8, sd, x_ptr, C.byref(gate), C.byref(up), C.byref(down),
                                                  sy.data_ptr(), sg.data_ptr(), su.data_ptr(), sa.data_ptr()))
        else:
            k.check(lib.tf_shared_expert_int4(h, None, x_ptr, 0, d * 2, C.byref(gate), C.byref(up), C.byref(down), sy.data_ptr(), 0, d * 2,
                                              sg.data_ptr(), 0, fs * 2, su.data_ptr(), 0, fs * 2, sa.data_ptr(), 0, fs * 2, 4, sd))
            assert M._decode_step_call(k, t, c, d, f, E, outs, sd) == tfk.TF_OK
        results.append(M._read_outs(outs, d, f) + tuple(host(b_, np.uint16) for b_ in (sy, sg, su, sa)))
    for a, b_ in zip(*results):
        assert np.array_equal(a, b_)
    # and the shared part is the shared expert the oracle computes
    if sd == tfk.TF_BF16:
        ref = tfo.shared_expert_ref(shared["gate"], shared["up"], shared["down"], tfo.from_f16_bits(dense_x), threads=8)
        assert tfo.rel_error(tfo.from_f16_bits(results[1][4]), ref) < 6e-3
    assert lib.tf_moe_decode_step_shared(h, None, t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0, t["x"].data_ptr(),
                                         t["eff"].data_ptr(), 0, t["gain"].data_ptr(), 0, t["pool"].data_ptr(), c["stride"], E, off,
                                         t["x"].data_ptr(), acts.data_ptr(), t["res"].data_ptr(), y.data_ptr(), idx.data_ptr(),
                                         wts.data_ptr(), d, f, 8, sd, x_ptr, C.byref(gate), C.byref(up), C.byref(up),
                                         sy.data_ptr(), sg.data_ptr(), su.data_ptr(), sa.data_ptr()) == tfk.TF_ERR_DIMENSION_MISMATCH


@pytest.mark.parametrize("d,f,fs,in_place,misalign,sd", [(D, F_MOE, F_SHARED, False, 0, tfk.TF_BF16), (D, F_MOE, F_SHARED, False, 0, tfk.TF_FP16),
                                                         (D, F_MOE, F_SHARED, True, 0, tfk.TF_BF16), (D, F_MOE, F_SHARED, False, 2, tfk.TF_BF16),
                                                         (256, 128, 192, False, 0, tfk.TF_BF16), (4096, 704, 2112, False, 0, tfk.TF_BF16)])
def test_post_attention_setup_inside_the_decode_step_equals_the_two_calls(d, f, fs, in_place, misalign, sd):
    # tf_moe_decode_step_shared_post_attn = tf_fused_post_attn_setup + tf_moe_decode_step_shared, every output bit for bit.  At the
    # production widths with separate buffers the setup runs in the prologue of every block of the first launch; written over its
    # own input, with a misaligned attention row or with rows too short for the shared launches it runs as a launch of its own.
    # With TF_FP16 the same bits are read as fp16 scales and biases: other numbers, the same equality.
    c = M._decode_step_case(d, f, E, 0x9A7 + d + fs)
    shared = dict(gate=refcases.synthetic_int4(fs, d, 0x61, "sg"), up=refcases.synthetic_int4(fs, d, 0x62, "su"),
                  down=refcases.synthetic_int4(d, fs, 0x63, "sd"))
    rng = np.random.default_rng(0x64 + d)
    weights = [tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(d).astype(np.float32)) for _ in range(3)]
    hidden_bits, attn_bits = refcases.normal_f16(d, 0x65), refcases.normal_f16(d, 0x66)
    k = ctx()
    lib, h = k.lib, k.handle
    t = M._decode_step_tensors(c)
    st = {n: [dev(a) for a in shared[n]] for n in shared}
    gate, up, down = (tfk.projection(*st[n], r, cc) for n, r, cc in (("gate", fs, d), ("up", fs, d), ("down", d, fs)))
    d_w = [dev(w) for w in weights]
    d_attn = dev(np.concatenate([np.zeros(misalign // 2, np.uint16), attn_bits]))
    attn_ptr = d_attn.data_ptr() + misalign
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    results = []
    for one_call in (False, True):
        outs = M._fresh_outs(d, f)
        idx, wts, acts, y = outs
        sy, sg, su, sa = (dev(np.full(n, 0x7BFF, np.uint16)) for n in (d, fs, fs, fs))
        hidden = dev(hidden_bits)
        hidden_out = hidden if in_place else dev(np.full(d, 0x7BFF, np.uint16))
        dense_x, routed_x, router_x = (dev(np.full(d, 0x7BFF, np.uint16)) for _ in range(3))
        step = (t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0, router_x.data_ptr(), t["eff"].data_ptr(), 0,
                t["gain"].data_ptr(), 0, t["pool"].data_ptr(), c["stride"], E, off, routed_x.data_ptr(), acts.data_ptr(), t["res"].data_ptr(),
                y.data_ptr(), idx.data_ptr(), wts.data_ptr(), d, f, 8, sd, dense_x.data_ptr(), C.byref(gate), C.byref(up), C.byref(down),
                sy.data_ptr(), sg.data_ptr(), su.data_ptr(), sa.data_ptr())
        if one_call:
            k.check(lib.tf_moe_decode_step_shared_post_attn(h, None, hidden.data_ptr(), attn_ptr, hidden_out.data_ptr(), d_w[0].data_ptr(), 0,
                                                            d_w[1].data_ptr(), 0, d_w[2].data_ptr(), 0, EPS, *step))
        else:
            if not in_place:
                hidden_out.copy_(hidden)
            k.check(lib.tf_fused_post_attn_setup(h, None, hidden_out.data_ptr(), attn_ptr, dense_x.data_ptr(), routed_x.data_ptr(), router_x.data_ptr(),
                                                 d_w[0].data_ptr(), 0, d_w[1].data_ptr(), 0, d_w[2].data_ptr(), 0, d, EPS))
            k.check(lib.tf_moe_decode_step_shared(h, None, *step))
        results.append(M._read_outs(outs, d, f) + tuple(host(b_, np.uint16) for b_ in (sy, sg, su, sa, hidden_out, dense_x, routed_x, router_x)))
        if not in_place:
            assert np.array_equal(host(hidden, np.uint16), hidden_bits)      # the input row is left alone
    for a, b_ in zip(*results):
        assert np.array_equal(a, b_)
    # the setup itself against the oracle's post-attention setup
    want = tfo.k_post_attn_setup(hidden_bits, attn_bits, weights[0], weights[1], weights[2], EPS)
    for got, ref in zip(results[1][8:12], want):
        assert np.max(np.abs(tfo.from_f16_bits(got) - tfo.from_f16_bits(ref))) <= 2e-3 * max(1.0, float(np.max(np.abs(tfo.from_f16_bits(ref)))))


@pytest.mark.parametrize("in_place,misalign", [(False, 0), (True, 0), (False, 2)])
def test_a_refused_decode_step_with_setup_and_shared_expert_launches_nothing(in_place, misalign):
    # A broken precondition of the ROUTED step (topK != 8, too many experts, a null pool, an odd activation pointer) is found before
    # the post-attention setup or the shared expert are enqueued, also where those run as launches of their own (in place, or a
    # misaligned attention row): every output keeps its sentinel and the residual row its input.
    d, f, fs = D, F_MOE, F_SHARED
    c = M._decode_step_case(d, f, E, 0xBAD + misalign)
    shared = dict(gate=refcases.synthetic_int4(fs, d, 0x71, "sg"), up=refcases.synthetic_int4(fs, d, 0x72, "su"),
                  down=refcases.synthetic_int4(d, fs, 0x73, "sd"))
    rng = np.random.default_rng(0x74)
    weights = [tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(d).astype(np.float32)) for _ in range(3)]
    hidden_bits, attn_bits = refcases.normal_f16(d, 0x75), refcases.normal_f16(d, 0x76)
    k = ctx()
    lib, h = k.lib, k.handle
    t = M._decode_step_tensors(c)
    st = {n: [dev(a) for a in shared[n]] for n in shared}
    gate, up, down = (tfk.projection(*st[n], r, cc) for n, r, cc in (("gate", fs, d), ("up", fs, d), ("down", d, fs)))
    d_w = [dev(w) for w in weights]
    d_attn = dev(np.concatenate([np.zeros(misalign // 2, np.uint16), attn_bits]))
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    sentinel = 0x7BFF
    outs = M._fresh_outs(d, f)
    idx, wts, acts, y = outs
    before = M._read_outs(outs, d, f)
    sy, sg, su, sa = (dev(np.full(n, sentinel, np.uint16)) for n in (d, fs, fs, fs))
    hidden = dev(hidden_bits)
    hidden_out = hidden if in_place else dev(np.full(d, sentinel, np.uint16))
    dense_x, routed_x, router_x = (dev(np.full(d, sentinel, np.uint16)) for _ in range(3))

    def call(top_k=8, experts=E, pool=None, routed_ptr=None):
        step = (t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0, router_x.data_ptr(), t["eff"].data_ptr(), 0,
                t["gain"].data_ptr(), 0, t["pool"].data_ptr() if pool is None else pool, c["stride"], experts, off,
                routed_x.data_ptr() if routed_ptr is None else routed_ptr, acts.data_ptr(), t["res"].data_ptr(),
                y.data_ptr(), idx.data_ptr(), wts.data_ptr(), d, f, top_k, tfk.TF_BF16, dense_x.data_ptr(), C.byref(gate), C.byref(up), C.byref(down),
                sy.data_ptr(), sg.data_ptr(), su.data_ptr(), sa.data_ptr())
        return lib.tf_moe_decode_step_shared_post_attn(h, None, hidden.data_ptr(), d_attn.data_ptr() + misalign, hidden_out.data_ptr(),
                                                       d_w[0].data_ptr(), 0, d_w[1].data_ptr(), 0, d_w[2].data_ptr(), 0, EPS, *step)

    for kwargs in (dict(top_k=4), dict(experts=257), dict(pool=0), dict(routed_ptr=routed_x.data_ptr() + 1)):
        assert call(**kwargs) == tfk.TF_ERR_INVALID_ARGUMENT, kwargs
        k.synchronize()
        assert np.array_equal(host(hidden, np.uint16), hidden_bits), kwargs
        for buf in (sy, sg, su, sa, dense_x, routed_x, router_x) + (() if in_place else (hidden_out,)):
            assert np.all(host(buf, np.uint16) == sentinel), kwargs
        for a, b_ in zip(M._read_outs(outs, d, f), before):
            assert np.array_equal(a, b_), kwargs
    assert call() == tfk.TF_OK      # and the same buffers are accepted when the arguments are right
    k.synchronize()


@pytest.mark.parametrize("n,q_rows,kv_rows,in_place,misalign,sd", [(D, NQ * HD, NKV * HD, False, 0, tfk.TF_BF16), (D, NQ * HD, NKV * HD, False, 0, tfk.TF_FP16),
                                                                  (D, NQ * HD, NKV * HD, True, 0, tfk.TF_BF16), (D, NQ * HD, NKV * HD, False, 2, tfk.TF_BF16),
                                                                  (512, 96, 64, False, 0, tfk.TF_BF16), (4096, 130, 66, False, 0, tfk.TF_BF16)])
def test_layer_tail_inside_the_next_qkv_launch_equals_the_two_calls(n, q_rows, kv_rows, in_place, misalign, sd):
    # tf_fused_layer_tail_norm_qkv_gemv = tf_fused_layer_tail_shared_norm + tf_fused_norm_qkv_gemv, every output bit for bit: with
    # separate buffers at the production width every block of the projection launch repeats the tail in its prologue; written
    # over its own input, with a misaligned h2 row or with rows the row streamer does not take, the tail is a launch of its own
    rng = np.random.default_rng(n + 7)
    bits = lambda a: a.astype(np.float32).astype(np.float16).view(np.uint16)
    mats = [refcases.synthetic_int4(r, n, 0x87 + i, "qkv"[i]) for i, r in enumerate((q_rows, kv_rows, kv_rows))]
    h2, shared, hidden = bits(rng.standard_normal(n) * 0.3), bits(rng.standard_normal(n) * 2.0), bits(rng.standard_normal(n))
    w1, w2, w3, nw = (tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(n).astype(np.float32)) for _ in range(4))
    k = ctx()
    lib, h = k.lib, k.handle
    t = [[dev(a) for a in m] for m in mats]
    d_sh, d_w1, d_w2, d_w3, d_nw = dev(shared), dev(w1), dev(w2), dev(w3), dev(nw)
    d_h2 = dev(np.concatenate([np.zeros(misalign // 2, np.uint16), h2]))
    h2_ptr = d_h2.data_ptr() + misalign
    qkv = []
    for m in t:
        qkv += [m[0].data_ptr(), 0, m[1].data_ptr(), 0, m[2].data_ptr(), 0]
    results = []
    for one_call in (False, True):
        outs = [dev(np.full(r, 0x7BFF, np.uint16)) for r in (q_rows, kv_rows, kv_rows)]
        hid = dev(hidden)
        hid_out = hid if in_place else dev(np.full(n, 0x7BFF, np.uint16))
        out_args = (outs[0].data_ptr(), 0, outs[1].data_ptr(), 0, outs[2].data_ptr(), 0, q_rows, kv_rows, n, sd)
        if one_call:
            k.check(lib.tf_fused_layer_tail_norm_qkv_gemv(h, None, h2_ptr, d_sh.data_ptr(), hid.data_ptr(), hid_out.data_ptr(), d_w1.data_ptr(), 0,
                                                          d_w2.data_ptr(), 0, d_w3.data_ptr(), 0, EPS, LAYER_SCALAR, d_nw.data_ptr(), 0, EPS, *qkv, *out_args))
        else:
            if not in_place:
                hid_out.copy_(hid)
            k.check(lib.tf_fused_layer_tail_shared_norm(h, None, h2_ptr, d_sh.data_ptr(), hid_out.data_ptr(), d_w1.data_ptr(), 0, d_w2.data_ptr(), 0,
                                                        d_w3.data_ptr(), 0, n, EPS, LAYER_SCALAR))
            k.check(lib.tf_fused_norm_qkv_gemv(h, None, d_nw.data_ptr(), 0, EPS, *qkv, hid_out.data_ptr(), *out_args))
        results.append([host(o, np.uint16) for o in outs] + [host(hid_out, np.uint16)])
        if not in_place:
            assert np.array_equal(host(hid, np.uint16), hidden)       # the input row is left alone
    for a, b_ in zip(*results):
        assert np.array_equal(a, b_)
    want_hidden = tfo.k_layer_tail(h2, tfo.k_rmsnorm_bf16w(shared, w1, EPS), hidden, w2, w3, EPS, LAYER_SCALAR)
    assert tfo.rel_error(tfo.from_f16_bits(results[1][3]), tfo.from_f16_bits(want_hidden)) < tfo.Tolerance.fp16Reduction
    for got, m in zip(results[1][:3], mats):
        if sd != tfk.TF_BF16:
            break        # the same bits read as fp16 scales: the equality above is the check
        want = gemv(m, tfo.k_rmsnorm_bf16w(results[1][3], nw, EPS))
        assert tfo.rel_error(tfo.from_f16_bits(got), tfo.from_f16_bits(want)) < TOL
    assert lib.tf_fused_layer_tail_norm_qkv_gemv(h, None, h2_ptr, d_sh.data_ptr(), hid.data_ptr(), None, d_w1.data_ptr(), 0, d_w2.data_ptr(), 0,
                                                 d_w3.data_ptr(), 0, EPS, LAYER_SCALAR, d_nw.data_ptr(), 0, EPS, *qkv, *out_args) == tfk.TF_ERR_INVALID_ARGUMENT


def test_folded_stages_replayed_from_a_graph():
    # the two launches that fold a stage into their prologue (post-attention setup + decode step with the shared expert, then the
    # layer tail + input norm + q/k/v of the next layer), captured into a HIP graph and replayed three times with eager calls of
    # the same entry points in between: every replay must leave what the eager sequence leaves
    import torch
    d, f, fs, q_rows, kv_rows = D, F_MOE, F_SHARED, NQ * HD, NKV * HD
    c = M._decode_step_case(d, f, E, 0x6A11)
    shared = dict(gate=refcases.synthetic_int4(fs, d, 0x71, "sg"), up=refcases.synthetic_int4(fs, d, 0x72, "su"),
                  down=refcases.synthetic_int4(d, fs, 0x73, "sd"))
    mats = [refcases.synthetic_int4(r, d, 0x97 + i, "qkv"[i]) for i, r in enumerate((q_rows, kv_rows, kv_rows))]
    rng = np.random.default_rng(0x74)
    norm = [dev(tfo.bf16_bits_array(1.0 + 0.1 * rng.standard_normal(d).astype(np.float32))) for _ in range(7)]
    hidden_bits, attn_bits = refcases.normal_f16(d, 0x75), refcases.normal_f16(d, 0x76)
    k = ctx()
    lib, h = k.lib, k.handle
    t = M._decode_step_tensors(c)
    st = {n: [dev(a) for a in shared[n]] for n in shared}
    gate, up, down = (tfk.projection(*st[n], r, cc) for n, r, cc in (("gate", fs, d), ("up", fs, d), ("down", d, fs)))
    tq = [[dev(a) for a in m] for m in mats]
    qkv = []
    for m in tq:
        qkv += [m[0].data_ptr(), 0, m[1].data_ptr(), 0, m[2].data_ptr(), 0]
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    d_attn, hidden = dev(attn_bits), dev(hidden_bits)
    names = ("mid", "next_hidden", "dense_x", "routed_x", "router_x", "y", "sy")
    sizes = dict(q=q_rows, kk=kv_rows, v=kv_rows, sg=fs, su=fs, sa=fs, acts=8 * f)

    def fresh():
        b = {n: dev(np.full(d, 0x7BFF, np.uint16)) for n in names}
        b.update({n: dev(np.full(s_, 0x7BFF, np.uint16)) for n, s_ in sizes.items()})
        b["idx"], b["wts"] = zeros_bytes(32), zeros_bytes(16)
        return b

    def run(b, stream):
        p = lambda n: b[n].data_ptr()
        k.check(lib.tf_moe_decode_step_shared_post_attn(h, stream, hidden.data_ptr(), d_attn.data_ptr(), p("mid"), norm[0].data_ptr(), 0, norm[1].data_ptr(), 0,
                                                        norm[2].data_ptr(), 0, EPS, t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0,
                                                        p("router_x"), t["eff"].data_ptr(), 0, t["gain"].data_ptr(), 0, t["pool"].data_ptr(), c["stride"], E, off,
                                                        p("routed_x"), p("acts"), t["res"].data_ptr(), p("y"), p("idx"), p("wts"), d, f, 8, tfk.TF_BF16,
                                                        p("dense_x"), C.byref(gate), C.byref(up), C.byref(down), p("sy"), p("sg"), p("su"), p("sa")))
        k.check(lib.tf_fused_layer_tail_norm_qkv_gemv(h, stream, p("y"), p("sy"), p("mid"), p("next_hidden"), norm[3].data_ptr(), 0, norm[4].data_ptr(), 0,
                                                      norm[5].data_ptr(), 0, EPS, LAYER_SCALAR, norm[6].data_ptr(), 0, EPS, *qkv, p("q"), 0, p("kk"), 0, p("v"), 0,
                                                      q_rows, kv_rows, d, tfk.TF_BF16))

    def read(b):
        return {n: host(b[n], np.uint16) for n in list(names) + ["q", "kk", "v", "sa", "acts"]}

    eager = fresh()
    run(eager, None)
    k.synchronize()
    want = read(eager)
    assert not np.all(want["q"] == 0x7BFF) and not np.all(want["next_hidden"] == 0x7BFF)
    side = torch.cuda.Stream()
    gb = fresh()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            run(gb, side.cuda_stream)
    for replay in range(3):
        for buf in gb.values():
            buf.fill_(0x55) if buf.dtype == torch.uint8 else buf.zero_()
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        got = read(gb)
        for n in want:
            assert np.array_equal(got[n], want[n]), (replay, n)
        again = fresh()                   # eager work between the replays
        run(again, None)
        k.synchronize()
        for n, v in read(again).items():
            assert np.array_equal(v, want[n]), (replay, n)

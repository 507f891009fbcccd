"""Wrapper scratch is sized at set-up (tf_ctx_create / tf_ctx_reserve), never inside an entry point: calls beyond the limits
are refused, calls within them can be recorded into a HIP graph on a context that has never run anything, and a larger
later call does not move the buffers under a graph recorded earlier."""
import numpy as np
import pytest

from gpu_helpers import dev, host, tfk, zeros_bytes
from oracle import tfo
from test_gpu_attention import draw as draw_attention

pytestmark = pytest.mark.gpu

DEFAULTS = dict(max_vocab=262144, max_block_tokens=2048, max_experts=256, max_shared_intermediate=2112, max_q_heads=16, max_head_dim=512,
                max_attention_block_tokens=128)


def limits_dict(lim):
    return {name: getattr(lim, name) for name, _ in lim._fields_}


def f16(a):
    return np.asarray(a, np.float32).astype(np.float16).view(np.uint16)


def short_head(vocab, d, seed):
    rng = np.random.default_rng(seed)
    W = rng.integers(0, 256, (vocab, d // 2), dtype=np.uint8)
    S = tfo.bf16_bits_array(rng.uniform(0.005, 0.02, vocab * (d // 64)).astype(np.float32)).reshape(vocab, d // 64)
    B = tfo.bf16_bits_array(rng.uniform(-0.1, 0.1, vocab * (d // 64)).astype(np.float32)).reshape(vocab, d // 64)
    hidden = f16(rng.standard_normal(d))
    norm = tfo.bf16_bits_array(rng.uniform(0.5, 1.5, d).astype(np.float32))
    return W, S, B, hidden, norm


def test_limits_start_at_the_model_shape_and_only_grow():
    k = tfk.Context(0)
    assert limits_dict(k.scratch_limits()) == DEFAULTS
    grown = limits_dict(k.reserve(max_vocab=300000, max_block_tokens=16))
    assert grown == dict(DEFAULTS, max_vocab=300000)
    assert limits_dict(k.reserve()) == grown
    k.close()


def test_calls_beyond_the_limits_are_refused_until_reserved():
    import torch
    k = tfk.Context(0)
    # greedy head on short rows (d <= 1024 goes through fp32 logits in wrapper scratch): one row more than the limit
    vocab, d = 262144 + 64, 64
    W, S, B, hidden, norm = short_head(vocab, d, 0x4E5)
    t = [dev(a) for a in (hidden, norm, W, S, B)]
    tok = zeros_bytes(4, 0xEE)
    rc = k.lm_head_greedy(*t, tok, d, vocab, raise_on_error=False)
    assert rc == tfk.TF_ERR_SCRATCH_TOO_SMALL and "tf_ctx_reserve" in k.last_error()
    assert host(tok, np.uint32, 1)[0] == 0xEEEEEEEE                      # nothing was enqueued
    # the truncating sampler keeps up to 256 candidates of every 1024-element tile in wrapper scratch
    probs = dev(f16(np.full(vocab, 1.0 / vocab)))
    rc = k.lib.tf_sample(k.handle, None, probs.data_ptr(), tok.data_ptr(), vocab, 1.0, 200, 0.9, 7, 0)
    assert rc == tfk.TF_ERR_SCRATCH_TOO_SMALL and "tf_ctx_reserve" in k.last_error()
    assert host(tok, np.uint32, 1)[0] == 0xEEEEEEEE
    k.reserve(max_vocab=vocab)
    k.check(k.lm_head_greedy(*t, tok, d, vocab, raise_on_error=False))
    torch.cuda.synchronize()
    assert int(host(tok, np.uint32, 1)[0]) == tfo.lm_head_cpu_greedy(hidden, norm, W, S, B, threads=8)
    k.close()


def test_fresh_context_records_every_scratch_user_into_a_graph():
    """Nothing has run on this context before the capture, and the sizes are the largest the limits allow for each buffer
    that used to grow on demand: block router logits, shared-expert block activations, sampler cells / pair buffers, the
    short-row head's logits, attention partial states.  Replays must reproduce the eager results bit for bit."""
    import ctypes as C
    import torch
    k = tfk.Context(0)
    side = torch.cuda.Stream()
    st = side.cuda_stream
    rng = np.random.default_rng(0x6EA9)
    keep = {}

    # block router: 2048 tokens x 128 experts x 256 (matrix-core path with split reduction planes)
    T, E, d = 2048, 128, 256
    keep["rW"] = dev(rng.integers(0, 256, (E, d), dtype=np.uint8))
    keep["rS"] = dev(tfo.bf16_bits_array(rng.uniform(0.0002, 0.0008, E * (d // 64)).astype(np.float32)))
    keep["rB"] = dev(tfo.bf16_bits_array(rng.uniform(-0.1, 0.0, E * (d // 64)).astype(np.float32)))
    keep["rH"] = dev(f16(rng.standard_normal(T * d)))
    keep["rEff"] = dev(tfo.bf16_bits_array((rng.uniform(0.5, 1.5, d) / np.sqrt(d)).astype(np.float32)))
    keep["rGain"] = dev(tfo.bf16_bits_array(rng.uniform(0.6, 1.4, E).astype(np.float32)))
    r_idx, r_w = zeros_bytes(T * 8 * 4), zeros_bytes(T * 8 * 2)

    def router():
        k.check(k.lib.tf_prefill_router_gemma4_block(k.handle, st, keep["rW"].data_ptr(), 0, keep["rS"].data_ptr(), 0, keep["rB"].data_ptr(), 0,
                                                     keep["rH"].data_ptr(), 0, keep["rEff"].data_ptr(), 0, keep["rGain"].data_ptr(), 0,
                                                     r_idx.data_ptr(), 0, r_w.data_ptr(), 0, T, E, d, 8, d))

    # shared expert block: 2048 rows, intermediate 2112 (the largest activations buffer the limits allow), d = 128
    rows, sd, sf = 2048, 128, 2112

    def int4(r, c):
        return (dev(rng.integers(0, 256, (r, c // 2), dtype=np.uint8)),
                dev(tfo.bf16_bits_array(rng.uniform(0.005, 0.02, r * (c // 64)).astype(np.float32))),
                dev(tfo.bf16_bits_array(rng.uniform(-0.1, 0.1, r * (c // 64)).astype(np.float32))))
    keep["g"], keep["u"], keep["dn"] = int4(sf, sd), int4(sf, sd), int4(sd, sf)
    keep["sx"] = dev(f16(rng.standard_normal(rows * sd)))
    s_y = zeros_bytes(rows * sd * 2)
    s_scr = [zeros_bytes(sf * 2) for _ in range(3)]
    pg, pu, pd = (tfk.projection(*keep[n], r, c) for n, r, c in (("g", sf, sd), ("u", sf, sd), ("dn", sd, sf)))

    def shared():
        k.check(k.lib.tf_prefill_shared_expert_int4_block(k.handle, st, keep["sx"].data_ptr(), 0, s_y.data_ptr(), 0, C.byref(pg), C.byref(pu), C.byref(pd),
                                                          s_scr[0].data_ptr(), 0, sf * 2, s_scr[1].data_ptr(), 0, sf * 2, s_scr[2].data_ptr(), 0, sf * 2,
                                                          rows, sd, sf, sd, sd, 4, tfk.TF_BF16))

    # samplers at the full vocabulary
    V = 262144
    logits16 = f16(rng.uniform(-20.0, 20.0, V))
    keep["lg"] = dev(logits16)
    probs, tok_k, tok_s = zeros_bytes(V * 2), zeros_bytes(4), zeros_bytes(4)

    def sample():
        k.check(k.lib.tf_logit_softcap_softmax(k.handle, st, keep["lg"].data_ptr(), probs.data_ptr(), V, 30.0, tfk.TF_FP16))
        k.check(k.lib.tf_sample_topk64(k.handle, st, probs.data_ptr(), tok_k.data_ptr(), V, 0.8, 0.95, 1234))
        k.check(k.lib.tf_sample(k.handle, st, probs.data_ptr(), tok_s.data_ptr(), V, 1.0, 0, 1.0, 99, 3))

    # short-row greedy head (fp32 logits in wrapper scratch)
    hv, hd = 200000, 64
    W, S, B, hidden, norm = short_head(hv, hd, 0x4E6)
    keep["head"] = [dev(a) for a in (hidden, norm, W, S, B)]
    tok_h = zeros_bytes(4)

    def head():
        hh, nn, ww, ss, bb = keep["head"]
        k.check(k.lib.tf_lm_head_greedy_int4(k.handle, st, hh.data_ptr(), 0, nn.data_ptr(), 0, ww.data_ptr(), 0, ss.data_ptr(), 0, bb.data_ptr(), 0,
                                             tok_h.data_ptr(), hd, hv, 1e-6, tfk.TF_BF16))

    # decode attention of a global layer at 8192 positions (512 chunks of partial states)
    hq, hkv, ad, seq = 16, 2, 512, 8192
    qb, kb, vb = draw_attention(0x7A1, "reserve-attn", hq, hkv, ad, seq)
    keep["aq"], keep["ak"], keep["av"] = dev(qb), dev(kb), dev(vb)
    a_out = zeros_bytes(hq * ad * 2)

    def attention():
        k.check(k.lib.tf_attention_full(k.handle, st, keep["aq"].data_ptr(), 0, keep["ak"].data_ptr(), 0, keep["av"].data_ptr(), 0, a_out.data_ptr(), 0,
                                        ad, hq, hkv, seq, 0.0))

    outputs = dict(r_idx=r_idx, r_w=r_w, s_y=s_y, probs=probs, tok_k=tok_k, tok_s=tok_s, tok_h=tok_h, a_out=a_out)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):       # the context's first calls ever
            for fn in (router, shared, sample, head, attention):
                fn()
    torch.cuda.synchronize()
    replays = []
    for _ in range(2):
        for t in outputs.values():
            t.fill_(0xEE)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        replays.append({n: host(t, np.uint8) for n, t in outputs.items()})
    with torch.cuda.stream(side):
        for t in outputs.values():
            t.fill_(0xEE)
        for fn in (router, shared, sample, head, attention):
            fn()
    torch.cuda.synchronize()
    eager = {n: host(t, np.uint8) for n, t in outputs.items()}
    for n in outputs:
        assert np.array_equal(replays[0][n], eager[n]) and np.array_equal(replays[1][n], eager[n]), n
    assert int(eager["tok_h"].view(np.uint32)[0]) == tfo.lm_head_cpu_greedy(hidden, norm, W, S, B, threads=8)
    ref = tfo.attention_ref(tfo.from_f16_bits(qb), tfo.from_f16_bits(kb), tfo.from_f16_bits(vb), ad, hq, hkv, seq, None, None)
    assert tfo.rel_error(tfo.from_f16_bits(eager["a_out"].view(np.uint16)), ref) < tfo.Tolerance.fp16ChainedReduction
    k.close()


def test_graph_of_a_short_context_survives_a_longer_eager_call():
    """A graph recorded at 256 positions keeps writing its partial states where it always did after an eager call at 32768
    positions has run on the same context (the scratch no longer moves when a larger call arrives)."""
    import torch
    k = tfk.Context(0)
    side = torch.cuda.Stream()
    hq, hkv, ad = 16, 2, 512
    qb, kb, vb = draw_attention(0x7A2, "reserve-attn-short", hq, hkv, ad, 256)
    q, kk, v = dev(qb), dev(kb), dev(vb)
    out = zeros_bytes(hq * ad * 2)
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(g, stream=side):
            k.check(k.lib.tf_attention_full(k.handle, side.cuda_stream, q.data_ptr(), 0, kk.data_ptr(), 0, v.data_ptr(), 0, out.data_ptr(), 0, ad, hq, hkv, 256, 0.0))
    g.replay()
    torch.cuda.synchronize()
    first = host(out, np.uint16)
    ref = tfo.attention_ref(tfo.from_f16_bits(qb), tfo.from_f16_bits(kb), tfo.from_f16_bits(vb), ad, hq, hkv, 256, None, None)
    assert tfo.rel_error(tfo.from_f16_bits(first), ref) < tfo.Tolerance.fp16ChainedReduction
    long_seq = 32768
    big_k = torch.randn((long_seq, hkv, ad), device="cuda").to(torch.float16)
    big_out = zeros_bytes(hq * ad * 2)
    k.check(k.lib.tf_attention_full(k.handle, None, q.data_ptr(), 0, big_k.data_ptr(), 0, big_k.data_ptr(), 0, big_out.data_ptr(), 0, ad, hq, hkv, long_seq, 0.0))
    torch.cuda.synchronize()
    out.fill_(0)
    g.replay()
    torch.cuda.synchronize()
    assert np.array_equal(host(out, np.uint16), first)
    k.close()

"""GPU parity, through the C ABI, of the norms, the rotation and the Q/K/V epilogue of a block of tokens, and of the
single-token norm variants they are compared with: a block must equal its tokens done one by one (bit for bit: the
reference suite's own check, PrefillPerHeadNormTests.swift, PrefillRoPETests.swift, PrefillQKVEpilogueTests.swift), the
oracle's kernel-order restatement and the exact references within the suite's tolerances; padding between token rows stays."""
import numpy as np
import pytest

from gpu_helpers import ctx, dev, host, tfk
from oracle import tfo
from test_gpu_rope import same_up_to_rounding
from test_oracle_prefill_qkv import EPS, block, closed_form

pytestmark = pytest.mark.gpu


def one_ulp(got_bits, want_bits):
    assert np.max(np.abs(got_bits.astype(np.int32) - want_bits.astype(np.int32))) <= 1


# PrefillPerHeadNormTests.swift:152-162 (q / k / v shapes of both layer kinds, stride = used + 23) plus an aligned stride
@pytest.mark.parametrize("tokens,heads,d", [(3, 16, 256), (3, 8, 256), (2, 16, 512), (2, 2, 512), (5, 3, 40)])
@pytest.mark.parametrize("pad", [23, 0, 8])
@pytest.mark.parametrize("weighted", [True, False])
def test_per_head_norm_block_equals_rows_one_by_one(tokens, heads, d, pad, weighted):
    x, w, stride = block(tokens, heads, d, pad, 0xB501 + d + heads + pad)
    k = ctx()
    d_w = dev(w)
    # in place, as the runner uses it
    blk = dev(x)
    if weighted:
        k.check(k.lib.tf_prefill_rmsnorm_bf16w_perhead_block(k.handle, None, blk.data_ptr(), 0, d_w.data_ptr(), 0, blk.data_ptr(), 0, tokens, d,
                                                             heads, stride, EPS))
    else:
        k.check(k.lib.tf_prefill_rmsnorm_no_scale_perhead_block(k.handle, None, blk.data_ptr(), 0, blk.data_ptr(), 0, tokens, d, heads, stride, EPS))
    rows = dev(x)
    for t in range(tokens):
        off = t * stride * 2
        if weighted:
            k.check(k.lib.tf_rmsnorm_bf16w_perhead(k.handle, None, rows.data_ptr(), off, d_w.data_ptr(), 0, rows.data_ptr(), off, d, heads, EPS))
        else:
            k.check(k.lib.tf_rmsnorm_no_scale_perhead(k.handle, None, rows.data_ptr(), off, rows.data_ptr(), off, d, heads, EPS))
    got, one_by_one = host(blk, np.uint16), host(rows, np.uint16)
    assert np.array_equal(got, one_by_one)
    one_ulp(got, tfo.k_rmsnorm_rows(x, w if weighted else None, EPS, tokens, heads, d, stride))
    used = tfo.from_f16_bits(got).reshape(tokens, stride)[:, :heads * d].reshape(tokens, heads, d)
    want = closed_form(x, w if weighted else None, tokens, heads, d, stride)
    assert tfo.rel_error(used.ravel(), want.ravel().astype(np.float32)) < tfo.Tolerance.fp16Reduction
    assert np.array_equal(got.reshape(tokens, stride)[:, heads * d:], x.reshape(tokens, stride)[:, heads * d:])


def test_single_row_variants_and_the_row_block():
    # rmsnorm_no_scale on one row, out of place with odd offsets; prefill_rmsnorm_bf16w_block over T contiguous rows = rows one by one
    k = ctx()
    d, T = 2816, 5
    x, w, _ = block(T, 1, d, 0, 0xB5A0)
    src, dst = dev(np.concatenate([np.zeros(1, np.uint16), x[:d]])), dev(np.zeros(d + 3, np.uint16))
    k.check(k.lib.tf_rmsnorm_no_scale(k.handle, None, src.data_ptr(), 2, dst.data_ptr(), 6, d, EPS))
    got = host(dst, np.uint16)
    assert np.all(got[:3] == 0)
    one_ulp(got[3:], tfo.k_rmsnorm_rows(x[:d], None, EPS, 1, 1, d, d))
    d_w, blk, rows = dev(w), dev(np.zeros(T * d, np.uint16)), dev(np.zeros(T * d, np.uint16))
    d_x = dev(x)
    k.check(k.lib.tf_prefill_rmsnorm_bf16w_block(k.handle, None, d_x.data_ptr(), 0, d_w.data_ptr(), 0, blk.data_ptr(), 0, T, d, EPS))   # PrefillPrimitiveTests.swift:85
    for t in range(T):
        k.check(k.lib.tf_rmsnorm_bf16w(k.handle, None, d_x.data_ptr(), t * d * 2, d_w.data_ptr(), 0, rows.data_ptr(), t * d * 2, d, EPS))
    assert np.array_equal(host(blk, np.uint16), host(rows, np.uint16))
    one_ulp(host(blk, np.uint16), tfo.k_rmsnorm_rows(x, w, EPS, T, 1, d, d))


# PrefillRoPETests.swift:37-150: 8 heads of 256 from position 1023 (default), 2 heads of 512 with 64 pairs from 4095 (proportional)
@pytest.mark.parametrize("tokens,heads,d,pairs,start,theta", [(3, 8, 256, None, 1023, 1e4), (2, 2, 512, 64, 4095, 1e6), (4, 3, 64, 10, 0, 1e4)])
@pytest.mark.parametrize("pad", [19, 0])
def test_rope_block_equals_rows_one_by_one_at_absolute_positions(tokens, heads, d, pairs, start, theta, pad):
    x, _, stride = block(tokens, heads, d, pad, 0xB700 + d + pad)
    k = ctx()
    blk, rows = dev(x), dev(x)
    rotated = d // 2 if pairs is None else pairs
    if pairs is None:
        k.check(k.lib.tf_prefill_rope_default_neox_block(k.handle, None, blk.data_ptr(), 0, start, tokens, d, heads, stride, theta))
    else:
        k.check(k.lib.tf_prefill_rope_proportional_neox_block(k.handle, None, blk.data_ptr(), 0, start, tokens, d, heads, pairs, stride, theta))
    want = x.copy()
    for t in range(tokens):
        off = t * stride
        if pairs is None:
            k.check(k.lib.tf_rope_default_neox(k.handle, None, rows.data_ptr(), off * 2, start + t, d, heads, 1, theta))
        else:
            k.check(k.lib.tf_rope_proportional_neox(k.handle, None, rows.data_ptr(), off * 2, start + t, d, heads, 1, pairs, theta))
        want[off:off + heads * d] = tfo.k_rope_neox(x[off:off + heads * d], 1, heads, d, rotated, start + t, theta)
    got = host(blk, np.uint16)
    assert np.array_equal(got, host(rows, np.uint16))
    same_up_to_rounding(got, want)
    for t in range(tokens):
        off = t * stride
        ref = tfo.rope_neox_ref(tfo.from_f16_bits(x[off:off + heads * d]), 1, heads, d, rotated, start + t, theta)
        assert tfo.rel_error(tfo.from_f16_bits(got[off:off + heads * d]), ref) < tfo.Tolerance.fp16Reduction
        assert np.array_equal(got[off + heads * d:off + stride], x[off + heads * d:off + stride])


# PrefillQKVEpilogueTests.swift:8-32: a sliding-window layer and a full layer whose k and v start from the same raw rows
@pytest.mark.parametrize("tokens,hq,hkv,d,start,theta,pairs,shared_raw", [(3, 16, 8, 256, 1023, 1e4, 128, False), (2, 16, 2, 512, 4095, 1e6, 64, True),
                                                                          (4, 2, 1, 64, 5, 1e4, 7, False)])
def test_qkv_epilogue_block_equals_tokens_one_by_one(tokens, hq, hkv, d, start, theta, pairs, shared_raw):
    q, qw, q_stride = block(tokens, hq, d, 13, 0x7A50 + d)
    kk, kw, kv_stride = block(tokens, hkv, d, 17, 0x7A51 + d)
    vv = kk.copy() if shared_raw else block(tokens, hkv, d, 17, 0x7A52 + d)[0]
    k = ctx()
    d_qw, d_kw = dev(qw), dev(kw)
    bq, bk, bv = dev(q), dev(kk), dev(vv)
    k.check(k.lib.tf_prefill_qkv_epilogue_block(k.handle, None, bq.data_ptr(), 0, bk.data_ptr(), 0, bv.data_ptr(), 0, d_qw.data_ptr(), 0,
                                                d_kw.data_ptr(), 0, start, tokens, d, hq, hkv, q_stride, kv_stride, theta, pairs, EPS))
    rq, rk, rv = dev(q), dev(kk), dev(vv)
    wq, wk, wv = q.copy(), kk.copy(), vv.copy()
    for t in range(tokens):
        qo, ko = t * q_stride, t * kv_stride
        k.check(k.lib.tf_fused_qkv_epilogue(k.handle, None, rq.data_ptr(), qo * 2, rk.data_ptr(), ko * 2, rv.data_ptr(), ko * 2, d_qw.data_ptr(), 0,
                                            d_kw.data_ptr(), 0, d, hq, hkv, start + t, theta, pairs, EPS))
        wq[qo:qo + hq * d], wk[ko:ko + hkv * d], wv[ko:ko + hkv * d] = tfo.k_fused_qkv_epilogue(
            q[qo:qo + hq * d], kk[ko:ko + hkv * d], vv[ko:ko + hkv * d], qw, kw, d, hq, hkv, start + t, theta, pairs, EPS)
    for got, one_by_one, want in ((bq, rq, wq), (bk, rk, wk), (bv, rv, wv)):
        g = host(got, np.uint16)
        assert np.array_equal(g, host(one_by_one, np.uint16))
        same_up_to_rounding(g, want)
    if shared_raw:
        assert not np.array_equal(host(bk, np.uint16), host(bv, np.uint16))        # k and v diverge: norm weight + rotation against no scale
    # the five separate calls of the reference's wrapper give the same block
    sq, sk, sv = dev(q), dev(kk), dev(vv)
    lib, h = k.lib, k.handle
    k.check(lib.tf_prefill_rmsnorm_bf16w_perhead_block(h, None, sq.data_ptr(), 0, d_qw.data_ptr(), 0, sq.data_ptr(), 0, tokens, d, hq, q_stride, EPS))
    k.check(lib.tf_prefill_rmsnorm_bf16w_perhead_block(h, None, sk.data_ptr(), 0, d_kw.data_ptr(), 0, sk.data_ptr(), 0, tokens, d, hkv, kv_stride, EPS))
    k.check(lib.tf_prefill_rmsnorm_no_scale_perhead_block(h, None, sv.data_ptr(), 0, sv.data_ptr(), 0, tokens, d, hkv, kv_stride, EPS))
    k.check(lib.tf_prefill_rope_proportional_neox_block(h, None, sq.data_ptr(), 0, start, tokens, d, hq, pairs, q_stride, theta))
    k.check(lib.tf_prefill_rope_proportional_neox_block(h, None, sk.data_ptr(), 0, start, tokens, d, hkv, pairs, kv_stride, theta))
    for fused, separate in ((bq, sq), (bk, sk), (bv, sv)):
        same_up_to_rounding(host(fused, np.uint16), host(separate, np.uint16), ulps=1, share=0.01)


def test_contracts():
    k = ctx()
    lib, h = k.lib, k.handle
    buf, w = dev(np.zeros(4096, np.uint16)), dev(np.zeros(512, np.uint16))
    p = buf.data_ptr()
    bad = tfk.TF_ERR_INVALID_ARGUMENT
    assert lib.tf_prefill_rmsnorm_bf16w_perhead_block(h, None, p, 0, w.data_ptr(), 0, p, 0, 0, 64, 2, 128, EPS) == bad        # queryCount must be positive
    assert lib.tf_prefill_rmsnorm_bf16w_perhead_block(h, None, p, 0, w.data_ptr(), 0, p, 0, 2, 64, 2, 127, EPS) == bad        # token stride is too small
    assert lib.tf_prefill_rmsnorm_no_scale_perhead_block(h, None, p, 0, p, 0, 2, 0, 2, 128, EPS) == bad                       # headDim must be positive
    assert lib.tf_prefill_rmsnorm_no_scale_perhead_block(h, None, p, 0, p, 0, 2, 64, 0, 128, EPS) == bad                      # numHeads must be positive
    assert lib.tf_rmsnorm_bf16w_perhead(h, None, p, 1, w.data_ptr(), 0, p, 0, 64, 2, EPS) == bad                              # odd byte offset
    assert lib.tf_prefill_rope_default_neox_block(h, None, p, 0, 0, 0, 64, 2, 128, 1e4) == bad                                # queryCount
    assert lib.tf_prefill_rope_default_neox_block(h, None, p, 0, 0, 2, 63, 2, 128, 1e4) == bad                                # headDim must be even
    assert lib.tf_prefill_rope_proportional_neox_block(h, None, p, 0, 0, 2, 64, 2, 33, 128, 1e4) == bad                       # rotatedPairs * 2 > headDim
    assert lib.tf_prefill_rope_proportional_neox_block(h, None, p, 0, 0, 2, 64, 2, 8, 127, 1e4) == bad                        # token stride
    args = (p, 0, p, 0, p, 0, w.data_ptr(), 0, w.data_ptr(), 0)
    assert lib.tf_prefill_qkv_epilogue_block(h, None, *args, 0, 0, 64, 2, 1, 128, 64, 1e4, 8, EPS) == bad                     # queryCount
    assert lib.tf_prefill_qkv_epilogue_block(h, None, *args, 0, 2, 64, 2, 1, 128, 64, 1e4, 0, EPS) == bad                     # rotatedPairs must be positive
    assert lib.tf_prefill_qkv_epilogue_block(h, None, *args, 0, 2, 64, 2, 1, 127, 64, 1e4, 8, EPS) == bad                     # Q token stride
    assert lib.tf_prefill_qkv_epilogue_block(h, None, *args, 0, 2, 64, 2, 1, 128, 63, 1e4, 8, EPS) == bad                     # KV token stride
    assert lib.tf_prefill_qkv_epilogue_block(h, None, *args, 0, 2, 64, 0, 1, 128, 64, 1e4, 8, EPS) == bad                     # numQHeads
    assert lib.tf_prefill_qkv_epilogue_block(h, None, *args, 0, 2, 1024, 1, 1, 1024, 1024, 1e4, 8, EPS) == bad                # head_dim beyond the scratch

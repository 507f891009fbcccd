"""Pins the attention part of the oracle: AttentionRef's restatement against torch's float64 attention and against what
the mathematics fixes, the split geometry against the reference test's literal numbers, and the kernel-order split-KV
restatement against the full-matrix reference on the reference suite's shapes (AttentionTests.swift).  CPU only."""
import numpy as np
import pytest
import torch

from oracle import tfo


def draw(seed, label, hq, hkv, d, t):
    """AttentionTests.swift:121-136: q, k, v ~ U(-0.5, 0.5) from one keyed stream, rounded to fp16."""
    rng = tfo.SeedTree(seed).key(label)
    q = rng.uniform_array(-0.5, 0.5, hq * d)
    k = rng.uniform_array(-0.5, 0.5, t * hkv * d)
    v = rng.uniform_array(-0.5, 0.5, t * hkv * d)
    return [tfo.to_f16_bits(a) for a in (q, k, v)]


def torch_attention(q, k, v, d, hq, hkv, t, window, scale):
    qt = torch.from_numpy(q.astype(np.float64)).reshape(hq, 1, d)
    kt = torch.from_numpy(k.astype(np.float64)).reshape(t, hkv, d)
    vt = torch.from_numpy(v.astype(np.float64)).reshape(t, hkv, d)
    start = t - window if (window is not None and t > window) else 0
    kt, vt = kt[start:], vt[start:]
    group = hq // hkv
    kt = kt.permute(1, 0, 2).repeat_interleave(group, dim=0)       # [hq, T', d]
    vt = vt.permute(1, 0, 2).repeat_interleave(group, dim=0)
    s = (qt @ kt.transpose(1, 2)) * (scale if scale is not None else 1.0 / np.sqrt(d))
    p = torch.softmax(s, dim=-1)
    return (p @ vt).reshape(-1).numpy()


@pytest.mark.parametrize("hq,hkv,d,t,window,scale", [(4, 2, 64, 128, 64, None), (4, 2, 64, 32, 128, None), (16, 8, 256, 256, 128, None),
                                                     (8, 1, 64, 128, None, None), (16, 2, 512, 128, None, None), (4, 2, 64, 8, 8, 1.0),
                                                     (6, 3, 40, 17, 5, 0.37)])
def test_attention_ref_equals_torch_float64(hq, hkv, d, t, window, scale):
    q, k, v = [tfo.from_f16_bits(b) for b in draw(0x171, f"attn-{hq}-{hkv}-{d}-{t}", hq, hkv, d, t)]
    got = tfo.attention_ref(q, k, v, d, hq, hkv, t, window, scale)
    want = torch_attention(q, k, v, d, hq, hkv, t, window, scale)
    assert np.max(np.abs(got - want)) < 2e-6


def test_attention_ref_closed_forms():
    hq, hkv, d, t = 4, 2, 16, 12
    rng = np.random.default_rng(1)
    q = rng.standard_normal(hq * d).astype(np.float32)
    v = rng.standard_normal((t, hkv, d)).astype(np.float32)
    # identical keys: uniform probabilities -> the mean of V over the window, per kv head
    k = np.tile(rng.standard_normal((1, hkv, d)).astype(np.float32), (t, 1, 1))
    for window in (None, 5):
        got = tfo.attention_ref(q, k, v, d, hq, hkv, t, window).reshape(hq, d)
        rows = v if window is None else v[t - window:]
        for h in range(hq):
            assert np.allclose(got[h], rows[:, h // 2].mean(axis=0), atol=1e-6)
    # one key aligned with q and scaled up: its V row comes out
    k2 = rng.standard_normal((t, hkv, d)).astype(np.float32) * 0.01
    k2[7, 0] = q[:d] * 50.0
    got = tfo.attention_ref(q, k2, v, d, hq, hkv, t).reshape(hq, d)
    assert np.allclose(got[0], v[7, 0], atol=1e-5)
    # scale enters the scores, not the values: scale -> tiny gives the mean again
    got = tfo.attention_ref(q, k2, v, d, hq, hkv, t, None, 1e-12).reshape(hq, d)
    assert np.allclose(got[3], v[:, 1].mean(axis=0), atol=1e-5)
    # a window of one returns the last row
    got = tfo.attention_ref(q, k2, v, d, hq, hkv, t, 1).reshape(hq, d)
    assert np.allclose(got[2], v[-1, 1], atol=1e-6)


def test_split_geometry_literals_of_the_reference_test():
    # AttentionTests.swift:25-47
    swa = tfo.attention_split_geometry(16, 8, 1536, 512, True)
    assert swa == dict(effectiveLength=1024, numChunks=16, chunkLength=64, partialThreadgroups=128, useSWAGroupedPartial=True)
    full = tfo.attention_split_geometry(16, 2, 1536, 0, False)
    assert full == dict(effectiveLength=1536, numChunks=16, chunkLength=96, partialThreadgroups=256, useSWAGroupedPartial=False)
    # short ranges: never more chunks than positions (Attention.swift:124-128), an empty range still makes one chunk
    assert tfo.attention_split_geometry(16, 2, 5, 0, False)["numChunks"] == 5
    assert tfo.attention_split_geometry(16, 2, 0, 0, False)["numChunks"] == 1
    assert tfo.attention_split_geometry(16, 8, 0, 0, True)["numChunks"] == 2      # grouped: base chunks x query heads per kv head (:138-140)
    # grouped partial only for at most two query heads per kv head (:136)
    assert not tfo.attention_split_geometry(16, 2, 64, 0, True)["useSWAGroupedPartial"]


@pytest.mark.parametrize("hq,hkv,d,t,window,seed", [(4, 2, 64, 128, 64, 0x171), (4, 2, 64, 32, 128, 0x172), (16, 8, 256, 256, 128, 0x173),
                                                    (8, 1, 64, 128, None, 0x174), (16, 2, 512, 128, None, 0x175)])
def test_kernel_order_split_matches_the_full_matrix_reference(hq, hkv, d, t, window, seed):
    # AttentionTests.swift:204-232, 363-391: rel error below fp16ChainedReduction
    qb, kb, vb = draw(seed, f"attn-h{hq}-kv{hkv}-d{d}-T{t}-kv=false", hq, hkv, d, t)
    kv_start = t - window if (window is not None and t > window) else 0
    geo = tfo.attention_split_geometry(hq, hkv, t, kv_start, window is not None)
    scale = 1.0 / np.sqrt(np.float32(d))
    got = tfo.k_attention_split(qb, kb, vb, d, hq, hkv, t, kv_start, geo["chunkLength"], geo["numChunks"], scale)
    ref = tfo.attention_ref(tfo.from_f16_bits(qb), tfo.from_f16_bits(kb), tfo.from_f16_bits(vb), d, hq, hkv, t, window)
    assert tfo.rel_error(tfo.from_f16_bits(got), ref) < tfo.Tolerance.fp16ChainedReduction
    # one chunk == many chunks up to fp32 rounding of the partial sums
    one = tfo.k_attention_split(qb, kb, vb, d, hq, hkv, t, kv_start, max(1, t - kv_start), 1, scale)
    assert np.max(np.abs(tfo.from_f16_bits(one) - tfo.from_f16_bits(got))) <= 2e-3


def test_ring_rows_equal_linear_rows():
    # AttentionTests.swift:219-285: window 16, ring of 24 rows, position p in row p % 24
    hq, hkv, d, t, window, ring = 4, 2, 64, 40, 16, 24
    qb, kb, vb = draw(0x174, "attn-swa-ring", hq, hkv, d, t)
    stride = hkv * d
    k_ring, v_ring = np.zeros(ring * stride, np.uint16), np.zeros(ring * stride, np.uint16)
    for p in range(t):
        k_ring[(p % ring) * stride:(p % ring + 1) * stride] = kb[p * stride:(p + 1) * stride]
        v_ring[(p % ring) * stride:(p % ring + 1) * stride] = vb[p * stride:(p + 1) * stride]
    scale = 1.0 / np.sqrt(np.float32(d))
    linear = tfo.k_attention_split(qb, kb, vb, d, hq, hkv, t, t - window, 2, 8, scale)
    wrapped = tfo.k_attention_split(qb, k_ring, v_ring, d, hq, hkv, t, t - window, 2, 8, scale, ring_capacity=ring)
    assert np.array_equal(linear, wrapped)

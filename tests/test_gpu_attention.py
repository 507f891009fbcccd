"""GPU parity of decode attention through the C ABI against the oracle: the reference suite's shapes and tolerances
(AttentionTests.swift), ring addressing, the generic path, long ranges and the contract."""
import numpy as np
import pytest

from gpu_helpers import ctx, dev, host, tfk, zeros_bytes
from oracle import tfo
from test_oracle_attention import draw

pytestmark = pytest.mark.gpu
TOL = tfo.Tolerance.fp16ChainedReduction


def run(qb, kb, vb, d, hq, hkv, t, window=None, scale=0.0, ring=0, share_kv=False, offsets=(0, 0, 0, 0), raise_on_error=False):
    k = ctx()
    pad = lambda bits, off: np.concatenate([np.zeros(off // 2, np.uint16), bits])
    keep = dict(q=dev(pad(qb, offsets[0])), k=dev(pad(kb, offsets[1])))
    keep["v"] = keep["k"] if share_kv else dev(pad(vb, offsets[2]))
    keep["out"] = zeros_bytes(hq * d * 2 + offsets[3], 0xEE)
    if window is None:
        rc = k.attention_full(keep["q"], keep["k"], keep["v"], keep["out"], d, hq, hkv, t, scale, offsets=offsets, raise_on_error=raise_on_error)
    else:
        rc = k.attention_swa(keep["q"], keep["k"], keep["v"], keep["out"], d, hq, hkv, t, window, scale, ring, offsets=offsets,
                             raise_on_error=raise_on_error)
    return rc, host(keep["out"], np.uint16)[offsets[3] // 2:]


def reference(qb, kb, vb, d, hq, hkv, t, window=None, scale=None):
    return tfo.attention_ref(tfo.from_f16_bits(qb), tfo.from_f16_bits(kb), tfo.from_f16_bits(vb), d, hq, hkv, t, window, scale)


@pytest.mark.parametrize("hq,hkv,d,t,window,seed,share", [
    (4, 2, 64, 128, 64, 0x171, False),        # attentionSWA_smallShape
    (4, 2, 64, 32, 128, 0x172, False),        # attentionSWA_shorterThanWindow
    (16, 8, 256, 256, 128, 0x173, False),     # attentionSWA_realShape
    (8, 1, 64, 128, None, 0x174, False),      # attentionFull_smallShape
    (16, 2, 512, 128, None, 0x175, False),    # attentionFull_realShape
    (8, 1, 64, 128, None, 0x176, True),       # attentionFull_kvShared_smallShape
    (16, 2, 512, 128, None, 0x177, True),     # attentionFull_kvShared_realShape
    (16, 4, 128, 77, None, 0x178, False),     # four query heads per kv head, a ragged length
    (2, 2, 128, 300, 200, 0x179, False),      # no grouping
])
def test_reference_suite_shapes(hq, hkv, d, t, window, seed, share):
    qb, kb, vb = draw(seed, f"attn-h{hq}-kv{hkv}-d{d}-T{t}-kv={str(share).lower()}", hq, hkv, d, t)
    if share:
        vb = kb
    rc, out = run(qb, kb, vb, d, hq, hkv, t, window, share_kv=share)
    assert rc == tfk.TF_OK
    assert tfo.rel_error(tfo.from_f16_bits(out), reference(qb, kb, vb, d, hq, hkv, t, window)) < TOL
    # and close to the kernel-order restatement with the reference's own split
    kv_start = t - window if (window is not None and t > window) else 0
    geo = tfo.attention_split_geometry(hq, hkv, t, kv_start, window is not None)
    split = tfo.k_attention_split(qb, kb, vb, d, hq, hkv, t, kv_start, geo["chunkLength"], geo["numChunks"], 1.0 / np.sqrt(np.float32(d)))
    assert np.max(np.abs(tfo.from_f16_bits(out) - tfo.from_f16_bits(split))) <= 2e-3


def test_unit_scale_is_honoured():
    # attentionSWA_unitScale_matchesReference_andDiffersFromDefault (AttentionTests.swift:55-109)
    hq, hkv, d, t = 4, 2, 64, 8
    qb, kb, vb = draw(0x501, "attn-scale1-swa", hq, hkv, d, t)
    rc, unit = run(qb, kb, vb, d, hq, hkv, t, window=8, scale=1.0)
    assert rc == tfk.TF_OK
    assert tfo.rel_error(tfo.from_f16_bits(unit), reference(qb, kb, vb, d, hq, hkv, t, 8, 1.0)) < TOL
    rc, default = run(qb, kb, vb, d, hq, hkv, t, window=8)
    assert rc == tfk.TF_OK and not np.array_equal(unit, default)


def ring_copy(bits, t, ring, stride):
    out = np.zeros(ring * stride, np.uint16)
    for p in range(t):
        out[(p % ring) * stride:(p % ring + 1) * stride] = bits[p * stride:(p + 1) * stride]
    return out


@pytest.mark.parametrize("hq,hkv,d,t,window,ring", [(4, 2, 64, 40, 16, 24),          # attentionSWA_ringCapacityMatchesLinearReference
                                                    (16, 8, 256, 1400, 1024, 1152)])  # ...MatchesLinearKernelAtWrapRealShape
def test_ring_rows_match_linear_rows(hq, hkv, d, t, window, ring):
    qb, kb, vb = draw(0x181, "attn-swa-ring", hq, hkv, d, t)
    rc, linear = run(qb, kb, vb, d, hq, hkv, t, window)
    assert rc == tfk.TF_OK
    rc, wrapped = run(qb, ring_copy(kb, t, ring, hkv * d), ring_copy(vb, t, ring, hkv * d), d, hq, hkv, t, window, ring=ring)
    assert rc == tfk.TF_OK
    assert np.array_equal(linear, wrapped)          # the same rows in the same order: bit-identical
    assert tfo.rel_error(tfo.from_f16_bits(wrapped), reference(qb, kb, vb, d, hq, hkv, t, window)) < TOL


@pytest.mark.parametrize("hq,hkv,d,t,window,offsets", [(6, 2, 40, 50, None, (0, 0, 0, 0)),      # head_dim and group size off the fast path
                                                      (4, 2, 64, 90, 33, (2, 6, 10, 2)),       # 2-byte aligned operands
                                                      (12, 4, 96, 130, 128, (0, 0, 0, 0)),
                                                      (5, 5, 512, 20, None, (0, 0, 0, 0))])
def test_generic_path(hq, hkv, d, t, window, offsets):
    qb, kb, vb = draw(0x190, f"attn-generic-{hq}-{d}-{t}", hq, hkv, d, t)
    rc, out = run(qb, kb, vb, d, hq, hkv, t, window, offsets=offsets)
    assert rc == tfk.TF_OK
    assert tfo.rel_error(tfo.from_f16_bits(out), reference(qb, kb, vb, d, hq, hkv, t, window)) < TOL


def test_long_ranges_at_production_shapes():
    # full attention of a global layer (16 query heads on 2 kv heads, head_dim 512) and a sliding window of 1024 rows
    for hq, hkv, d, t, window in ((16, 2, 512, 8192, None), (16, 8, 256, 5000, 1024)):
        rng = np.random.default_rng(t)
        qb = rng.uniform(-0.5, 0.5, hq * d).astype(np.float32).astype(np.float16).view(np.uint16)
        kb = rng.uniform(-0.5, 0.5, t * hkv * d).astype(np.float32).astype(np.float16).view(np.uint16)
        vb = rng.uniform(-0.5, 0.5, t * hkv * d).astype(np.float32).astype(np.float16).view(np.uint16)
        rc, out = run(qb, kb, vb, d, hq, hkv, t, window)
        assert rc == tfk.TF_OK
        assert tfo.rel_error(tfo.from_f16_bits(out), reference(qb, kb, vb, d, hq, hkv, t, window)) < TOL
        # identical keys: every position weighs the same, whatever the length -> the mean of the window's V rows
        kb_same = np.tile(kb[:hkv * d], t)
        rc, out = run(qb, kb_same, vb, d, hq, hkv, t, window)
        rows = tfo.from_f16_bits(vb).reshape(t, hkv, d)[(t - window if window else 0):]
        want = np.stack([rows[:, h // (hq // hkv)].astype(np.float64).mean(axis=0) for h in range(hq)]).reshape(-1)
        assert np.max(np.abs(tfo.from_f16_bits(out) - want)) < 2e-3


def test_edges_and_contract():
    hq, hkv, d = 4, 2, 64
    qb, kb, vb = draw(0x1A0, "attn-edges", hq, hkv, d, 8)
    # one position: the output is that V row
    rc, out = run(qb, kb, vb, d, hq, hkv, 1)
    assert rc == tfk.TF_OK
    v0 = vb[:hkv * d].reshape(hkv, d)
    assert np.array_equal(out.reshape(hq, d), np.stack([v0[h // 2] for h in range(hq)]))
    # an empty sliding-window range writes zeros; full attention refuses it (Attention.swift:196)
    rc, out = run(qb, kb, vb, d, hq, hkv, 0, window=4)
    assert rc == tfk.TF_OK and not out.any()
    assert run(qb, kb, vb, d, hq, hkv, 0)[0] == tfk.TF_ERR_INVALID_ARGUMENT
    assert run(qb, kb, vb, d, 3, 2, 8)[0] == tfk.TF_ERR_INVALID_ARGUMENT                       # :166-167
    assert run(qb, kb, vb, 514, hq, hkv, 8)[0] == tfk.TF_ERR_INVALID_ARGUMENT                  # :168-169
    assert run(np.zeros(32 * d, np.uint16), kb, vb, d, 32, 2, 8)[0] == tfk.TF_ERR_INVALID_ARGUMENT   # :229-230
    assert run(qb, kb, vb, d, hq, hkv, 8, window=8, ring=4)[0] == tfk.TF_ERR_INVALID_ARGUMENT  # the window must fit the ring
    # the reference's own split geometry (AttentionTests.swift:25-47)
    import ctypes as C
    geo = tfk.AttentionSplitGeometry()
    ctx().lib.tf_attention_split_geometry(16, 8, 1536, 512, 1, C.byref(geo))
    assert (geo.effective_length, geo.num_chunks, geo.chunk_length, geo.partial_threadgroups, geo.use_swa_grouped_partial) == (1024, 16, 64, 128, 1)
    ctx().lib.tf_attention_split_geometry(16, 2, 1536, 0, 0, C.byref(geo))
    assert (geo.effective_length, geo.num_chunks, geo.chunk_length, geo.partial_threadgroups, geo.use_swa_grouped_partial) == (1536, 16, 96, 256, 0)
    for args in ((16, 8, 0, 0, True), (16, 2, 5, 0, False), (8, 1, 4000, 100, False), (16, 8, 77, 13, True)):
        ctx().lib.tf_attention_split_geometry(args[0], args[1], args[2], args[3], int(args[4]), C.byref(geo))
        want = tfo.attention_split_geometry(*args)
        assert (geo.effective_length, geo.num_chunks, geo.chunk_length, geo.partial_threadgroups, bool(geo.use_swa_grouped_partial)) == \
            (want["effectiveLength"], want["numChunks"], want["chunkLength"], want["partialThreadgroups"], want["useSWAGroupedPartial"])

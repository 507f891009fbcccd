"""GPU parity of the block (prefill) attention through the C ABI against the oracle: the reference suite's cases with their
padded strides (generic path), the same shapes with aligned strides (matrix-core path), a production chunk, ring rows and
the contract (PrefillAttentionTests.swift)."""
import numpy as np
import pytest

from gpu_helpers import ctx, dev, host, tfk
from oracle import tfo
from test_oracle_prefill_attention import CASES, kernel_order, make_fixture, reference

pytestmark = pytest.mark.gpu
SENTINEL = 0x7BFF


def run(fx, ring=0, k=None, v=None, raise_on_error=False, **override):
    kk = ctx()
    keep = dict(q=dev(tfo.to_f16_bits(fx["q"])), k=dev(tfo.to_f16_bits(fx["k"] if k is None else k)),
                v=dev(tfo.to_f16_bits(fx["v"] if v is None else v)), out=dev(np.full(fx["chunk"] * fx["o_stride"], SENTINEL, np.uint16)))
    p = tfk.PrefillAttentionParams(fx["start"], fx["chunk"], fx["head_dim"], fx["q_heads"], fx["kv_heads"], fx["kv_valid"], fx["window"],
                                   fx["kv_stride"], fx["q_stride"], fx["o_stride"], fx["scale"])
    for name, value in override.items():
        setattr(p, name, value)
    import ctypes as C
    rc = kk.lib.tf_prefill_attention_causal(kk.handle, None, keep["q"].data_ptr(), 0, keep["k"].data_ptr(), 0, keep["v"].data_ptr(), 0,
                                            keep["out"].data_ptr(), 0, C.byref(p), ring)
    if raise_on_error:
        kk.check(rc)
    rows = host(keep["out"], np.uint16).reshape(fx["chunk"], fx["o_stride"])
    return rc, rows


def check(fx, rows):
    hd, hq = fx["head_dim"], fx["q_heads"]
    assert np.all(rows[:, hq * hd:] == SENTINEL)                 # bytes between rows untouched
    got, ref = tfo.from_f16_bits(rows[:, :hq * hd].reshape(-1)), reference(fx)
    assert np.max(np.abs(got - ref)) <= 2e-2 and tfo.rel_error(got, ref) <= 2e-2      # PrefillAttentionTests.swift:238-239
    want = kernel_order(fx)
    assert np.all(np.abs(got - want) <= 2e-3 * np.maximum(1.0, np.abs(want)))       # about two fp16 steps


@pytest.mark.parametrize("label,start,chunk,window,hd,hq,hkv", CASES)
@pytest.mark.parametrize("pad", [(3, 5, 7), (0, 0, 0), (8, 16, 24)])
def test_reference_suite_cases(label, start, chunk, window, hd, hq, hkv, pad):
    fx = make_fixture(start, chunk, window, 0xA510, hd, hq, hkv, pad)
    rc, rows = run(fx)
    assert rc == tfk.TF_OK
    check(fx, rows)


@pytest.mark.parametrize("start,chunk,window,hd,hq,hkv", [(1000, 128, 1024, 256, 16, 8),     # a chunk of a sliding-window layer
                                                          (640, 128, 0, 512, 16, 2),        # a chunk of a global layer
                                                          (0, 77, 0, 128, 8, 8),            # no grouping, ragged count
                                                          (5, 33, 9, 64, 16, 1),            # sixteen query heads on one kv head
                                                          (1500, 64, 0, 512, 16, 2),        # long context: the keys are split into chunks
                                                          (2100, 128, 1024, 256, 16, 8),    # ... and a window that starts mid-cache
                                                          (700, 40, 0, 128, 4, 4),
                                                          (900, 24, 300, 64, 8, 2)])
def test_production_chunks(start, chunk, window, hd, hq, hkv):
    fx = make_fixture(start, chunk, window, 0xB000 + chunk, hd, hq, hkv, (0, 0, 0))
    rc, rows = run(fx)
    assert rc == tfk.TF_OK
    check(fx, rows)


def test_future_keys_masked_and_ring_rows():
    fx = make_fixture(5, 4, 0, 0xA620, head_dim=64, pad=(0, 0, 0))
    hd, hkv = fx["head_dim"], fx["kv_heads"]
    kk, vv = fx["k"].reshape(-1, fx["kv_stride"]), fx["v"].reshape(-1, fx["kv_stride"])
    for row in range(fx["start"], fx["kv_valid"]):
        for h in range(hkv):
            kk[row, h * hd:(h + 1) * hd] = (row - fx["start"] + 1) * 2.0 + np.arange(hd) * 0.125
            vv[row, h * hd:(h + 1) * hd] = (row - fx["start"] + 1) * -2.0 - np.arange(hd) * 0.125
    rc, rows = run(fx)
    assert rc == tfk.TF_OK
    check(fx, rows)
    # ring of 16 rows, window 8 (prefillAttentionRingCapacityMatchesLinearReference), both paths
    for hd, pad in ((32, (3, 5, 7)), (64, (0, 0, 0))):
        fx = make_fixture(20, 6, 8, 0xA630, head_dim=hd, pad=pad)
        ring = 16
        def wrap(a):
            r = a.reshape(-1, fx["kv_stride"])
            out = np.zeros((ring, fx["kv_stride"]), np.float32)
            for p in range(r.shape[0]):
                out[p % ring] = r[p]
            return out.reshape(-1)
        rc, linear = run(fx)
        rc2, wrapped = run(fx, ring=ring, k=wrap(fx["k"]), v=wrap(fx["v"]))
        assert rc == tfk.TF_OK and rc2 == tfk.TF_OK and np.array_equal(linear, wrapped)
        check(fx, wrapped)


def test_block_equals_decode_attention_row_by_row():
    """The last query of a block sees what a decode step at that position sees."""
    fx = make_fixture(200, 5, 64, 0xA700, head_dim=256, q_heads=16, kv_heads=8, pad=(0, 0, 0))
    rc, rows = run(fx)
    assert rc == tfk.TF_OK
    k = ctx()
    t = fx["chunk"] - 1
    qb = tfo.to_f16_bits(fx["q"]).reshape(fx["chunk"], -1)[t]
    keep = dict(q=dev(qb), k=dev(tfo.to_f16_bits(fx["k"])), v=dev(tfo.to_f16_bits(fx["v"])), out=dev(np.zeros(16 * 256, np.uint16)))
    k.attention_swa(keep["q"], keep["k"], keep["v"], keep["out"], 256, 16, 8, fx["start"] + t + 1, 64, 1.0)
    single = tfo.from_f16_bits(host(keep["out"], np.uint16))
    assert np.max(np.abs(single - tfo.from_f16_bits(rows[t, :16 * 256]))) <= 2e-3


@pytest.mark.parametrize("start,count,window,hd,hq,hkv", [(32640, 128, 0, 512, 16, 2),       # a global layer at the end of a 32768-token context
                                                          (8000, 128, 1024, 256, 16, 8)])   # a sliding-window layer deep into the context
def test_full_context_sizes_through_the_identical_keys_property(start, count, window, hd, hq, hkv):
    # every key row identical: all visible positions weigh the same whatever the queries are, so query t must return the mean
    # of the V rows it sees - a closed form that needs no O(N^2) reference at these sizes
    import torch
    rng = np.random.default_rng(0xC0DE + hd)
    kv_valid = start + count
    key = rng.standard_normal(hkv * hd).astype(np.float16) * np.float16(0.25)
    k_rows = np.broadcast_to(key, (kv_valid, hkv * hd)).copy()
    v_rows = rng.standard_normal((kv_valid, hkv * hd)).astype(np.float16)
    q_rows = (rng.standard_normal((count, hq * hd)) * 0.25).astype(np.float16)
    kk = ctx()
    d_q, d_k, d_v = dev(q_rows.view(np.uint16).ravel()), dev(k_rows.view(np.uint16).ravel()), dev(v_rows.view(np.uint16).ravel())
    out = dev(np.zeros(count * hq * hd, np.uint16))
    p = tfk.PrefillAttentionParams(start, count, hd, hq, hkv, kv_valid, window, hkv * hd, hq * hd, hq * hd, 1.0 / np.sqrt(hd))
    import ctypes as C
    kk.check(kk.lib.tf_prefill_attention_causal(kk.handle, None, d_q.data_ptr(), 0, d_k.data_ptr(), 0, d_v.data_ptr(), 0, out.data_ptr(), 0, C.byref(p), 0))
    got = tfo.from_f16_bits(host(out, np.uint16)).reshape(count, hq, hd)
    prefix = np.concatenate([np.zeros((1, hkv * hd)), np.cumsum(v_rows.astype(np.float64), axis=0)])
    group = hq // hkv
    for t in range(count):
        last = start + t + 1
        first = max(0, last - window) if window else 0
        mean = ((prefix[last] - prefix[first]) / (last - first)).reshape(hkv, hd)
        want = np.repeat(mean, group, axis=0)
        assert np.max(np.abs(got[t] - want)) <= 2e-3, t


def test_contract():
    fx = make_fixture(4, 3, 0, 1, head_dim=64, pad=(0, 0, 0))
    bad = tfk.TF_ERR_INVALID_ARGUMENT
    assert run(fx, head_dim=0)[0] == bad and run(fx, query_count=0)[0] == bad                   # PrefillAttention.swift:121-122
    assert run(fx, num_q_heads=3)[0] == bad                                                     # :125-126
    assert run(fx, q_token_stride_elements=255)[0] == bad and run(fx, o_token_stride_elements=255)[0] == bad   # :127-130
    assert run(fx, kv_token_stride_elements=127)[0] == bad                                      # :131-132
    assert run(fx, kv_valid_count=6)[0] == bad                                                  # :133-134

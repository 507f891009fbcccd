"""Pins the prefill-attention part of the oracle: the restated test reference against torch's float64 masked attention,
the kernel-order path against it on the reference suite's cases (PrefillAttentionTests.swift), and the properties the
masks fix (a query never sees a later key; one visible key returns its V row).  CPU only."""
import numpy as np
import pytest
import torch

from oracle import tfo


def make_fixture(start, chunk, window, seed, head_dim=8, q_heads=4, kv_heads=2, pad=(3, 5, 7)):
    """PrefillAttentionTests.swift:194-232: strides with padding, q / k / v ~ U(-0.35, 0.35), kv_valid = start + chunk, scale 1."""
    q_stride, kv_stride, o_stride = q_heads * head_dim + pad[0], kv_heads * head_dim + pad[1], q_heads * head_dim + pad[2]
    kv_valid = start + chunk
    rng = tfo.SeedTree(seed).key(f"prefill-attn-start{start}-chunk{chunk}-window{window}")
    q = np.zeros(chunk * q_stride, np.float32)
    k = np.zeros(kv_valid * kv_stride, np.float32)
    v = np.zeros(kv_valid * kv_stride, np.float32)
    q.reshape(chunk, q_stride)[:, :q_heads * head_dim] = rng.uniform_array(-0.35, 0.35, chunk * q_heads * head_dim).reshape(chunk, -1)
    kv = rng.uniform_array(-0.35, 0.35, 2 * kv_valid * kv_heads * head_dim).reshape(kv_valid, kv_heads, head_dim, 2)
    k.reshape(kv_valid, kv_stride)[:, :kv_heads * head_dim] = kv[..., 0].reshape(kv_valid, -1)
    v.reshape(kv_valid, kv_stride)[:, :kv_heads * head_dim] = kv[..., 1].reshape(kv_valid, -1)
    return dict(q=q, k=k, v=v, q_stride=q_stride, kv_stride=kv_stride, o_stride=o_stride, head_dim=head_dim, q_heads=q_heads,
                kv_heads=kv_heads, start=start, chunk=chunk, kv_valid=kv_valid, window=window, scale=1.0)


def reference(fx):
    f16 = lambda a: tfo.from_f16_bits(tfo.to_f16_bits(a))
    return tfo.prefill_attention_ref(f16(fx["q"]), f16(fx["k"]), f16(fx["v"]), fx["start"], fx["chunk"], fx["head_dim"], fx["q_heads"],
                                     fx["kv_heads"], fx["kv_valid"], fx["window"], fx["q_stride"], fx["kv_stride"], fx["scale"])


def kernel_order(fx, ring=0, k=None, v=None):
    out = np.full(fx["chunk"] * fx["o_stride"], 0x7BFF, np.uint16)
    got = tfo.k_prefill_attention(tfo.to_f16_bits(fx["q"]), tfo.to_f16_bits(fx["k"] if k is None else k), tfo.to_f16_bits(fx["v"] if v is None else v),
                                  out, fx["start"], fx["chunk"], fx["head_dim"], fx["q_heads"], fx["kv_heads"], fx["kv_valid"], fx["window"],
                                  fx["q_stride"], fx["kv_stride"], fx["o_stride"], fx["scale"], ring)
    rows = got.reshape(fx["chunk"], fx["o_stride"])
    assert np.all(rows[:, fx["q_heads"] * fx["head_dim"]:] == 0x7BFF)          # padding between rows untouched
    return tfo.from_f16_bits(rows[:, :fx["q_heads"] * fx["head_dim"]].reshape(-1))


CASES = [("full-origin", 0, 3, 0, 8, 4, 2), ("full-offset", 4, 3, 0, 8, 4, 2), ("swa-inside-window", 2, 4, 16, 8, 4, 2),
         ("swa-truncated", 7, 4, 5, 8, 4, 2), ("swa-current-key-at-1023", 1023, 1, 1, 256, 16, 8), ("full-short-gqa", 3, 1, 0, 512, 16, 2),
         ("swa-production-window-1024", 1023, 4, 1024, 256, 16, 8), ("full-production-gqa", 31, 8, 0, 512, 16, 2)]


@pytest.mark.parametrize("label,start,chunk,window,hd,hq,hkv", CASES)
def test_reference_equals_torch_masked_attention(label, start, chunk, window, hd, hq, hkv):
    fx = make_fixture(start, chunk, window, 0xA510, hd, hq, hkv)
    got = reference(fx).reshape(chunk, hq, hd)
    f16 = lambda a: tfo.from_f16_bits(tfo.to_f16_bits(a)).astype(np.float64)
    q = torch.from_numpy(f16(fx["q"]).reshape(chunk, fx["q_stride"])[:, :hq * hd].reshape(chunk, hq, hd))
    k = torch.from_numpy(f16(fx["k"]).reshape(-1, fx["kv_stride"])[:, :hkv * hd].reshape(-1, hkv, hd)).repeat_interleave(hq // hkv, dim=1)
    v = torch.from_numpy(f16(fx["v"]).reshape(-1, fx["kv_stride"])[:, :hkv * hd].reshape(-1, hkv, hd)).repeat_interleave(hq // hkv, dim=1)
    s = torch.einsum("thd,phd->htp", q, k)
    pos = torch.arange(fx["kv_valid"])[None, :]
    absq = (start + torch.arange(chunk))[:, None]
    mask = pos <= absq
    if window:
        mask &= pos > absq - window
    s = s.masked_fill(~mask[None], float("-inf"))
    want = torch.einsum("htp,phd->thd", torch.softmax(s, dim=-1), v).numpy()
    assert np.max(np.abs(got - want)) < 2e-6


@pytest.mark.parametrize("label,start,chunk,window,hd,hq,hkv", CASES)
def test_kernel_order_path_within_the_reference_tolerance(label, start, chunk, window, hd, hq, hkv):
    # PrefillAttentionTests.swift:234-240: maxAbs <= 2e-2 and rel <= 2e-2
    fx = make_fixture(start, chunk, window, 0xA510, hd, hq, hkv)
    got, ref = kernel_order(fx), reference(fx)
    assert np.max(np.abs(got - ref)) <= 2e-2 and tfo.rel_error(got, ref) <= 2e-2


def test_future_keys_are_masked_and_single_key_returns_its_row():
    # prefillAttentionMasksFutureChunkTokens (:73-92): rows of the chunk itself carry huge keys; a query must not see later ones
    fx = make_fixture(5, 4, 0, 0xA620)
    hd, hkv = fx["head_dim"], fx["kv_heads"]
    kk, vv = fx["k"].reshape(-1, fx["kv_stride"]), fx["v"].reshape(-1, fx["kv_stride"])
    for row in range(fx["start"], fx["kv_valid"]):
        for h in range(hkv):
            kk[row, h * hd:(h + 1) * hd] = (row - fx["start"] + 1) * 2.0 + np.arange(hd) * 0.125
            vv[row, h * hd:(h + 1) * hd] = (row - fx["start"] + 1) * -2.0 - np.arange(hd) * 0.125
    got, ref = kernel_order(fx), reference(fx)
    assert np.max(np.abs(got - ref)) <= 2e-2 and tfo.rel_error(got, ref) <= 2e-2
    # window 1: every query sees only its own key -> its own V row
    one = make_fixture(9, 3, 1, 0xA621)
    out = kernel_order(one).reshape(3, one["q_heads"], one["head_dim"])
    vrows = tfo.from_f16_bits(tfo.to_f16_bits(one["v"])).reshape(-1, one["kv_stride"])
    for t in range(3):
        for h in range(one["q_heads"]):
            kvh = h // 2
            assert np.array_equal(out[t, h], vrows[9 + t, kvh * 8:(kvh + 1) * 8])


def test_ring_rows_equal_linear_rows():
    # prefillAttentionRingCapacityMatchesLinearReference (:42-71)
    fx = make_fixture(20, 6, 8, 0xA630, head_dim=32)
    ring = 16
    def wrap(a):
        rows = a.reshape(-1, fx["kv_stride"])
        out = np.zeros((ring, fx["kv_stride"]), np.float32)
        for p in range(rows.shape[0]):
            out[p % ring] = rows[p]
        return out.reshape(-1)
    assert np.array_equal(kernel_order(fx), kernel_order(fx, ring=ring, k=wrap(fx["k"]), v=wrap(fx["v"])))

"""GPU: a packed-experts layer file uploaded into a resident pool in logical order, then used by the decode step."""
import ctypes as C

import numpy as np
import pytest

import test_gpu_moe as M
from gpu_helpers import ctx, dev, host, tfk, zeros_bytes

pytestmark = pytest.mark.gpu


def test_layer_file_upload_in_logical_order_feeds_the_decode_step(tmp_path):
    d, f, num_experts = 2816, 128, 16
    c = M._decode_step_case(d, f, num_experts, 0x10AD)
    stride = 16384 * ((c["blobs"][0].size + 16383) // 16384)          # GTurboFormatV1.alignmentBytes
    ranks = np.random.default_rng(3).permutation(num_experts).astype(np.uint32)     # logical expert -> position in the file
    layer = np.zeros(num_experts * stride, np.uint8)
    for e, blob in enumerate(c["blobs"]):
        layer[int(ranks[e]) * stride:int(ranks[e]) * stride + blob.size] = blob
    path = tmp_path / "layer_00.bin"
    layer.tofile(path)
    k = ctx()
    pool = zeros_bytes(num_experts * stride, 0xEE)
    k.check(k.lib.tf_upload_packed_experts_layer(k.handle, None, str(path).encode(), stride, num_experts, ranks.ctypes.data_as(C.POINTER(C.c_uint32)),
                                                 pool.data_ptr()))
    got = host(pool, np.uint8).reshape(num_experts, stride)
    for e, blob in enumerate(c["blobs"]):
        assert np.array_equal(got[e, :blob.size], blob), e
    # the same step through the uploaded pool and through a pool laid out by hand
    t = M._decode_step_tensors(c)
    want = M._fresh_outs(d, f)
    k.check(M._decode_step_call(k, t, c, d, f, num_experts, want))
    t["pool"] = pool
    c2 = dict(c, stride=stride)
    outs = M._fresh_outs(d, f)
    k.check(M._decode_step_call(k, t, c2, d, f, num_experts, outs))
    for a, b in zip(M._read_outs(outs, d, f), M._read_outs(want, d, f)):
        assert np.array_equal(a, b)
    # identity order, and the contract
    k.check(k.lib.tf_upload_packed_experts_layer(k.handle, None, str(path).encode(), stride, num_experts, None, pool.data_ptr()))
    assert np.array_equal(host(pool, np.uint8), layer)
    bad = tfk.TF_ERR_INVALID_ARGUMENT
    assert k.lib.tf_upload_packed_experts_layer(k.handle, None, str(tmp_path / "missing.bin").encode(), stride, num_experts, None, pool.data_ptr()) == bad
    assert k.lib.tf_upload_packed_experts_layer(k.handle, None, str(path).encode(), stride, num_experts + 1, None, pool.data_ptr()) == tfk.TF_ERR_DIMENSION_MISMATCH
    twice = ranks.copy()
    twice[1] = twice[0]
    assert k.lib.tf_upload_packed_experts_layer(k.handle, None, str(path).encode(), stride, num_experts, twice.ctypes.data_as(C.POINTER(C.c_uint32)),
                                                pool.data_ptr()) == bad
    assert k.lib.tf_upload_packed_experts_layer(k.handle, None, str(tmp_path).encode(), stride, num_experts, None, pool.data_ptr()) == bad   # a directory


def test_resident_payload_upload_and_shared_expert_through_tensor_views(tmp_path):
    """model_weights.bin = index region (16 KiB aligned) + payload: the payload goes to one device allocation
    (ResidentBuffer.swift:15-78) and the shared expert runs on (payload, offset) operands as Model.resident hands them out
    (Model.swift:186-227)."""
    import refcases
    from oracle import tfo
    d, f = 128, 64
    c = refcases.shared_expert_case(d, f)
    index_size = 16384
    # payload: filler so that the copy takes several staging chunks, then gate / up / down as W, S, B back to back
    filler = np.random.default_rng(5).integers(0, 256, 35 * 1024 * 1024 + 2, dtype=np.uint8)
    parts, offsets, pos = [filler], {}, filler.size
    for name in ("gate", "up", "down"):
        for role, arr in zip(("w", "s", "b"), c[name]):
            raw = np.ascontiguousarray(arr).view(np.uint8).ravel()
            offsets[name, role] = pos
            parts.append(raw)
            pos += raw.size
    payload = np.concatenate(parts)
    path = tmp_path / "model_weights.bin"
    with open(path, "wb") as fh:
        fh.write(bytes(index_size))
        fh.write(payload.tobytes())
    k = ctx()
    device = zeros_bytes(payload.size, 0xEE)
    k.check(k.lib.tf_upload_file_region(k.handle, None, str(path).encode(), index_size, payload.size, device.data_ptr()))
    assert np.array_equal(host(device, np.uint8), payload)

    def proj(name, rows, cols):
        return tfk.projection(device, device, device, rows, cols, offsets=(offsets[name, "w"], offsets[name, "s"], offsets[name, "b"]))
    x, y = dev(c["x_bits"]), zeros_bytes(d * 2)
    sg, su, sa = zeros_bytes(f * 2), zeros_bytes(f * 2), zeros_bytes(f * 2)
    k.shared_expert_int4(x, proj("gate", f, d), proj("up", f, d), proj("down", d, f), y, sg, su, sa)
    ref = tfo.shared_expert_ref(c["gate"], c["up"], c["down"], tfo.from_f16_bits(c["x_bits"]))
    assert tfo.rel_error(tfo.from_f16_bits(host(y, np.uint16, d)), ref) < 6e-3
    # the contract
    enc = str(path).encode()
    assert k.lib.tf_upload_file_region(k.handle, None, enc, index_size, payload.size + 1, device.data_ptr()) == tfk.TF_ERR_DIMENSION_MISMATCH
    assert k.lib.tf_upload_file_region(k.handle, None, enc, index_size, 0, device.data_ptr()) == tfk.TF_ERR_INVALID_ARGUMENT
    assert k.lib.tf_upload_file_region(k.handle, None, str(tmp_path).encode(), 0, 16, device.data_ptr()) == tfk.TF_ERR_INVALID_ARGUMENT
    assert k.lib.tf_upload_file_region(k.handle, None, str(tmp_path / "missing.bin").encode(), 0, 16, device.data_ptr()) == tfk.TF_ERR_INVALID_ARGUMENT
    # a sub-range in the middle
    part = zeros_bytes(1000, 0xEE)
    k.check(k.lib.tf_upload_file_region(k.handle, None, enc, index_size + 12345, 1000, part.data_ptr()))
    assert np.array_equal(host(part, np.uint8), payload[12345:13345])

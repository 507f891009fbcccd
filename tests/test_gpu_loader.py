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

"""The decode step that allocates nothing (tf_moe_decode_step_static: router logits in a load-time device array) against
tf_moe_decode_step, bit for bit, through the C ABI: two calls in a row, the second on a smaller problem."""
import numpy as np
import pytest

from gpu_helpers import ctx, host, tfk
from test_gpu_moe import _decode_step_call, _decode_step_case, _decode_step_tensors, _fresh_outs, _read_outs

pytestmark = pytest.mark.gpu


def _static_call(k, t, c, d, f, num_experts, outs):
    idx, wts, acts, y = outs
    off = tfk.ExpertOffsets(*c["off"].as_tuple())
    return k.lib.tf_moe_decode_step_static(k.handle, None, t["rW"].data_ptr(), 0, t["rS"].data_ptr(), 0, t["rB"].data_ptr(), 0,
                                           t["x"].data_ptr(), t["eff"].data_ptr(), 0, t["gain"].data_ptr(), 0, t["pool"].data_ptr(),
                                           c["stride"], num_experts, off, t["x"].data_ptr(), acts.data_ptr(), t["res"].data_ptr(),
                                           y.data_ptr(), idx.data_ptr(), wts.data_ptr(), d, f, 8, tfk.TF_BF16)


def test_static_decode_step_equals_the_allocating_one_on_two_calls_in_a_row():
    k = ctx()
    # production shape (the fused selection inside phase 1), then a smaller one (200 -> 16 experts, short rows: the
    # separate selection kernel and the half-wave row kernels); the second call finds the first call's logits in the array
    shapes = [(2816, 704, 200), (704, 128, 16)]
    cases = [(_decode_step_case(d, f, e, 0xA110C + d), d, f, e) for d, f, e in shapes]
    tensors = [_decode_step_tensors(c) for c, _, _, _ in cases]
    want = []
    for (c, d, f, e), t in zip(cases, tensors):
        o = _fresh_outs(d, f)
        k.check(_decode_step_call(k, t, c, d, f, e, o))
        k.synchronize()
        want.append(_read_outs(o, d, f))
    outs = [_fresh_outs(d, f) for _, d, f, _ in cases]
    for (c, d, f, e), t, o in zip(cases, tensors, outs):      # back to back on one stream, no host wait in between
        k.check(_static_call(k, t, c, d, f, e, o))
    k.synchronize()
    for (c, d, f, e), o, w in zip(cases, outs, want):
        for name, a, b in zip(("indices", "weights", "acts", "y"), _read_outs(o, d, f), w):
            assert np.array_equal(a, b), (name, d, f, e)
    assert len(set(want[0][0])) == 8 and max(want[0][0]) < 200


def test_static_decode_step_rejects_more_experts_than_its_scratch_holds():
    k = ctx()
    c = _decode_step_case(704, 128, 16, 0xA110C)
    t = _decode_step_tensors(c)
    o = _fresh_outs(704, 128)
    rc = _static_call(k, t, c, 704, 128, 257, o)
    assert rc == tfk.TF_ERR_SCRATCH_TOO_SMALL
    assert "256" in k.last_error()
    assert not host(o[3], np.uint8).any()       # nothing was enqueued

"""Pins the oracle's prefill pieces: grouping against the reference's literal expected arrays,
struct layouts, and the numeric references against float64."""
import ctypes as C

import numpy as np
import pytest
import torch

import refcases
from test_oracle_quant_gemv import np_dequant


def P(tfo, rows):
    return tfo.pairs_from_tuples(rows)


def test_struct_layouts(tfo):
    # PrefillRouterTests.swift:12-19; MoE.swift:4-29
    assert tfo.PAIR_DTYPE.itemsize == 16
    assert [tfo.PAIR_DTYPE.fields[n][1] for n in ("token", "expert", "rank", "weight_bits")] == [0, 4, 8, 12]
    assert C.sizeof(tfo.ExpertOffsets) == 36
    assert tfo.GROUP_DTYPE.itemsize == 12 and tfo.TILE_DTYPE.itemsize == 16


def test_grouping_literal_known_answer(tfo):
    # PrefillMoEGroupingTests.swift:6-56
    rows = [(0, 3, 0, 10), (0, 1, 1, 11), (0, 4, 2, 12), (1, 1, 0, 13), (1, 3, 1, 14), (1, 2, 2, 15),
            (2, 4, 0, 16), (2, 3, 1, 17), (2, 1, 2, 18), (3, 5, 0, 19), (3, 1, 1, 20), (3, 4, 2, 21)]
    g = tfo.group_pairs(P(tfo, rows[::-1]), 4, 3, 6, tile_expert_count=2)
    sp = g["sorted_pairs"]
    assert list(sp["expert"]) == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert [[int(t), int(r)] for t, r in zip(sp["token"], sp["rank"])] == [
        [0, 1], [1, 0], [2, 2], [3, 1], [1, 2], [0, 0], [1, 1], [2, 1], [0, 2], [2, 0], [3, 2], [3, 0]]
    assert list(g["per_expert_offsets"]) == [0xFFFFFFFF, 0, 4, 5, 8, 11]
    assert list(g["per_expert_counts"]) == [0, 4, 1, 3, 3, 1]
    assert [tuple(int(v) for v in x) for x in g["groups"]] == [(1, 0, 4), (2, 4, 1), (3, 5, 3), (4, 8, 3), (5, 11, 1)]
    assert [tuple(int(v) for v in x) for x in g["tiles"]] == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]
    assert max(int(x) for x in g["groups"]["pair_count"]) == 4
    assert max(int(x) for x in g["tiles"]["pair_count"]) == 6
    assert max(int(x) for x in g["tiles"]["group_count"]) == 2


def test_grouping_is_order_independent_and_keeps_weight_bits(tfo):
    # PrefillMoEGroupingTests.swift:58-87
    tm = [(0, 2, 0, 101), (0, 1, 1, 102), (1, 2, 0, 103), (1, 0, 1, 104), (2, 1, 0, 105), (2, 2, 1, 106)]
    sh = [tm[5], tm[1], tm[3], tm[0], tm[4], tm[2]]
    a = tfo.group_pairs(P(tfo, tm), 3, 2, 3, tile_expert_count=2)
    b = tfo.group_pairs(P(tfo, sh), 3, 2, 3, tile_expert_count=2)
    for k in ("sorted_pairs", "per_expert_offsets", "per_expert_counts", "groups", "tiles"):
        assert np.array_equal(a[k], b[k])
    assert list(a["sorted_pairs"]["weight_bits"]) == [104, 102, 105, 101, 103, 106]


def test_grouping_with_expert_sort_keys(tfo):
    # PrefillMoEGroupingTests.swift:89-123
    rows = [(0, 1, 0, 10), (0, 2, 1, 20), (1, 3, 0, 30), (1, 1, 1, 11), (2, 2, 0, 21), (2, 3, 1, 31)]
    g = tfo.group_pairs(P(tfo, rows), 3, 2, 4, tile_expert_count=2, expert_sort_keys=[0, 30, 10, 20])
    assert list(g["groups"]["expert"]) == [2, 3, 1]
    assert list(g["sorted_pairs"]["expert"]) == [2, 2, 3, 3, 1, 1]
    assert list(g["per_expert_offsets"]) == [0xFFFFFFFF, 4, 0, 2]
    assert [tuple(int(v) for v in x) for x in g["tiles"]] == [(0, 2, 0, 4), (2, 1, 4, 2)]
    for t in g["tiles"]:
        sl = g["sorted_pairs"][int(t["pair_start"]):int(t["pair_start"] + t["pair_count"])]
        ex = g["groups"][int(t["group_start"]):int(t["group_start"] + t["group_count"])]["expert"]
        assert set(sl["expert"]) == set(ex)


def test_grouping_rejects_invalid_metadata(tfo):
    # PrefillMoEGroupingTests.swift:125-177 + the remaining guards of PrefillMoEGrouping.swift:99-139
    cases = [
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=1, tile=17), "invalidTileExpertCount"),
        (dict(pairs=[(0, 2, 0, 1)], q=1, k=1, e=2, tile=1), "expertOutOfRange"),
        (dict(pairs=[(0, 0, 0, 1), (0, 1, 0, 2)], q=1, k=2, e=2, tile=1), "duplicateTokenRank"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=2, tile=1, keys=[0]), "expertSortKeyCountMismatch"),
        (dict(pairs=[(0, 0, 0, 1)], q=-1, k=1, e=1, tile=1), "invalidQueryCount"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=0, e=1, tile=1), "invalidTopK"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=0, tile=1), "invalidNumExperts"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=1, tile=0), "invalidTileExpertCount"),
        (dict(pairs=[(0, 0, 0, 1)], q=2, k=1, e=1, tile=1), "pairCountMismatch"),
        (dict(pairs=[(1, 0, 0, 1)], q=1, k=1, e=1, tile=1), "tokenOutOfRange"),
        (dict(pairs=[(0, 0, 1, 1)], q=1, k=1, e=1, tile=1), "rankOutOfRange"),
    ]
    for c, want in cases:
        with pytest.raises(tfo.GroupingError) as ei:
            tfo.group_pairs(P(tfo, c["pairs"]), c["q"], c["k"], c["e"], tile_expert_count=c["tile"],
                            expert_sort_keys=c.get("keys"))
        assert ei.value.case == want


def test_grouping_real_trace_pressure_t32(tfo):
    # PrefillMoEGroupingTests.swift:179-207
    rows = [(t, (t + r * 7) % 74, r, t * 8 + r) for t in range(32) for r in range(8)]
    g = tfo.group_pairs(P(tfo, rows), 32, 8, 128, tile_expert_count=16)
    assert g["sorted_pairs"].size == 256 and g["groups"].size <= 74
    assert all(int(t["group_count"]) <= 16 and int(t["pair_count"]) > 0 for t in g["tiles"])
    assert int(g["per_expert_counts"].sum()) == 256
    # empty input is legal: zero groups, zero tiles
    e = tfo.group_pairs(P(tfo, []), 0, 8, 128)
    assert e["groups"].size == 0 and e["tiles"].size == 0 and np.all(e["per_expert_offsets"] == 0xFFFFFFFF)


def test_make_pairs_is_token_major(tfo):
    # PrefillRouterTests.swift:21-31
    w = tfo.to_f16_bits(np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6], np.float32))
    p = tfo.make_pairs([3, 1, 2, 4, 0, 5], w, 2, 3)
    assert list(p["token"]) == [0, 0, 0, 1, 1, 1] and list(p["rank"]) == [0, 1, 2, 0, 1, 2]
    assert list(p["expert"]) == [3, 1, 2, 4, 0, 5] and list(p["weight_bits"]) == list(w)


def test_reduce_token_major_vs_float64(tfo):
    # PrefillMoETests.swift:11-18 inputs
    rows, top_k, d = 3, 8, 64
    rng = tfo.SplitMix64(0x4D0E2026)
    partials = tfo.to_f16_bits(rng.uniform_array(-2.0, 2.0, rows * top_k * d))
    weights = tfo.to_f16_bits(rng.uniform_array(-1.0, 1.0, rows * top_k))
    got = tfo.from_f16_bits(tfo.prefill_reduce_token_major(partials, weights, rows, top_k, d))
    p = tfo.from_f16_bits(partials).astype(np.float64).reshape(rows, top_k, d)
    w = tfo.from_f16_bits(weights).astype(np.float64).reshape(rows, top_k, 1)
    assert np.max(np.abs(got.reshape(rows, d) - (p * w).sum(axis=1))) <= 2e-3


def test_route_partials_vs_float64(tfo):
    # PrefillGroupedRoutedMoETests+Execution.swift:8-40 (d=f=64, 3 rows, top-2, 16 synthetic experts)
    d = f = 64
    rows, top_k = 3, 2
    g = tfo.group_pairs(P(tfo, [(0, 2, 0, 0), (0, 0, 1, 0), (1, 1, 0, 0), (1, 2, 1, 0), (2, 0, 0, 0), (2, 1, 1, 0)]),
                        rows, top_k, 16)
    pool, off, stride = refcases.synthetic_expert_pool(16, d, f)
    hidden = tfo.to_f16_bits(((np.arange(rows * d) % 17) - 8).astype(np.float32) * np.float32(0.01))
    got = tfo.from_f16_bits(tfo.prefill_route_partials(g["sorted_pairs"], rows, hidden, d, pool, stride, off, top_k, d, f))
    got = got.reshape(rows, top_k, d)

    def mat(e, w_off, s_off, b_off, r, c):
        base = e * stride
        W = pool[base + w_off: base + w_off + r * c // 2].reshape(r, c // 2)
        S = pool[base + s_off: base + s_off + r * c // 64 * 2].view("<u2").reshape(r, c // 64)
        B = pool[base + b_off: base + b_off + r * c // 64 * 2].view("<u2").reshape(r, c // 64)
        return np_dequant(W, S, B, 4, tfo).astype(np.float64)

    for p in g["sorted_pairs"]:
        t, e, r = int(p["token"]), int(p["expert"]), int(p["rank"])
        x = tfo.from_f16_bits(hidden[t * d:(t + 1) * d]).astype(np.float64)
        gate = mat(e, off.gate_W_off, off.gate_s_off, off.gate_b_off, f, d) @ x
        up = mat(e, off.up_W_off, off.up_s_off, off.up_b_off, f, d) @ x
        act = torch.nn.functional.gelu(torch.from_numpy(gate), approximate="tanh").numpy() * up
        want = mat(e, off.down_W_off, off.down_s_off, off.down_b_off, d, f) @ act
        assert np.max(np.abs(got[t, r] - want)) <= 0.0015


def test_qmm_reference_vs_float64(tfo):
    # MPPPrefillInt4QMMTests.swift:19-60 inputs (plain affine), m=5 n=40 k=128
    m, n, k = 5, 40, 128
    groups = k // 64
    W = ((np.arange(n * k // 2, dtype=np.uint64) * 37 + 0x29) & 0xFF).astype(np.uint8).reshape(n, k // 2)
    r, g = np.arange(n)[:, None], np.arange(groups)[None, :]
    S = tfo.bf16_bits_array((np.float32(0.001) + ((r + g) % 5).astype(np.float32) * np.float32(0.00025))).reshape(n, groups)
    B = tfo.bf16_bits_array((np.float32(-0.01) + ((r * 3 + g) % 7).astype(np.float32) * np.float32(0.002))).reshape(n, groups)
    x = tfo.to_f16_bits((((np.arange(m * k) * 11) % 29 - 14).astype(np.float32) / np.float32(64.0)))
    got = tfo.qmm_cpu_reference(W, S, B, x, m, n, k)
    want = tfo.from_f16_bits(x).astype(np.float64).reshape(m, k) @ np_dequant(W, S, B, 4, tfo).astype(np.float64).T
    assert np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-3)) <= 1e-3
    assert np.array_equal(tfo.qmm_cpu_reference(W, S, B, x, m, n, k, threads=3), got)

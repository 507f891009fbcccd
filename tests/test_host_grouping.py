"""The library's host-side (pure CPU) prefill grouping through the C ABI, against the reference's literal expected arrays
(Tests/TurboFieldfare/Core/Kernels/Prefill/PrefillMoEGroupingTests.swift) and against the oracle.  No GPU needed."""
import ctypes as C
import importlib

import numpy as np
import pytest

tfk = importlib.import_module("turbo-fieldfare_amd")


def test_struct_layouts():
    # PrefillGroupedRoutedMoETests+Layout.swift:8-28 and PrefillRouterTests.swift:12-19
    P = tfk.StreamedParams
    assert C.sizeof(P) == 128
    assert [getattr(P, n).offset for n in ("pair_start", "pair_count", "d", "routed_intermediate", "top_k", "hidden_stride_elements",
                                            "live_expert_count", "local_expert", "gate_W_off", "down_b_off")] == \
        [0, 4, 8, 12, 16, 20, 24, 28, 92, 124]
    assert P.local_expert.offset + 15 * 4 == 88
    assert C.sizeof(tfk.PrefillPair) == 16 and C.sizeof(tfk.PrefillGroup) == 12 and C.sizeof(tfk.PrefillTile) == 16


def test_grouping_literal_known_answer():
    rows = [(0, 3, 0, 10), (0, 1, 1, 11), (0, 4, 2, 12), (1, 1, 0, 13), (1, 3, 1, 14), (1, 2, 2, 15),
            (2, 4, 0, 16), (2, 3, 1, 17), (2, 1, 2, 18), (3, 5, 0, 19), (3, 1, 1, 20), (3, 4, 2, 21)]
    g = tfk.group_token_expert_pairs(rows[::-1], 4, 3, 6, tile_expert_count=2)
    assert [p[1] for p in g["sorted_pairs"]] == [1, 1, 1, 1, 2, 3, 3, 3, 4, 4, 4, 5]
    assert [[p[0], p[2]] for p in g["sorted_pairs"]] == [[0, 1], [1, 0], [2, 2], [3, 1], [1, 2], [0, 0], [1, 1], [2, 1],
                                                         [0, 2], [2, 0], [3, 2], [3, 0]]
    assert g["per_expert_offsets"] == [0xFFFFFFFF, 0, 4, 5, 8, 11]
    assert g["per_expert_counts"] == [0, 4, 1, 3, 3, 1]
    assert g["groups"] == [(1, 0, 4), (2, 4, 1), (3, 5, 3), (4, 8, 3), (5, 11, 1)]
    assert g["tiles"] == [(0, 2, 0, 5), (2, 2, 5, 6), (4, 1, 11, 1)]


def test_grouping_order_independent_and_keeps_weight_bits():
    tm = [(0, 2, 0, 101), (0, 1, 1, 102), (1, 2, 0, 103), (1, 0, 1, 104), (2, 1, 0, 105), (2, 2, 1, 106)]
    sh = [tm[5], tm[1], tm[3], tm[0], tm[4], tm[2]]
    a = tfk.group_token_expert_pairs(tm, 3, 2, 3, tile_expert_count=2)
    b = tfk.group_token_expert_pairs(sh, 3, 2, 3, tile_expert_count=2)
    for k in ("sorted_pairs", "per_expert_offsets", "per_expert_counts", "groups", "tiles"):
        assert a[k] == b[k]
    assert [p[3] for p in a["sorted_pairs"]] == [104, 102, 105, 101, 103, 106]


def test_grouping_with_expert_sort_keys():
    rows = [(0, 1, 0, 10), (0, 2, 1, 20), (1, 3, 0, 30), (1, 1, 1, 11), (2, 2, 0, 21), (2, 3, 1, 31)]
    g = tfk.group_token_expert_pairs(rows, 3, 2, 4, tile_expert_count=2, expert_sort_keys=[0, 30, 10, 20])
    assert [x[0] for x in g["groups"]] == [2, 3, 1]
    assert [p[1] for p in g["sorted_pairs"]] == [2, 2, 3, 3, 1, 1]
    assert g["per_expert_offsets"] == [0xFFFFFFFF, 4, 0, 2]
    assert g["tiles"] == [(0, 2, 0, 4), (2, 1, 4, 2)]


def test_grouping_rejects_invalid_metadata():
    cases = [
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=1, tile=17), "invalidTileExpertCount"),
        (dict(pairs=[(0, 2, 0, 1)], q=1, k=1, e=2, tile=1), "expertOutOfRange"),
        (dict(pairs=[(0, 0, 0, 1), (0, 1, 0, 2)], q=1, k=2, e=2, tile=1), "duplicateTokenRank"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=2, tile=1, keys=[0]), "expertSortKeyCountMismatch"),
        (dict(pairs=[(0, 0, 0, 1)], q=-1, k=1, e=1, tile=1), "invalidQueryCount"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=0, e=1, tile=1), "invalidTopK"),
        (dict(pairs=[(0, 0, 0, 1)], q=1, k=1, e=0, tile=1), "invalidNumExperts"),
        (dict(pairs=[(0, 0, 0, 1)], q=2, k=1, e=1, tile=1), "pairCountMismatch"),
        (dict(pairs=[(1, 0, 0, 1)], q=1, k=1, e=1, tile=1), "tokenOutOfRange"),
        (dict(pairs=[(0, 0, 1, 1)], q=1, k=1, e=1, tile=1), "rankOutOfRange"),
    ]
    for c, want in cases:
        with pytest.raises(tfk.TFError) as ei:
            tfk.group_token_expert_pairs(c["pairs"], c["q"], c["k"], c["e"], tile_expert_count=c["tile"], expert_sort_keys=c.get("keys"))
        assert tfk.GROUP_ERRORS[ei.value.status] == want


def test_grouping_matches_oracle_on_random_routes(tfo):
    rng = np.random.default_rng(9)
    for T, k, E, tile in [(32, 8, 128, 16), (7, 3, 5, 2), (200, 8, 64, 8), (0, 8, 128, 16)]:
        idx = np.stack([rng.choice(E, size=k, replace=False) for _ in range(T)]).astype(np.uint32) if T else np.zeros((0, k), np.uint32)
        w = rng.integers(0, 0x3C00, (T, k)).astype(np.uint16)
        pairs = tfk.make_token_expert_pairs(idx.ravel(), w.ravel(), T, k)
        mine = tfk.group_token_expert_pairs([(p.token, p.expert, p.rank, p.weight_bits_and_reserved) for p in pairs[:T * k]], T, k, E, tile)
        ref = tfo.group_pairs(tfo.make_pairs(idx.ravel(), w.ravel(), T, k), T, k, E, tile)
        assert mine["sorted_pairs"] == [tuple(int(v) for v in p) for p in ref["sorted_pairs"]]
        assert mine["per_expert_offsets"] == [int(v) for v in ref["per_expert_offsets"]]
        assert mine["per_expert_counts"] == [int(v) for v in ref["per_expert_counts"]]
        assert mine["groups"] == [tuple(int(v) for v in g) for g in ref["groups"]]
        assert mine["tiles"] == [tuple(int(v) for v in t) for t in ref["tiles"]]


def test_make_pairs_is_token_major():
    w = np.array([0.1, 0.2, 0.3, 0.4, 0.5, 0.6], np.float16).view(np.uint16)
    p = tfk.make_token_expert_pairs([3, 1, 2, 4, 0, 5], w, 2, 3)
    assert [x.token for x in p[:6]] == [0, 0, 0, 1, 1, 1] and [x.rank for x in p[:6]] == [0, 1, 2, 0, 1, 2]
    assert [x.expert for x in p[:6]] == [3, 1, 2, 4, 0, 5] and [x.weight_bits_and_reserved for x in p[:6]] == list(w)

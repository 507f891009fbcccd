"""The committed fixtures under tests/golden/ against the CPU oracle: every array the generator would write today must
equal the stored one bit for bit (so a change of the oracle shows up here), plus known answers that do not come from
the oracle at all (the published SplitMix64 vector, closed forms for the stored outputs)."""
import importlib.util
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
_spec = importlib.util.spec_from_file_location("make_golden", os.path.join(GOLDEN, "make_golden.py"))
make_golden = importlib.util.module_from_spec(_spec)
_spec.loader.exec_module(make_golden)


def load(case):
    with np.load(os.path.join(GOLDEN, case + ".npz"), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


@pytest.mark.parametrize("case", sorted(make_golden.CASES))
def test_oracle_reproduces_fixture_bit_for_bit(case):
    stored, fresh = load(case), make_golden.generate(case)
    assert sorted(stored) == sorted(fresh)
    for name in stored:
        assert stored[name].dtype == fresh[name].dtype and stored[name].shape == fresh[name].shape, name
        assert stored[name].tobytes() == fresh[name].tobytes(), f"{case}:{name}"


def test_splitmix64_published_vector():
    # Steele/Lea/Flood SplitMix64, seed 0 and seed 1234567: the values every public implementation lists
    z = load("prng_streams")
    assert [int(v) for v in z["next_0"][:3]] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    assert [int(v) for v in z["next_12d687"][:2]] == [6457827717110365317, 3203168211198807973]


def test_gemv_fixture_outputs_follow_from_its_inputs_in_float64():
    z = load("gemv_int4_m64_k128")
    W = z["W"]
    q = np.empty((64, 128), np.float64)
    q[:, 0::2], q[:, 1::2] = W & 0xF, W >> 4                     # low nibble = even element
    s = (z["S"].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    b = (z["B"].astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    w = q * np.repeat(s, 64, axis=1) + np.repeat(b, 64, axis=1)
    assert np.array_equal(w.astype(np.float32), z["dequantized"])
    x = z["x_bits"].view(np.float16).astype(np.float64)
    y = w @ x
    assert np.max(np.abs(z["y_ref"] - y)) < 2e-5 and np.max(np.abs(z["y_kernel_order"] - y)) < 2e-5
    assert np.max(np.abs(z["dequantized"] - z["raw"])) <= float(s.max()) * 0.5 + 4e-3   # RTN error bound incl. bf16 rounding of s, b


def test_router_fixture_matches_the_reference_tests_literals():
    z = load("router_e16_d128")
    assert list(z["tie_indices"]) == [0, 1, 2, 3, 4, 5, 6, 8]                     # RouterTopKTests.swift:64-69
    for name in ("prod", "tie"):
        logits, idx = z[f"{name}_logits"].astype(np.float64), z[f"{name}_indices"]
        order = sorted(range(16), key=lambda e: (-logits[e], e))[:8]
        assert list(idx) == order
        p = np.exp(logits[idx] - logits[idx].max())
        gains = (z[f"{name}_per_expert_bits"].astype(np.uint32) << 16).view(np.float32)[idx]
        assert np.allclose(z[f"{name}_weights"], p / p.sum() * gains, rtol=2e-6, atol=1e-7)


def test_lm_head_fixture_known_tokens():
    z = load("lm_head_d64_v1024")
    assert int(z["tie_token"][0]) == 17 and int(z["target_token"][0]) == 1021     # LMHeadChainInt4Tests.swift:136-193
    finite = np.where(np.isfinite(z["logits"]), z["logits"], -np.inf)
    assert int(z["token"][0]) == int(np.argmax(finite))


def test_prefill_fixture_is_a_stable_sort_and_a_weighted_sum():
    z = load("prefill_grouped_e6_d128_f64")
    rec = np.dtype([("token", "<u4"), ("expert", "<u4"), ("rank", "<u4"), ("w", "<u2"), ("pad", "<u2")])
    pairs, srt = z["pairs_bytes"].copy().view(rec).ravel(), z["sorted_pairs_bytes"].copy().view(rec).ravel()
    order = sorted(range(pairs.size), key=lambda i: (int(pairs["expert"][i]), i))
    assert [tuple(srt[i].tolist()[:4]) for i in range(srt.size)] == [tuple(pairs[j].tolist()[:4]) for j in order]
    assert list(z["expert_counts"]) == [2, 3, 1, 0, 3, 1] and list(z["expert_offsets"]) == [0, 2, 5, 0xFFFFFFFF, 6, 9]   # absent expert: UInt32.max
    parts = z["route_partials_bits"].view(np.float16).astype(np.float64).reshape(5, 2, 128)
    w = z["weights_bits"].view(np.float16).astype(np.float64).reshape(5, 2, 1)
    red = z["reduced_bits"].view(np.float16).astype(np.float64).reshape(5, 128)
    assert np.max(np.abs(red - (parts * w).sum(1))) <= 1e-3 + 2e-3 * np.max(np.abs(red))

"""bench.py's input streams and its profiler guard, on the CPU.

The benchmark draws the headline workload from the reference's seeded streams in counter form on the device
(Sources/TurboFieldfareValidation/Support/PRNG/SplitMix64.swift:11-23, SeedTree.swift:12-19).  Pinned here by the published
SplitMix64 outputs for seed 0, by the FNV-1a key of a label the reference's own suite uses, and draw for draw against the
sequential generator of the oracle."""
import os
import subprocess
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
import bench  # noqa: E402
from oracle import tfo  # noqa: E402


def test_counter_form_equals_the_published_vectors_and_the_sequential_generator():
    z = bench.splitmix64_draws(torch, 0, 0, 3, device="cpu")
    assert [int(v) & bench._M64 for v in z] == [0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    # a stream entered in the middle continues the same sequence
    whole = bench.splitmix64_draws(torch, 0xDEADBEEF, 0, 1000, device="cpu")
    assert torch.equal(bench.splitmix64_draws(torch, 0xDEADBEEF, 400, 600, device="cpu"), whole[400:])
    # DequantInt4GEMVTests.swift:45 draws from SeedTree(0xC2).key("int4-gemv-kernel-m1024-n2816")
    assert bench.seed_tree_key(0xC2, "int4-gemv-kernel-m1024-n2816") == 0xA38BB6725F0AC119
    assert bench.seed_tree_key(0xC2, "int4-gemv-kernel-m1024-n2816") == tfo.SeedTree(0xC2).key_state("int4-gemv-kernel-m1024-n2816")
    for lo, hi in ((0.005, 0.02), (-0.1, 0.1), (0.0002, 0.0008), (0.0, 1.0)):
        want = tfo.SplitMix64(0x5EED).uniform_array(lo, hi, 4096)
        got = bench.splitmix64_uniform(torch, 0x5EED, 0, 4096, lo, hi, device="cpu").numpy()
        assert np.array_equal(got, want), (lo, hi)


def test_nibbles_are_packed_low_first_and_activations_are_standard_normal():
    seed = 0x1234
    draws = [int(v) & 0xF for v in bench.splitmix64_draws(torch, seed, 0, 64, device="cpu")]
    packed = bench.splitmix64_nibble_bytes(torch, seed, 32, device="cpu", chunk=5).tolist()      # chunking must not show
    assert packed == [draws[2 * b] | (draws[2 * b + 1] << 4) for b in range(32)]
    x = bench.splitmix64_normal_f16(torch, seed, 200000, device="cpu").float()
    assert bool(torch.isfinite(x).all())
    assert abs(float(x.mean())) < 0.01 and abs(float(x.std()) - 1.0) < 0.01
    assert abs(float((x.abs() < 1.0).float().mean()) - 0.6827) < 0.01


def test_all_sections_run_is_refused_under_a_profiler():
    env = dict(os.environ, ROCP_TOOL_LIBRARIES="/opt/rocm/lib/rocprofiler-sdk/librocprofiler-sdk-tool.so")
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--no-cpu"], env=env, capture_output=True, text=True, timeout=120)
    assert res.returncode == 2 and "profiler" in res.stderr and not res.stdout.strip()
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--only-decode-step", "--layer-chain-fork"], env=env, capture_output=True,
                         text=True, timeout=120)
    assert res.returncode == 2
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 2 and "ONE GPU" in res.stderr

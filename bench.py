#!/usr/bin/env python3
"""Benchmark of the int4 MoE matmul path on one MI355X.

A "step" is one token through one MoE layer of the reference model's shape: int8 router (128 x 2816) ->
top-8 + softmax -> phase 1 (gate/up/GeGLU of the 8 selected experts, 704 x 2816 each) -> phase 2 (down 2816 x 704,
weighted reduce).  Expert selection stays on the device.  Weights are synthetic (uniform nibbles, bf16 scale
~U(0.005,0.02), bias ~U(-0.1,0.1)), resident in HBM before the timed region; consecutive steps walk through
several layer replicas and different hidden states so that reads come from HBM, not from L2 / Infinity Cache.

Prints ONE JSON line.  `value` = algorithmic bytes of the step / time per step.
"""
from __future__ import annotations

import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

D, F_MOE, F_SHARED, E, TOPK, VOCAB = 2816, 704, 2112, 128, 8, 262144
HBM_PEAK_GBPS = 8000.0   # MI355X HBM3E, published


def int4_matrix_bytes(rows, cols):
    return rows * cols // 2 + 2 * rows * (cols // 64) * 2


# per-unit algorithmic bytes (what one launch must move at least once)
ROUTER_BYTES = E * D + 2 * E * (D // 64) * 2 + D * 2 + D * 2 + E * 2 + TOPK * 4 + TOPK * 2   # W + s/b + hidden + eff + gains + outputs
# HBM bytes one fused phase-1 launch moves, from hardware counters of `bench.py --only-decode-step` (two rocprofv3 --pmc runs,
# FETCH_SIZE then WRITE_SIZE; profiles/decode_step_counters.txt gives the commands, the raw KiB per dispatch and the factors a
# plain copy of known size calibrates).  The literal below is that file's figure.
PHASE1_TRAFFIC_BYTES = int(8908.2 * 1024 * 1.9999 + 22.1 * 1024)
PHASE1_TRAFFIC_FROM = ("profiles/decode_step_counters.txt: FETCH_SIZE 8908.2 KiB x 1.9999 + WRITE_SIZE 22.1 KiB x 1.0000 per launch of the fused "
                       "phase-1 kernel (factors from the 1 GiB copy of the same runs)")
PHASE1_BYTES = TOPK * 2 * int4_matrix_bytes(F_MOE, D) + D * 2 + TOPK * F_MOE * 2             # gate+up of 8 experts + x + acts out
PHASE2_BYTES = TOPK * int4_matrix_bytes(D, F_MOE) + TOPK * F_MOE * 2 + TOPK * 2 + D * 2 + D * 2   # down of 8 + acts in + w + residual + y
STEP_BYTES = ROUTER_BYTES + PHASE1_BYTES + PHASE2_BYTES
SHARED_BYTES = 2 * int4_matrix_bytes(F_SHARED, D) + int4_matrix_bytes(D, F_SHARED) + D * 2 + 4 * F_SHARED * 2 + D * 2
LM_HEAD_BYTES = int4_matrix_bytes(VOCAB, D) + D * 2 + 4


# (blocks, threads per block) of the decode step's three launches at the production shape: one block per router row, one wave
# per two-row gate/up tile, eleven down rows per block of eight waves
STEP_GRID_SHAPES = ((E, 256), (TOPK * (F_MOE // 2) // 4, 256), (D // 11, 512))


def expert_layout():
    """Byte offsets of the nine sub-tensors in one routed-expert blob, in the reference's order
    (gate W,S,B, up W,S,B, down W,S,B) with the stride rounded to 16 KiB."""
    offs, pos = [], 0
    for rows, cols in ((F_MOE, D), (F_MOE, D), (D, F_MOE)):
        for nbytes in (rows * cols // 2, rows * (cols // 64) * 2, rows * (cols // 64) * 2):
            offs.append(pos)
            pos += nbytes
    stride = (pos + 16383) // 16384 * 16384
    return offs, pos, stride


def bf16_bits_cuda(t):
    import torch
    return t.to(torch.bfloat16).view(torch.int16)


# ---- the reference's seeded streams (Sources/TurboFieldfareValidation/Support/PRNG/SplitMix64.swift:11-23, SeedTree.swift:12-19),
# evaluated in counter form on the device: draw number i (from 1) of a stream with seed s is mix(s + i * GAMMA), so a whole
# tensor is drawn at once and equals the sequential generator draw for draw.
_M64 = (1 << 64) - 1


def _s64(v):
    """A 64-bit pattern as the signed value torch.int64 holds."""
    v &= _M64
    return v - (1 << 64) if v >= (1 << 63) else v


def seed_tree_key(root, label):
    """SeedTree(root).key(label): the SplitMix64 seed root ^ FNV-1a(label)."""
    h = 0xCBF29CE484222325
    for byte in label.encode("utf-8"):
        h = ((h ^ byte) * 0x100000001B3) & _M64
    return (root ^ h) & _M64


def _lsr(z, k):
    return (z >> k) & ((1 << (64 - k)) - 1)


def splitmix64_draws(torch, seed, first, count, device="cuda"):
    """Draws first+1 ... first+count of SplitMix64(seed) as the int64 bit patterns of the UInt64 values."""
    i = torch.arange(first + 1, first + count + 1, dtype=torch.int64, device=device)
    z = i * _s64(0x9E3779B97F4A7C15) + _s64(seed)                 # two's-complement wrap = the reference's &+ / &*
    z = (z ^ _lsr(z, 30)) * _s64(0xBF58476D1CE4E5B9)
    z = (z ^ _lsr(z, 27)) * _s64(0x94D049BB133111EB)
    return z ^ _lsr(z, 31)


def splitmix64_uniform(torch, seed, first, count, lo, hi, device="cuda"):
    """SplitMix64.uniform(lo, hi) for draws first+1 ... first+count: lo + (hi - lo) * Float(next >> 40) / 2^24 in fp32."""
    u = _lsr(splitmix64_draws(torch, seed, first, count, device), 40).to(torch.float32) / 16777216.0
    lo32 = np.float32(lo)
    return float(np.float32(hi) - lo32) * u + float(lo32)          # (hi - lo) formed in fp32, as the reference's Float arithmetic does


def splitmix64_nibble_bytes(torch, seed, nbytes, device="cuda", chunk=1 << 25):
    """nbytes packed int4 bytes: nibble j = next() & 0xF, low nibble first (byte b = draws 2b+1 and 2b+2)."""
    out = torch.empty(nbytes, dtype=torch.uint8, device=device)
    for b0 in range(0, nbytes, chunk):
        n = min(chunk, nbytes - b0)
        nib = (splitmix64_draws(torch, seed, 2 * b0, 2 * n, device) & 0xF).view(n, 2)
        out[b0:b0 + n] = (nib[:, 0] | (nib[:, 1] << 4)).to(torch.uint8)
    return out


def splitmix64_normal_f16(torch, seed, count, device="cuda"):
    """count N(0,1) values by Box-Muller on `uniform`: value j = sqrt(-2 ln(1 - u1)) cos(2 pi u2) with (u1, u2) = draws 2j+1, 2j+2
    of uniform(0, 1); rounded to fp16."""
    u = splitmix64_uniform(torch, seed, 0, 2 * count, 0.0, 1.0, device).view(count, 2)
    r = torch.sqrt(-2.0 * torch.log1p(-u[:, 0]))
    return (r * torch.cos(6.283185307179586 * u[:, 1])).to(torch.float16)


BENCH_ROOT_SEED = 0x7F1E1DFA      # SeedTree root of every stream below


def make_layer_seeded(torch, layer, offs, stride):
    """One layer's resident weights drawn as the measurement plan of the reference-side survey states: uniform nibbles
    (next() & 0xF, low nibble first), scale ~U(0.005, 0.02) and bias ~U(-0.1, 0.1) rounded to bf16, every tensor from a
    SeedTree stream of its own label.  Router: 8-bit weights (next() & 0xFF), scale ~U(0.0002, 0.0008), bias ~U(-0.1, 0)."""
    key = lambda what: seed_tree_key(BENCH_ROOT_SEED, f"bench-layer{layer}-{what}")
    pool = splitmix64_nibble_bytes(torch, key("expert-nibbles"), E * stride).view(E, stride)
    shapes = ((F_MOE, D), (F_MOE, D), (D, F_MOE))
    for p, (rows, cols) in enumerate(shapes):
        n = rows * (cols // 64)
        for j, (what, lo, hi) in ((1, ("scales", 0.005, 0.02)), (2, ("biases", -0.1, 0.1))):
            vals = splitmix64_uniform(torch, key(f"{('gate', 'up', 'down')[p]}-{what}"), 0, E * n, lo, hi).view(E, n)
            o = offs[3 * p + j]
            pool[:, o:o + 2 * n] = bf16_bits_cuda(vals).view(torch.uint8).view(E, 2 * n)
    uni = lambda what, n, lo, hi: splitmix64_uniform(torch, key(what), 0, n, lo, hi)
    router = dict(
        W=(splitmix64_draws(torch, key("router-weights"), 0, E * D) & 0xFF).to(torch.uint8).view(E, D),
        S=bf16_bits_cuda(uni("router-scales", E * (D // 64), 0.0002, 0.0008).view(E, D // 64)),
        B=bf16_bits_cuda(uni("router-biases", E * (D // 64), -0.1, 0.0).view(E, D // 64)),
        eff=bf16_bits_cuda(uni("router-effective-scale", D, 0.5, 1.5) / (D ** 0.5)),
        gain=bf16_bits_cuda(uni("router-per-expert-scale", E, 0.6, 1.4)),
    )
    return pool, router


def make_int4(torch, gen, rows, cols):
    W = torch.randint(0, 256, (rows, cols // 2), dtype=torch.uint8, device="cuda", generator=gen)
    S = bf16_bits_cuda(torch.rand((rows, cols // 64), device="cuda", generator=gen) * 0.015 + 0.005)
    B = bf16_bits_cuda(torch.rand((rows, cols // 64), device="cuda", generator=gen) * 0.2 - 0.1)
    return W, S, B


def calibration_copy(torch):
    """One plain 1 GiB device-to-device copy: a launch of known size to scale hardware byte counters by."""
    src = torch.zeros(1 << 30, dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    dst.copy_(src)
    torch.cuda.synchronize()
    del src, dst


def profiler_attached():
    """True when a rocprofiler tool library rides in this process (rocprofv3 preloads it and names it in the environment)."""
    env = " ".join(os.environ.get(v, "") for v in ("LD_PRELOAD", "ROCP_TOOL_LIBRARIES", "ROCPROFILER_REGISTER_FORCE_LOAD", "ROCPROF_OUTPUT_PATH"))
    if "rocprof" in env.lower():
        return True
    try:
        with open("/proc/self/maps") as f:
            return any("rocprofiler-sdk-tool" in line or "librocprofiler" in line for line in f)
    except OSError:
        return False


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=640)
    ap.add_argument("--warmup", type=int, default=64)
    ap.add_argument("--layers", type=int, default=4, help="layer replicas the steps rotate through")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="skip lm_head / GEMV / shared-expert side measurements")
    ap.add_argument("--no-layer-chain", action="store_true", help="skip the whole-decoder-layer graph")
    ap.add_argument("--layer-chain-fork", action="store_true",
                    help="also replay the layer chain with the shared expert on a second captured stream (a graph that forks and joins; "
                         "not part of the default run; refused under a profiler)")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="also run one plain 1 GiB device copy (a known-size reference for hardware byte counters)")
    ap.add_argument("--only-decode-step", action="store_true",
                    help="run nothing but the headline decode-step measurement (graph-replayed steps and the one- and two-stage chains) and "
                         "print its JSON: the short program a profiler attributes the step's three kernels with")
    ap.add_argument("--chain-launches", type=int, default=64,
                    help="launches per graph of the one-, two- and three-stage chains (a counter-collecting profiler serialises every "
                         "dispatch: give it short chains and few --steps)")
    ap.add_argument("--only-lm-head", action="store_true",
                    help="run nothing but the lm_head measurements (configs[2]) and print their JSON")
    ap.add_argument("--only-small-m", type=int, nargs="+", metavar="M",
                    help="run nothing but the few-token routed-MoE measurement at these token counts and print its JSON "
                         "(a short program whose launches a profiler can attribute to one size)")
    ap.add_argument("--prefill-balanced", action="store_true",
                    help="with --only-prefill-2048: every expert gets exactly 128 of the 16384 pairs instead of the Zipf(1.1) draw "
                         "(all row tiles full: the grouped kernels' rate without the skew)")
    ap.add_argument("--only-prefill-2048", action="store_true",
                    help="run nothing but the 2048-token prefill measurement (configs[4]) and print its JSON")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        sys.exit(2)
    sub_command = bool(args.only_decode_step or args.only_lm_head or args.only_small_m or args.only_prefill_2048)
    if profiler_attached() and (not sub_command or args.layer_chain_fork):
        # The all-sections run ended the GPU box twice under `rocprofv3 --kernel-trace --stats` (no output came back either time)
        # and the cause has not been shown; the --only-* sub-commands run the same measurements one at a time and profile fine.
        print("bench.py: refusing to run every section (or --layer-chain-fork) with a profiler attached; profile one of "
              "--only-decode-step, --only-lm-head, --only-small-m M, --only-prefill-2048 instead", file=sys.stderr)
        sys.exit(2)

    import torch
    tfk = importlib.import_module("turbo-fieldfare_amd")
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    k = tfk.Context(0)
    gen = torch.Generator(device="cuda")       # side measurements (extras) draw from torch's generator
    gen.manual_seed(0x7F1E1DFA)
    offs, payload, stride = expert_layout()
    off = tfk.ExpertOffsets(*offs)
    global TIMING_STREAM
    side = torch.cuda.Stream()            # default priority; everything timed is recorded on it
    TIMING_STREAM = side
    lib, h = k.lib, k.handle
    if args.only_lm_head:
        note("lm_head only")
        print(json.dumps(head_extras(torch, tfk, k, gen, lib, h, side.cuda_stream)))
        return
    note("resident weights: SplitMix64 / SeedTree streams")
    n_layers = 1 if (args.only_small_m or args.only_prefill_2048) else args.layers
    layers = [make_layer_seeded(torch, li, offs, stride) for li in range(n_layers)]
    if args.only_small_m or args.only_prefill_2048:
        only = multi_token_extras(torch, tfk, k, gen, k.lib, k.handle, side.cuda_stream, layers[0], offs, stride,
                                  small_sizes=tuple(args.only_small_m or ()), small_only=not args.only_prefill_2048,
                                  prefill_only=bool(args.only_prefill_2048), balanced=bool(args.prefill_balanced))
        print(json.dumps(only))
        return
    n_hidden = 64
    hidden = splitmix64_normal_f16(torch, seed_tree_key(BENCH_ROOT_SEED, "bench-hidden-states"), n_hidden * D).view(n_hidden, D)
    idx = torch.zeros((n_hidden, TOPK), dtype=torch.int32, device="cuda")
    wts = torch.zeros((n_hidden, TOPK), dtype=torch.float16, device="cuda")
    acts = torch.zeros(TOPK * F_MOE, dtype=torch.float16, device="cuda")
    residual = torch.zeros(D, dtype=torch.float16, device="cuda")
    y = torch.zeros((n_hidden, D), dtype=torch.float16, device="cuda")

    import ctypes as C

    def step_args(i, stream):
        li, hi = i % args.layers, i % n_hidden
        pool, r = layers[li]
        hp = hidden.data_ptr() + hi * D * 2
        ip, wp = idx.data_ptr() + hi * TOPK * 4, wts.data_ptr() + hi * TOPK * 2
        return (h, stream, r["W"].data_ptr(), 0, r["S"].data_ptr(), 0, r["B"].data_ptr(), 0, hp, r["eff"].data_ptr(), 0, r["gain"].data_ptr(), 0,
                pool.data_ptr(), stride, E, C.byref(off), hp, acts.data_ptr(), residual.data_ptr(), y.data_ptr() + hi * D * 2, ip, wp, D, F_MOE,
                TOPK, tfk.TF_BF16)

    def step(i, stream):
        # one call = router logits -> (top-8 + gate/up/GeGLU of the 8 chosen experts) -> down + weighted sum + residual
        if lib.tf_moe_decode_step(*step_args(i, stream)) != 0:
            raise RuntimeError("kernel call failed: " + k.last_error())

    def run_steps(first, count, stream):
        for j in range(count):
            step(first + j, stream)

    # ---- the decode loop is launch-bound on the host (3 short kernels per step), so the steps are captured once
    # into HIP graphs and replayed: `graph_steps` steps per graph, plus one remainder graph, exactly `steps` in all.
    # One ROUND = exactly `steps` steps; rounds repeat until MIN_TIMED_MS of device time have passed (with the driver's
    # --steps 20 a single round lasts 0.3 ms, far too short a sample) and the median round is reported.
    note("decode step: warm-up, graph capture, timed rounds")
    graph_steps = min(64, args.steps)
    n_full, rem = divmod(args.steps, graph_steps)
    graphs = {}
    with torch.cuda.stream(side):
        run_steps(0, args.warmup, side.cuda_stream)   # untimed warm-up (eager)
        side.synchronize()
        for count in {graph_steps, rem} - {0}:
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                run_steps(0, count, side.cuda_stream)
            graphs[count] = g
        graphs[graph_steps].replay()      # one untimed replay
        side.synchronize()

    def one_round():
        for _ in range(n_full):
            graphs[graph_steps].replay()
        if rem:
            graphs[rem].replay()
    rounds_ms, wall_ms = replay_rounds(torch, side, one_round)
    ms_graph = float(np.median(rounds_ms)) / args.steps
    stream = side.cuda_stream
    # The same rounds launched call by call.  A graph launch costs the device about 12 us before its first kernel runs (0.6 us a
    # step in a round of 20); three launches a step are within what the host sustains (3 us a launch against 4.6 us of device
    # time), so a round of few steps is the faster for being launched eagerly.  Both medians are printed; the round a caller
    # would choose - the faster one - is the headline, and `launch` says which it is.
    note("decode step: timed rounds, eager launches")
    eager_ms, eager_wall_ms = replay_rounds(torch, side, lambda: run_steps(0, args.steps, stream))
    ms_eager = float(np.median(eager_ms)) / args.steps
    if ms_eager < ms_graph:
        ms_per_step, ms_per_step_wall, n_rounds = ms_eager, eager_wall_ms / (len(eager_ms) * args.steps), len(eager_ms)
        launch_how = f"eager launches (3 per step); {n_rounds} rounds of {args.steps} steps, median round reported"
    else:
        ms_per_step, ms_per_step_wall, n_rounds = ms_graph, wall_ms / (len(rounds_ms) * args.steps), len(rounds_ms)
        launch_how = f"HIP graph replay, {graph_steps} steps per graph; {n_rounds} rounds of {args.steps} steps, median round reported"
    value = STEP_BYTES / (ms_per_step * 1e-3) / 1e9

    # ---- each kernel's share of the step: the step's first launch alone and its first two launches, replayed as chains of 64
    # like the step itself (same operands, same rotation).  Launches on one stream run one after the other, so
    # router = chain of 1, phase 1 = chain of 2 - chain of 1, phase 2 = chain of 3 - chain of 2; each share includes the boundary
    # to the launch before it.  No events sit between the kernels.
    note("decode step: one- and two-stage chains")

    def stages(n_stages):
        def fn(i):
            if lib.tf_bench_moe_decode_step_stages(*step_args(i, stream), n_stages) != 0:
                raise RuntimeError("kernel call failed: " + k.last_error())
        return fn
    us_chain = {n: time_loop(torch, stages(n), args.chain_launches) for n in (1, 2, 3)}
    t_router, t_p1 = us_chain[1], us_chain[2] - us_chain[1]
    t_p2 = us_chain[3] - us_chain[2]
    p1_gbps = PHASE1_BYTES / (t_p1 * 1e-6) / 1e9

    out = {
        "metric": "int4 MoE decode GEMV GB/s (% HBM peak) + batch-1 decode step/s; prefill tok/s",
        "value": round(value, 2), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int4 weights x fp16 activations, fp32 accumulate", "data": "synthetic",
        "config": {"workload": "configs[1]: routed MoE FFN decode step, batch 1, hidden 2816, int8 router 128x2816 + top-8, "
                               "8 of 128 int4 g64 experts (gate/up 704x2816, down 2816x704), GeGLU, weighted sum",
                   "layer_replicas": args.layers, "resident_expert_bytes": args.layers * E * stride,
                   "algorithmic_bytes_per_step": STEP_BYTES,
                   "inputs": "every tensor of the headline workload (expert pools, routers, hidden states) from SplitMix64 streams keyed by "
                             f"SeedTree({BENCH_ROOT_SEED:#x}) labels: nibbles next() & 0xF low first, scale ~U(0.005,0.02), bias ~U(-0.1,0.1) as bf16, "
                             "activations N(0,1) by Box-Muller as fp16; the side measurements in `extras` draw from torch's generator"},
        "roofline": {"bound": "hbm", "kernel": "phase1_long_kernel<2,3,bf16,fused top-8> (expert selection + gate/up/GeGLU of 8 experts)",
                     "achieved": round(p1_gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(p1_gbps / HBM_PEAK_GBPS, 4), "traffic": PHASE1_TRAFFIC_BYTES,
                     "traffic_from": PHASE1_TRAFFIC_FROM,
                     "algorithmic_bytes_per_launch": PHASE1_BYTES, "avg_launch_us": round(t_p1, 3),
                     "duration_from": "HIP events around graph replays on the launch stream: (chain of the step's first two launches) - (chain of "
                                      "its first launch), 64 launches per graph, >= 50 ms per figure; includes the boundary to the router launch, so "
                                      "the kernel's own duration in a profiler's trace is shorter by about that boundary",
                     },
        "launch": launch_how,
        "ms_per_step_graph_rounds": round(ms_graph, 6), "ms_per_step_eager_rounds": round(ms_eager, 6),
        "ms_per_step_wallclock_all_rounds": round(ms_per_step_wall, 6),
        "step_per_s": round(1e3 / ms_per_step, 1),
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "kernels_us": {"router": round(t_router, 3), "phase1": round(t_p1, 3), "phase2": round(t_p2, 3),
                       "how": "chains of the step's first 1, 2 and 3 launches replayed from graphs; differences of their times",
                       "chain_us": {str(n): round(v, 3) for n, v in us_chain.items()},
                       "phase1_GBps": round(p1_gbps, 1), "phase2_GBps": round(PHASE2_BYTES / (t_p2 * 1e-6) / 1e9, 1)},
    }
    if args.only_decode_step:
        if args.calibration_copy:
            calibration_copy(torch)
        print(json.dumps(out))
        return

    # the same loop launched call by call (no graph): what a host that encodes every step itself would see
    note("decode step: eager launches")
    with torch.cuda.stream(side):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        run_steps(args.warmup, max(args.steps, 256), stream)
        torch.cuda.synchronize()
        out["ms_per_step_eager_launch"] = round((time.perf_counter() - t0) * 1e3 / max(args.steps, 256), 6)

    # ---- latency floor of the step: three dependent launches of the step's grid shapes that move no data, plus the step's
    # bytes at the rate a plain streaming read reaches in this run.  The step cannot go below that with three launches.
    note("latency floor: empty launch chain, streaming read")
    words = torch.zeros(8, dtype=torch.int32, device="cuda")
    wp0 = words.data_ptr()
    shapes = STEP_GRID_SHAPES

    def empty_chain(i):
        rc = 0
        for j, (blocks, threads) in enumerate(shapes):
            rc |= lib.tf_bench_empty_launch(h, stream, blocks, threads, wp0 + 4 * j, wp0 + 4 * ((j + 1) % 3))
        assert rc == 0, k.last_error()
    empty_chain_us = time_loop(torch, empty_chain, 64)
    read_bufs = [torch.randint(0, 256, (400 << 20,), dtype=torch.uint8, device="cuda", generator=gen) for _ in range(2)]

    def stream_read(i):
        assert lib.tf_bench_stream_read(h, stream, read_bufs[i % 2].data_ptr(), 400 << 20, wp0 + 16) == 0, k.last_error()
    read_us = time_loop(torch, stream_read, 10)
    read_gbps = (400 << 20) / (read_us * 1e-6) / 1e9
    del read_bufs
    latency_floor_us = empty_chain_us + STEP_BYTES / (read_gbps * 1e9) * 1e6
    out["roofline"]["latency_floor_us"] = round(latency_floor_us, 3)
    out["roofline"]["latency_floor"] = {"what": "three dependent launches of the step's grid shapes that move no data + the step's "
                                                "algorithmic bytes at the plain streaming-read rate, both measured in this run",
                                        "empty_three_launch_chain_us": round(empty_chain_us, 3),
                                        "stream_read_GBps": round(read_gbps, 1), "stream_read_frac_of_peak": round(read_gbps / HBM_PEAK_GBPS, 4),
                                        "step_us": round(ms_per_step * 1e3, 3),
                                        "step_over_floor": round(ms_per_step * 1e3 / latency_floor_us, 3)}

    if args.calibration_copy:
        calibration_copy(torch)
    if not args.no_extras:
        note("extras: lm_head, GEMV, attention, shared expert")
        out["extras"] = head_extras(torch, tfk, k, gen, lib, h, stream)
        out["extras"].update(extras(torch, tfk, k, gen, lib, h, stream))
        note("extras: small-M verification sizes, 2048-token prefill")
        out["extras"].update(multi_token_extras(torch, tfk, k, gen, lib, h, stream, layers[0], offs, stride))
        if not args.no_layer_chain:
            note("extras: whole decoder layer chain")
            out["extras"].update(layer_chain_extra(torch, tfk, k, gen, lib, h, layers, offs, stride, fork=args.layer_chain_fork))

    if not args.no_cpu:
        note("CPU baseline legs")
        out["cpu_baseline"] = cpu_baseline(torch, layers, hidden, idx, wts, y, offs, stride, payload, args)
        if not args.no_extras:
            cpu_extras(torch, gen, out["extras"], layers[0], offs, stride, payload)
    print(json.dumps(out))


MIN_TIMED_MS = 50.0     # every figure comes from at least this much device time


def note(section):
    """Names the section that is about to use the GPU, on stderr and flushed: the last line seen names the case if a run dies."""
    print(f"[bench] {section}", file=sys.stderr, flush=True)


def replay_rounds(torch, side, replay_once, min_ms=MIN_TIMED_MS, min_rounds=5, max_rounds=4000):
    """Replays `replay_once()` (graph launches on `side`) round after round until `min_ms` of device time have gone by;
    every round is bracketed by events on that stream.  Returns (per-round ms list, wall-clock ms over all rounds between
    two synchronisations)."""
    events = []
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    with torch.cuda.stream(side):
        while True:
            batch = []
            for _ in range(min_rounds):
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record(side)
                replay_once()
                e1.record(side)
                batch.append((e0, e1))
            events += batch
            side.synchronize()
            if (time.perf_counter() - t0) * 1e3 >= min_ms or len(events) >= max_rounds:
                break
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return [a.elapsed_time(b) for a, b in events], wall_ms


def time_loop(torch, fn, iters, warmup=3, side=None):
    """Median device time of one call of fn, in microseconds: `iters` consecutive calls (fn(0) ... fn(iters-1), so that
    rotating operands rotate) are recorded into a HIP graph once and the graph is replayed until MIN_TIMED_MS have passed.
    The host only launches graphs, so its jitter stays out of the figure."""
    side = side or TIMING_STREAM
    with torch.cuda.stream(side):
        for i in range(warmup):
            fn(i)
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for i in range(iters):
                fn(i)
        g.replay()
        side.synchronize()
    rounds, _ = replay_rounds(torch, side, g.replay)
    return float(np.median(rounds)) * 1e3 / iters


TIMING_STREAM = None     # the side stream every measurement records on (set in main)


def head_extras(torch, tfk, k, gen, lib, h, stream):
    """configs[2]: the int4 lm_head, greedy and with fp32 logits."""
    res = {}
    # configs[2]: int4 lm_head 262144 x 2816 -> greedy argmax; two replicas alternate (830 MB > Infinity Cache)
    heads = [make_int4(torch, gen, VOCAB, D) for _ in range(2)]
    hid = torch.randn((8, D), device="cuda", generator=gen).to(torch.float16)
    norm_w = bf16_bits_cuda(torch.rand(D, device="cuda", generator=gen) + 0.5)
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")

    def head(i):
        W, S, B = heads[i % 2]
        rc = lib.tf_lm_head_greedy_int4(h, stream, hid.data_ptr(), (i % 8) * D * 2, norm_w.data_ptr(), 0, W.data_ptr(), 0,
                                        S.data_ptr(), 0, B.data_ptr(), 0, tok.data_ptr(), D, VOCAB, 1e-6, tfk.TF_BF16)
        assert rc == 0, k.last_error()
    us = time_loop(torch, head, 30)
    res["lm_head_greedy"] = {"workload": "configs[2]: int4 lm_head 262144x2816 -> argmax (rmsnorm + rows + reduce)",
                             "us_per_call": round(us, 2), "GBps": round(LM_HEAD_BYTES / (us * 1e-6) / 1e9, 1),
                             "frac_hbm_peak": round(LM_HEAD_BYTES / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                             "algorithmic_bytes": LM_HEAD_BYTES}
    logits = torch.zeros(VOCAB, dtype=torch.float32, device="cuda")

    def head_logits(i):
        W, S, B = heads[i % 2]
        rc = lib.tf_lm_head_logits_int4(h, stream, hid.data_ptr(), (i % 8) * D * 2, norm_w.data_ptr(), 0, W.data_ptr(), 0,
                                        S.data_ptr(), 0, B.data_ptr(), 0, logits.data_ptr(), 0, D, VOCAB, 1e-6, tfk.TF_BF16, tfk.TF_FP32)
        assert rc == 0, k.last_error()
    us = time_loop(torch, head_logits, 30)
    nbytes = LM_HEAD_BYTES + VOCAB * 4
    res["lm_head_logits_fp32"] = {"us_per_call": round(us, 2), "GBps": round(nbytes / (us * 1e-6) / 1e9, 1),
                                  "frac_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4)}
    del heads
    return res


def extras(torch, tfk, k, gen, lib, h, stream):
    """Side measurements on the other single-GPU configurations (not the headline value)."""
    res = {}
    # configs[0]: int4 GEMV 2112 x 2816, rotating over 192 replicas (644 MB)
    reps = 192
    W, S, B = make_int4(torch, gen, reps * F_SHARED, D)
    xs = torch.randn((8, D), device="cuda", generator=gen).to(torch.float16)
    yv = torch.zeros(F_SHARED, dtype=torch.float16, device="cuda")
    row_w, row_s = D // 2, (D // 64) * 2

    def gemv(i):
        r = (i % reps) * F_SHARED
        rc = lib.tf_dequant_int4_gemv(h, stream, W.data_ptr(), r * row_w, S.data_ptr(), r * row_s, B.data_ptr(), r * row_s,
                                      xs.data_ptr(), (i % 8) * D * 2, yv.data_ptr(), 0, F_SHARED, D, tfk.TF_BF16, tfk.TF_FP16)
        assert rc == 0, k.last_error()
    us = time_loop(torch, gemv, 400, warmup=20)
    nbytes = int4_matrix_bytes(F_SHARED, D) + D * 2 + F_SHARED * 2
    res["gemv_2112x2816"] = {"workload": "configs[0]: int4 g64 GEMV 2112x2816, batch 1", "us_per_call": round(us, 3),
                             "GBps": round(nbytes / (us * 1e-6) / 1e9, 1), "algorithmic_bytes": nbytes,
                             "note": "3.3 MB per call: at 8 TB/s the bytes take 0.4 us, the rest is one launch and one memory round trip; "
                                     "a latency figure, not an HBM-bandwidth measurement (configs[2] is the bandwidth-sized GEMV)"}

    # q / k / v projections of one token in one launch (4096 + 2 x 2048 rows of 2816), rotating over the same 644 MB
    q_rows, kv_rows = 4096, 2048
    span = q_rows + 2 * kv_rows
    qkv_reps = (reps * F_SHARED) // span
    qo, ko, vo = (torch.zeros(r, dtype=torch.float16, device="cuda") for r in (q_rows, kv_rows, kv_rows))

    def qkv(i):
        r = (i % qkv_reps) * span
        args = []
        for first in (r, r + q_rows, r + q_rows + kv_rows):
            args += [W.data_ptr(), first * row_w, S.data_ptr(), first * row_s, B.data_ptr(), first * row_s]
        rc = lib.tf_fused_qkv_gemv(h, stream, *args, xs.data_ptr() + (i % 8) * D * 2, qo.data_ptr(), 0, ko.data_ptr(), 0, vo.data_ptr(), 0,
                                   q_rows, kv_rows, D, tfk.TF_BF16)
        assert rc == 0, k.last_error()
    us = time_loop(torch, qkv, 200, warmup=20)
    nbytes = int4_matrix_bytes(span, D) + D * 2 + span * 2
    res["fused_qkv_gemv_8192x2816"] = {"us_per_call": round(us, 3), "GBps": round(nbytes / (us * 1e-6) / 1e9, 1),
                                       "frac_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes}

    # decode attention over an fp16 KV cache: a global layer (16 query heads on 2 kv heads, head_dim 512) at 32768 positions and a
    # sliding-window layer (16 on 8, head_dim 256, window 1024); three caches each, rotated, so the rows come from HBM
    attn = {}
    for name, hd, nq, nkv, seq, window in (("full_16q_2kv_d512_T32768", 512, 16, 2, 32768, None), ("swa_16q_8kv_d256_w1024", 256, 16, 8, 4096, 1024)):
        caches = [(torch.randn((seq, nkv, hd), device="cuda", generator=gen).to(torch.float16) * 0.3,
                   torch.randn((seq, nkv, hd), device="cuda", generator=gen).to(torch.float16)) for _ in range(3)]
        qv = torch.randn((nq, hd), device="cuda", generator=gen).to(torch.float16) * 0.3
        ov = torch.zeros((nq, hd), dtype=torch.float16, device="cuda")

        def attend(i):
            kc, vc = caches[i % 3]
            if window is None:
                k.attention_full(qv, kc, vc, ov, hd, nq, nkv, seq, 1.0)
            else:
                k.attention_swa(qv, kc, vc, ov, hd, nq, nkv, seq, window, 1.0)
        us = time_loop(torch, attend, 100, warmup=10)
        rows = seq if window is None else min(seq, window)
        nbytes = rows * nkv * hd * 2 * 2 + 2 * nq * hd * 2
        attn[name] = {"us_per_call": round(us, 2), "GBps": round(nbytes / (us * 1e-6) / 1e9, 1),
                      "frac_hbm_peak": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4), "algorithmic_bytes": nbytes}
        del caches
    res["decode_attention"] = attn

    # block (prefill) attention: 128 queries appended at position 3968 of a global layer (all keys visible) and of a
    # sliding-window layer (1024 keys each)
    block = {}
    for name, hd, nq, nkv, window in (("full_16q_2kv_d512_128q_at_3968", 512, 16, 2, 0), ("swa_16q_8kv_d256_128q_at_3968_w1024", 256, 16, 8, 1024)):
        start, count = 3968, 128
        kc = torch.randn((start + count, nkv, hd), device="cuda", generator=gen).to(torch.float16) * 0.3
        vc = torch.randn((start + count, nkv, hd), device="cuda", generator=gen).to(torch.float16)
        qv = torch.randn((count, nq, hd), device="cuda", generator=gen).to(torch.float16) * 0.3
        ov = torch.zeros((count, nq, hd), dtype=torch.float16, device="cuda")
        prm = tfk.PrefillAttentionParams(start, count, hd, nq, nkv, start + count, window, nkv * hd, nq * hd, nq * hd, 1.0)
        import ctypes as C

        def attend_block(i):
            rc = lib.tf_prefill_attention_causal(h, stream, qv.data_ptr(), 0, kc.data_ptr(), 0, vc.data_ptr(), 0, ov.data_ptr(), 0, C.byref(prm), 0)
            assert rc == 0, k.last_error()
        us = time_loop(torch, attend_block, 30, warmup=3)
        keys = sum(min(start + t + 1, window) if window else start + t + 1 for t in range(count))
        flop = 4.0 * keys * nq * hd
        block[name] = {"us_per_call": round(us, 2), "TFLOPs": round(flop / (us * 1e-6) / 1e12, 2), "queries_per_s": round(count / (us * 1e-6), 1)}
    res["prefill_attention"] = block

    # shared expert chain (gate/up 2112x2816 fused + GeGLU, down 2816x2112), rotating over 64 replicas of each matrix
    sreps = 64
    gu = W[: sreps * 2 * F_SHARED], S[: sreps * 2 * F_SHARED], B[: sreps * 2 * F_SHARED]
    dW, dS, dB = make_int4(torch, gen, sreps * D, F_SHARED)
    sg, su, sa = (torch.zeros(F_SHARED, dtype=torch.float16, device="cuda") for _ in range(3))
    ys = torch.zeros(D, dtype=torch.float16, device="cuda")
    import ctypes as C
    drow_w, drow_s = F_SHARED // 2, (F_SHARED // 64) * 2

    def shared(i):
        r = (i % sreps) * 2 * F_SHARED
        g = tfk.Projection(gu[0].data_ptr(), r * row_w, gu[1].data_ptr(), r * row_s, gu[2].data_ptr(), r * row_s, F_SHARED, D)
        u = tfk.Projection(gu[0].data_ptr(), (r + F_SHARED) * row_w, gu[1].data_ptr(), (r + F_SHARED) * row_s, gu[2].data_ptr(),
                           (r + F_SHARED) * row_s, F_SHARED, D)
        dr = (i % sreps) * D
        dn = tfk.Projection(dW.data_ptr(), dr * drow_w, dS.data_ptr(), dr * drow_s, dB.data_ptr(), dr * drow_s, D, F_SHARED)
        rc = lib.tf_shared_expert_int4(h, stream, xs.data_ptr(), (i % 8) * D * 2, 8 * D * 2, C.byref(g), C.byref(u), C.byref(dn),
                                       ys.data_ptr(), 0, D * 2, sg.data_ptr(), 0, F_SHARED * 2, su.data_ptr(), 0, F_SHARED * 2,
                                       sa.data_ptr(), 0, F_SHARED * 2, 4, tfk.TF_BF16)
        assert rc == 0, k.last_error()
    us = time_loop(torch, shared, 300, warmup=20)
    res["shared_expert_int4"] = {"us_per_call": round(us, 3), "GBps": round(SHARED_BYTES / (us * 1e-6) / 1e9, 1),
                                 "algorithmic_bytes": SHARED_BYTES}

    # the same chain with 8-bit projections (one byte per weight), rotating over 32 replicas of each matrix
    r8 = 32
    def int8_matrix(rows, cols):
        return (torch.randint(0, 256, (rows, cols), dtype=torch.uint8, device="cuda", generator=gen),
                bf16_bits_cuda(torch.rand((rows, cols // 64), device="cuda", generator=gen) * 0.0012 + 0.0004),
                bf16_bits_cuda(torch.rand((rows, cols // 64), device="cuda", generator=gen) * 0.2 - 0.2))
    g8, u8, d8 = int8_matrix(r8 * F_SHARED, D), int8_matrix(r8 * F_SHARED, D), int8_matrix(r8 * D, F_SHARED)

    def shared8(i):
        r = i % r8
        def proj(m, first, rows, cols):
            return tfk.Projection(m[0].data_ptr(), first * cols, m[1].data_ptr(), first * (cols // 64) * 2, m[2].data_ptr(), first * (cols // 64) * 2,
                                  rows, cols)
        g, u, dn = proj(g8, r * F_SHARED, F_SHARED, D), proj(u8, r * F_SHARED, F_SHARED, D), proj(d8, r * D, D, F_SHARED)
        rc = lib.tf_shared_expert_int8(h, stream, xs.data_ptr(), (i % 8) * D * 2, 8 * D * 2, C.byref(g), C.byref(u), C.byref(dn), ys.data_ptr(), 0,
                                       D * 2, sa.data_ptr(), 0, F_SHARED * 2, tfk.TF_BF16)
        assert rc == 0, k.last_error()
    us = time_loop(torch, shared8, 200, warmup=20)
    bytes8 = 3 * (F_SHARED * D + 2 * F_SHARED * (D // 64) * 2) + 2 * D * 2 + 2 * F_SHARED * 2
    res["shared_expert_int8"] = {"us_per_call": round(us, 3), "GBps": round(bytes8 / (us * 1e-6) / 1e9, 1), "algorithmic_bytes": bytes8}
    return res


def layer_chain_extra(torch, tfk, k, gen, lib, h, layers, offs, stride, fork=False):
    """One token through whole sliding-window decoder layers, every stage a call of the library and nothing on the host in
    between, eight launches a layer: [previous layer's tail + input norm + q/k/v projections, k and v straight into their cache
    row] -> per-head norm + RoPE -> attention over a 1024-row window (two launches) -> output projection -> [post-attention
    setup + router logits + shared gate / up] -> [top-8 + routed phase 1 + shared down] -> routed phase 2.  The layers rotate
    over the resident expert pools and as many sets of dense weights; replayed from a HIP graph."""
    import ctypes as C
    HD, NQ, NKV, WINDOW = 256, 16, 8, 1024
    n_layers = len(layers)
    off = tfk.ExpertOffsets(*offs)
    def centered_int4(rows, cols):
        # zero-mean weights (bias = -7.5 scale): a token must survive 30 synthetic layers without leaving fp16's range
        W, S, _ = make_int4(torch, gen, rows, cols)
        return W, S, bf16_bits_cuda(S.view(torch.bfloat16).float() * -7.5)
    dense = []
    for _ in range(n_layers):
        w = {name: centered_int4(rows, cols) for name, rows, cols in (("q", NQ * HD, D), ("k", NKV * HD, D), ("v", NKV * HD, D), ("o", D, NQ * HD),
                                                                      ("gate", F_SHARED, D), ("up", F_SHARED, D), ("down", D, F_SHARED))}
        # What a branch adds to the residual stream goes through a norm whose weights are small and of random sign: the routed
        # experts of the resident pools have a positive mean, so their output has one common sign, and fed back through 30
        # synthetic layers that common component would grow until gate x up leaves fp16's range.
        for name, n, lo, span, signed in (("input_norm", D, 0.9, 0.2, False), ("pre_ffn", D, 0.9, 0.2, False), ("pre_ffn2", D, 0.9, 0.2, False),
                                          ("q_norm", HD, 0.9, 0.2, False), ("k_norm", HD, 0.9, 0.2, False), ("post_attn", D, 0.05, 0.02, True),
                                          ("post_ffn1", D, 0.05, 0.02, True), ("post_ffn2", D, 0.05, 0.02, True), ("post_ffn", D, 0.05, 0.02, True)):
            vals = torch.rand(n, device="cuda", generator=gen) * span + lo
            if signed:
                vals = vals * (torch.randint(0, 2, (n,), device="cuda", generator=gen).float() * 2.0 - 1.0)
            w[name] = bf16_bits_cuda(vals)
        w["k_cache"] = torch.randn((WINDOW + 128, NKV, HD), device="cuda", generator=gen).to(torch.float16)
        w["v_cache"] = torch.randn((WINDOW + 128, NKV, HD), device="cuda", generator=gen).to(torch.float16)
        w["proj"] = [tfk.projection(*w[n], r, c) for n, r, c in (("gate", F_SHARED, D), ("up", F_SHARED, D), ("down", D, F_SHARED))]
        dense.append(w)
    z = lambda n: torch.zeros(n, dtype=torch.float16, device="cuda")
    b = dict(hidden=(torch.randn(D, device="cuda", generator=gen) * 0.5).to(torch.float16), hidden_alt=z(D), x_norm=z(D), q=z(NQ * HD), attn=z(NQ * HD), o=z(D),
             dense_x=z(D), routed_x=z(D), router_x=z(D), shared=z(D), h1=z(D), h2=z(D), sg=z(F_SHARED), su=z(F_SHARED), sa=z(F_SHARED), zero=z(D),
             acts=z(TOPK * F_MOE), idx=torch.zeros(TOPK, dtype=torch.int32, device="cuda"), wts=z(TOPK))
    p = lambda name: b[name].data_ptr()
    position = WINDOW + 60
    kv_off = position * NKV * HD * 2

    def layer_step(i, st, branch=None, first=True, last=True):
        """One layer on stream handle `st`; first / last: whether the sequence of layers begins / ends with this one.
        The residual stream lives in two buffers: `hidden` (a layer's input) and `hidden_alt` (after the post-attention setup):
        a stage folded into the prologue of every block of another launch cannot write over the row those blocks are reading.
        The layer tail is folded into the NEXT layer's projection launch, so only the last layer of a sequence runs its own
        (in place on `hidden_alt`, where the sequence's output is then found).
        With `branch` (a torch stream) the stages are separate launches, in place on `hidden`, and the shared expert and its
        norm run beside the router and the routed experts, as the reference commits its shared-expert command buffer without
        waiting (RealForwardRunner.swift:1570-1594); the branch forks after the post-attention setup and joins before the tail."""
        w, (pool, r) = dense[i % n_layers], layers[i % n_layers]
        prev = dense[(i - 1) % n_layers]
        ptr = lambda name: w[name].data_ptr()
        qkv = []
        for name in ("q", "k", "v"):
            qkv += [w[name][0].data_ptr(), 0, w[name][1].data_ptr(), 0, w[name][2].data_ptr(), 0]
        qkv_out = (p("q"), 0, ptr("k_cache"), kv_off, ptr("v_cache"), kv_off, NQ * HD, NKV * HD, D, tfk.TF_BF16)
        if first or branch is not None:
            # the input norm runs inside the projection launch
            rc = lib.tf_fused_norm_qkv_gemv(h, st, ptr("input_norm"), 0, 1e-6, *qkv, p("hidden"), *qkv_out)
        else:
            # ... and so does the previous layer's tail (with the norm of the shared expert's output)
            rc = lib.tf_fused_layer_tail_norm_qkv_gemv(h, st, p("h2"), p("shared"), p("hidden_alt"), p("hidden"), prev["post_ffn1"].data_ptr(), 0,
                                                       prev["post_ffn2"].data_ptr(), 0, prev["post_ffn"].data_ptr(), 0, 1e-6, 1.0,
                                                       ptr("input_norm"), 0, 1e-6, *qkv, *qkv_out)
        rc |= lib.tf_fused_qkv_epilogue(h, st, p("q"), 0, ptr("k_cache"), kv_off, ptr("v_cache"), kv_off, ptr("q_norm"), 0, ptr("k_norm"), 0,
                                        HD, NQ, NKV, position, 1e4, HD // 2, 1e-6)
        rc |= lib.tf_attention_swa(h, st, p("q"), 0, ptr("k_cache"), 0, ptr("v_cache"), 0, p("attn"), 0, HD, NQ, NKV, position + 1, WINDOW, 1.0, 0)
        rc |= lib.tf_dequant_int4_gemv(h, st, w["o"][0].data_ptr(), 0, w["o"][1].data_ptr(), 0, w["o"][2].data_ptr(), 0, p("attn"), 0, p("o"), 0,
                                       D, NQ * HD, tfk.TF_BF16, tfk.TF_FP16)
        g, u, dn = w["proj"]
        step = (r["W"].data_ptr(), 0, r["S"].data_ptr(), 0, r["B"].data_ptr(), 0, p("router_x"), r["eff"].data_ptr(), 0, r["gain"].data_ptr(), 0,
                pool.data_ptr(), stride, E, C.byref(off), p("routed_x"), p("acts"), p("zero"), p("h2"), p("idx"), p("wts"), D, F_MOE, TOPK, tfk.TF_BF16)
        if branch is None:
            # post-attention setup, router + routed experts and the shared expert in three launches: the setup in the prologue of the
            # first, the shared expert's gate / up beside the router and its down beside phase 1
            rc |= lib.tf_moe_decode_step_shared_post_attn(h, st, p("hidden"), p("o"), p("hidden_alt"), ptr("post_attn"), 0, ptr("pre_ffn"), 0,
                                                          ptr("pre_ffn2"), 0, 1e-6, *step, p("dense_x"), C.byref(g), C.byref(u), C.byref(dn),
                                                          p("shared"), p("sg"), p("su"), p("sa"))
            if last:
                rc |= lib.tf_fused_layer_tail_shared_norm(h, st, p("h2"), p("shared"), p("hidden_alt"), ptr("post_ffn1"), 0, ptr("post_ffn2"), 0,
                                                          ptr("post_ffn"), 0, D, 1e-6, 1.0)
        else:
            rc |= lib.tf_fused_post_attn_setup(h, st, p("hidden"), p("o"), p("dense_x"), p("routed_x"), p("router_x"), ptr("post_attn"), 0,
                                               ptr("pre_ffn"), 0, ptr("pre_ffn2"), 0, D, 1e-6)
            fork = torch.cuda.Event()
            fork.record(torch.cuda.current_stream())
            branch.wait_event(fork)
            rc |= lib.tf_shared_expert_int4(h, branch.cuda_stream, p("dense_x"), 0, D * 2, C.byref(g), C.byref(u), C.byref(dn), p("shared"), 0, D * 2,
                                            p("sg"), 0, F_SHARED * 2, p("su"), 0, F_SHARED * 2, p("sa"), 0, F_SHARED * 2, 4, tfk.TF_BF16)
            rc |= lib.tf_moe_decode_step(h, st, *step)
            join = torch.cuda.Event()
            join.record(branch)
            torch.cuda.current_stream().wait_event(join)
            rc |= lib.tf_fused_layer_tail_shared_norm(h, st, p("h2"), p("shared"), p("hidden"), ptr("post_ffn1"), 0, ptr("post_ffn2"), 0, ptr("post_ffn"), 0,
                                                      D, 1e-6, 1.0)
        if rc != 0:
            raise RuntimeError("layer chain failed: " + k.last_error())

    per_graph = 30                                          # the model has 30 layers: one replay = one token's layers
    st0 = torch.cuda.current_stream().cuda_stream
    start_hidden = b["hidden"].clone()
    for i in range(2 * n_layers):                           # warm-up; also sizes every context-owned scratch before the capture
        layer_step(i, st0, first=i == 0, last=i == 2 * n_layers - 1)
    b["hidden"].copy_(start_hidden)
    torch.cuda.synchronize()
    side, branch = torch.cuda.Stream(), torch.cuda.Stream()      # both at the default priority
    results = {}
    with torch.cuda.stream(side):
        hidden0 = b["hidden"].clone()
        for label, br in (("serial", None), ("forked", branch)) if fork else (("serial", None),):
            g = torch.cuda.CUDAGraph()
            with torch.cuda.graph(g, stream=side):
                st = torch.cuda.current_stream().cuda_stream
                b["hidden"].copy_(hidden0)                  # every replay is the same token: synthetic weights would otherwise drift it away
                for i in range(per_graph):
                    layer_step(i, st, br, first=i == 0, last=i == per_graph - 1)
            g.replay()
            side.synchronize()
            rounds, _ = replay_rounds(torch, side, g.replay)
            results[label] = (float(np.median(rounds)) * 1e3 / per_graph, b["hidden" if br is not None else "hidden_alt"].clone())
        # four tokens' layers in one graph: a graph launch costs the device about 12 us before its first kernel, 0.4 us a layer of
        # a one-token graph and 0.1 us here
        tokens_per_graph = 4
        g4 = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g4, stream=side):
            st = torch.cuda.current_stream().cuda_stream
            for tkn in range(tokens_per_graph):
                b["hidden"].copy_(hidden0)
                for i in range(per_graph):
                    layer_step(i, st, None, first=i == 0, last=i == per_graph - 1)
        g4.replay()
        side.synchronize()
        rounds4, _ = replay_rounds(torch, side, g4.replay)
        us4 = float(np.median(rounds4)) * 1e3 / (per_graph * tokens_per_graph)
    us = results["serial"][0]
    if fork:
        assert torch.equal(results["forked"][1], results["serial"][1]), "forked and serial layer chains disagree"
    bad = [n for n, t in b.items() if t.dtype == torch.float16 and not bool(torch.isfinite(t.float()).all())]
    assert not bad, f"non-finite values after the replays in {bad}"
    layer_bytes = (int4_matrix_bytes(NQ * HD + 2 * NKV * HD, D) + int4_matrix_bytes(D, NQ * HD) + SHARED_BYTES + STEP_BYTES
                   + 2 * WINDOW * NKV * HD * 2)
    res = {"workload": "one token through one whole decoder layer (16q/8kv x 256, window 1024, shared 2112, 8 of 128 experts), 30 layers per graph replay",
           "us_per_layer": round(us, 2), "ms_per_30_layers": round(us * 30 / 1e3, 3), "algorithmic_bytes_per_layer": layer_bytes,
           "GBps": round(layer_bytes / (us * 1e-6) / 1e9, 1), "launches_per_layer": 8, "graph": "one in-order chain of launches",
           "us_per_layer_four_tokens_per_graph": round(us4, 2)}
    if fork:
        res["us_per_layer_shared_expert_on_forked_branch"] = round(results["forked"][0], 2)
        res["forked_branch_note"] = ("the shared expert + its norm on a second captured stream (event fork after the post-attention setup, join "
                                     "before the layer tail, as the reference commits sharedCB without waiting); bit-identical")
    return {"decode_layer_sliding_window": res}


def multi_token_extras(torch, tfk, k, gen, lib, h, stream, layer, offs, stride, small_sizes=(2, 4, 8, 16, 32, 64, 128), small_only=False,
                       prefill_only=False, balanced=False):
    """configs[3] (small-M verification, M in {2,4,8,16}) and configs[4] (2048-token prefill, Zipf(1.1) routing) over one
    resident layer: router block -> device grouping -> grouped experts -> token-major reduce, no host round trip."""
    import ctypes as C
    pool, r = layer
    off = tfk.ExpertOffsets(*offs)
    expert_bytes = 3 * int4_matrix_bytes(F_MOE, D)
    res = {}

    def run(T, idx_dev=None, wts_dev=None, iters=20, with_router=True, shared=None, one_call=False):
        n = T * TOPK
        cap = E + n // 64 + 1
        rows_gen = torch.Generator(device="cuda")
        rows_gen.manual_seed(0x51A0 + T)          # the same token rows for every way of running a size
        hid = torch.randn((T, D), device="cuda", generator=rows_gen).to(torch.float16)
        idx = torch.zeros((T, TOPK), dtype=torch.int32, device="cuda") if idx_dev is None else idx_dev
        wts = torch.zeros((T, TOPK), dtype=torch.float16, device="cuda") if wts_dev is None else wts_dev
        sp = torch.zeros(n * 4, dtype=torch.int32, device="cuda")
        offs_d, cnts_d = torch.zeros(E, dtype=torch.int32, device="cuda"), torch.zeros(E, dtype=torch.int32, device="cuda")
        chunks, nch = torch.zeros(cap * 3, dtype=torch.int32, device="cuda"), torch.zeros(1, dtype=torch.int32, device="cuda")
        acts = torch.zeros(n * F_MOE, dtype=torch.float16, device="cuda")
        partials = torch.zeros(n * D, dtype=torch.float16, device="cuda")
        h2 = torch.zeros(T * D, dtype=torch.float16, device="cuda")

        def fn(i):
            rc = 0
            if one_call:        # router, experts and reduce of a few token rows as one call of three launches
                rc = lib.tf_prefill_routed_moe_few_tokens(h, stream, r["W"].data_ptr(), 0, r["S"].data_ptr(), 0, r["B"].data_ptr(), 0, hid.data_ptr(), 0,
                                                          r["eff"].data_ptr(), 0, r["gain"].data_ptr(), 0, idx.data_ptr(), 0, wts.data_ptr(), 0, T, E, D,
                                                          TOPK, D, hid.data_ptr(), 0, D, pool.data_ptr(), stride, C.byref(off), acts.data_ptr(),
                                                          partials.data_ptr(), h2.data_ptr(), 0, F_MOE, tfk.TF_BF16)
                assert rc == 0, k.last_error()
                return
            if with_router:     # router block + device grouping as one call (one launch fewer up to 32 tokens)
                rc |= lib.tf_prefill_router_group_block(h, stream, r["W"].data_ptr(), 0, r["S"].data_ptr(), 0, r["B"].data_ptr(), 0,
                                                        hid.data_ptr(), 0, r["eff"].data_ptr(), 0, r["gain"].data_ptr(), 0,
                                                        idx.data_ptr(), 0, wts.data_ptr(), 0, T, E, D, TOPK, D, sp.data_ptr(),
                                                        offs_d.data_ptr(), cnts_d.data_ptr(), chunks.data_ptr(), nch.data_ptr())
            else:
                rc |= lib.tf_prefill_group_pairs_device(h, stream, idx.data_ptr(), wts.data_ptr(), T, TOPK, E, sp.data_ptr(),
                                                        offs_d.data_ptr(), cnts_d.data_ptr(), chunks.data_ptr(), nch.data_ptr())
            routed = (h, stream, hid.data_ptr(), 0, D, sp.data_ptr(), chunks.data_ptr(), nch.data_ptr(), cap, n, pool.data_ptr(), stride, E,
                      C.byref(off), acts.data_ptr(), partials.data_ptr(), D, F_MOE, TOPK, tfk.TF_BF16)
            if shared is None:
                rc |= lib.tf_prefill_grouped_routed_moe_resident(*routed)
            else:     # the shared expert of the same token rows in the same launches
                rc |= lib.tf_prefill_grouped_routed_moe_resident_shared(
                    *routed, hid.data_ptr(), 0, shared["y"].data_ptr(), 0, C.byref(shared["gate"]), C.byref(shared["up"]), C.byref(shared["down"]),
                    *(v for t in shared["row_scratch"] for v in (t.data_ptr(), 0, F_SHARED * 2)), T, F_SHARED, D, D, 4)
            rc |= lib.tf_prefill_moe_reduce_token_major(h, stream, partials.data_ptr(), 0, wts.data_ptr(), 0, h2.data_ptr(), 0, T, TOPK, D)
            assert rc == 0, k.last_error()
        us = time_loop(torch, fn, iters, warmup=2)
        unique = int(torch.unique(idx).numel()) if one_call else int((cnts_d > 0).sum().item())
        return us, unique

    small = {}
    for M in (() if prefill_only else small_sizes):      # by default: verification sizes, then the reference's prefill chunk sizes (RuntimeConfiguration.swift:24)
        us, unique = run(M, iters=50)
        entry = {"us_grouped_calls": round(us, 2)}
        if M <= 32:      # tf_prefill_routed_moe_few_tokens serves up to 32 token rows
            us_one, unique_one = run(M, iters=50, one_call=True)
            assert unique_one == unique, (unique_one, unique)
            entry["us_one_call"] = round(us_one, 2)
            us = min(us, us_one)
        nbytes = unique * expert_bytes + E * D + M * (2 * D * 2 + TOPK * F_MOE * 2 * 2 + TOPK * D * 2 * 2)
        small[str(M)] = {"us": round(us, 2), **entry, "unique_experts": unique, "GBps_on_unique_expert_bytes": round(nbytes / (us * 1e-6) / 1e9, 1),
                         "tokens_per_s": round(M / (us * 1e-6), 1)}
    if small:
        res["small_m"] = {"workload": "configs[3]: M tokens x top-8 over 128 resident experts (router block + grouping + grouped experts + reduce; "
                                      "us = the faster of the grouped calls, five launches, and the one-call form for up to 32 tokens: three launches of its own up to five tokens, the grouped calls made inside beyond)",
                          "per_M": small}
    if small_only:
        return res

    # configs[4]: 2048 tokens, Zipf(1.1) expert popularity, 8 distinct experts per token
    T = 2048
    rng = np.random.default_rng(0x21BF)
    p = 1.0 / np.arange(1, E + 1) ** 1.1
    p /= p.sum()
    idx_np = np.stack([rng.choice(E, size=TOPK, replace=False, p=p) for _ in range(T)]).astype(np.int32)
    if balanced:
        idx_np = np.stack([(np.arange(TOPK) * (E // TOPK) + t) % E for t in range(T)]).astype(np.int32)
    idx_dev = torch.from_numpy(idx_np).cuda()
    wts_dev = torch.softmax(torch.randn((T, TOPK), device="cuda", generator=gen), dim=1).to(torch.float16)
    us, unique = run(T, idx_dev, wts_dev, iters=5, with_router=False)
    routed_flop = T * TOPK * 2 * 3 * F_MOE * D
    res["prefill_routed_2048"] = {"workload": "configs[4] routed part: 2048 tokens, " + ("128 pairs for every one of" if balanced else "Zipf(1.1) top-8 over") +
                                  " 128 int4 experts, grouped GEMM on MFMA",
                                  "ms": round(us / 1e3, 3), "tokens_per_s": round(T / (us * 1e-6), 1), "unique_experts": unique,
                                  "TFLOPs": round(routed_flop / (us * 1e-6) / 1e12, 2),
                                  "frac_mfma_fp16_peak": round(routed_flop / (us * 1e-6) / 2.5e15, 4)}
    # the router block for the same 2048 tokens (8-bit projection on the matrix cores + one selection wave per token)
    hid_r = torch.randn((T, D), device="cuda", generator=gen).to(torch.float16)
    idx_r = torch.zeros((T, TOPK), dtype=torch.int32, device="cuda")
    wts_r = torch.zeros((T, TOPK), dtype=torch.float16, device="cuda")

    def router_fn(i):
        rc = lib.tf_prefill_router_gemma4_block(h, stream, r["W"].data_ptr(), 0, r["S"].data_ptr(), 0, r["B"].data_ptr(), 0,
                                                hid_r.data_ptr(), 0, r["eff"].data_ptr(), 0, r["gain"].data_ptr(), 0,
                                                idx_r.data_ptr(), 0, wts_r.data_ptr(), 0, T, E, D, TOPK, D)
        assert rc == 0, k.last_error()
    us_router = time_loop(torch, router_fn, 20, warmup=2)
    res["prefill_router_2048"] = {"us": round(us_router, 2), "tokens_per_s": round(T / (us_router * 1e-6), 1)}
    # shared expert over all tokens: gate, up (2112 x 2816), GeGLU, down (2816 x 2112) as dense int4 QMMs
    gW, gS, gB = make_int4(torch, gen, F_SHARED, D)
    uW, uS, uB = make_int4(torch, gen, F_SHARED, D)
    dW, dS, dB = make_int4(torch, gen, D, F_SHARED)
    x = torch.randn((T, D), device="cuda", generator=gen).to(torch.float16)
    g_out = torch.zeros((T, F_SHARED), dtype=torch.float16, device="cuda")
    u_out = torch.zeros((T, F_SHARED), dtype=torch.float16, device="cuda")
    a_out = torch.zeros((T, F_SHARED), dtype=torch.float16, device="cuda")
    y_out = torch.zeros((T, D), dtype=torch.float16, device="cuda")

    gate_p, up_p, down_p = tfk.projection(gW, gS, gB, F_SHARED, D), tfk.projection(uW, uS, uB, F_SHARED, D), tfk.projection(dW, dS, dB, D, F_SHARED)
    row_scratch = [torch.zeros(F_SHARED, dtype=torch.float16, device="cuda") for _ in range(3)]

    def shared(i):
        k.prefill_shared_expert_block(x, gate_p, up_p, down_p, y_out, row_scratch[0], row_scratch[1], row_scratch[2], T, D, F_SHARED)

    def shared_separate(i):
        rc = lib.tf_int4_qmm(h, stream, gW.data_ptr(), 0, gS.data_ptr(), 0, gB.data_ptr(), 0, x.data_ptr(), 0, g_out.data_ptr(), 0, T, F_SHARED, D, tfk.TF_BF16)
        rc |= lib.tf_int4_qmm(h, stream, uW.data_ptr(), 0, uS.data_ptr(), 0, uB.data_ptr(), 0, x.data_ptr(), 0, u_out.data_ptr(), 0, T, F_SHARED, D, tfk.TF_BF16)
        rc |= lib.tf_gelu_mul_fp16(h, stream, g_out.data_ptr(), 0, u_out.data_ptr(), 0, a_out.data_ptr(), 0, T * F_SHARED)
        rc |= lib.tf_int4_qmm(h, stream, dW.data_ptr(), 0, dS.data_ptr(), 0, dB.data_ptr(), 0, a_out.data_ptr(), 0, y_out.data_ptr(), 0, T, D, F_SHARED, tfk.TF_BF16)
        assert rc == 0, k.last_error()
    us_sep = time_loop(torch, shared_separate, 5, warmup=2)
    us_s = time_loop(torch, shared, 5, warmup=2)
    shared_flop = T * 2 * 3 * F_SHARED * D
    res["prefill_shared_2048"] = {"workload": "configs[4] shared expert: 2048 tokens through the block entry (gate+up+GeGLU in one pass, then down; int4 on MFMA)",
                                  "ms": round(us_s / 1e3, 3), "ms_as_three_qmm_calls_and_gelu_mul": round(us_sep / 1e3, 3), "TFLOPs": round(shared_flop / (us_s * 1e-6) / 1e12, 2),
                                  "frac_mfma_fp16_peak": round(shared_flop / (us_s * 1e-6) / 2.5e15, 4)}
    # routed and shared expert as one call: the shared expert's tiles ride in the routed stages' two launches
    us_both, _ = run(T, idx_dev, wts_dev, iters=5, with_router=False,
                     shared={"y": y_out, "gate": gate_p, "up": up_p, "down": down_p, "row_scratch": row_scratch})
    res["prefill_2048_total"] = {"workload": "configs[4]: grouping + routed experts + shared expert + token-major reduce of 2048 tokens, routed and shared "
                                             "expert through tf_prefill_grouped_routed_moe_resident_shared",
                                 "ms": round(us_both / 1e3, 3), "tokens_per_s": round(T / (us_both * 1e-6), 1),
                                 "ms_as_two_calls": round((us + us_s) / 1e3, 3),
                                 "GFLOP": round((routed_flop + shared_flop) / 1e9, 1),
                                 "frac_mfma_fp16_peak": round((routed_flop + shared_flop) / (us_both * 1e-6) / 2.5e15, 4)}
    return res


def cpu_baseline(torch, layers, hidden, idx, wts, y, offs, stride, payload, args):
    """The CPU restatement of the reference's FP32 path (the oracle) timed on this host on a bounded sample of the same
    steps; also checks the device results of those steps against it."""
    from oracle import tfo
    off = tfo.ExpertOffsets(*offs)
    n_sample = 64
    total_1, total_n, worst_rel, idx_match = 0.0, 0.0, 0.0, 0
    cores = max(1, min(os.cpu_count() or 1, 16))
    for sidx in range(n_sample):
        i = args.warmup + sidx          # a step of the timed region
        li, hi = i % args.layers, i % hidden.shape[0]
        pool, r = layers[li]
        hid_bits = hidden[hi].view(torch.int16).cpu().numpy().view(np.uint16)
        x = tfo.from_f16_bits(hid_bits)
        W, S, B = r["W"].cpu().numpy(), r["S"].cpu().numpy().view(np.uint16), r["B"].cpu().numpy().view(np.uint16)
        eff = tfo.bf16_array_to_float(r["eff"].cpu().numpy().view(np.uint16))
        gain = tfo.bf16_array_to_float(r["gain"].cpu().numpy().view(np.uint16))
        gpu_idx = idx[hi].cpu().numpy().view(np.uint32)
        blobs_all = {int(e): pool[int(e), :payload].cpu().numpy() for e in gpu_idx}
        t0 = time.perf_counter()
        ref_idx, ref_w, _ = tfo.router_reference(W, S, B, x, eff, gain)
        t_router = time.perf_counter() - t0
        for e in ref_idx:
            if int(e) not in blobs_all:
                blobs_all[int(e)] = pool[int(e), :payload].cpu().numpy()
        blobs = [blobs_all[int(e)] for e in ref_idx]
        zero = np.zeros(D, np.float32)
        t0 = time.perf_counter()
        ref_y = tfo.moe_apply_streamed_routed(blobs, off, x, zero, ref_w, D, F_MOE, threads=1)
        total_1 += time.perf_counter() - t0 + t_router
        t0 = time.perf_counter()
        tfo.moe_apply_streamed_routed(blobs, off, x, zero, ref_w, D, F_MOE, threads=cores)
        total_n += time.perf_counter() - t0 + t_router
        if list(ref_idx) == list(gpu_idx):
            idx_match += 1
            got = y[hi].float().cpu().numpy()
            worst_rel = max(worst_rel, tfo.rel_error(got, ref_y))
    per_step_1 = total_1 / n_sample
    return {"value": round(STEP_BYTES / per_step_1 / 1e9, 4), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": f"{n_sample} of the timed decode steps (router + 8 experts), serial C++ restatement of the reference's "
                      "bulk-dequantise-row-then-fp32-dot path",
            "ms_per_step": round(per_step_1 * 1e3, 3),
            "openmp": {"value": round(STEP_BYTES / (total_n / n_sample) / 1e9, 4), "cores": cores,
                       "ms_per_step": round(total_n / n_sample * 1e3, 3)},
            "parity_on_sample": {"steps_with_identical_expert_indices": idx_match, "of": n_sample,
                                 "worst_rel_error_vs_cpu": round(worst_rel, 6)}}


def cpu_extras(torch, gen, extras_out, layer, offs, stride, payload):
    """CPU rows beside the GPU numbers of configs 0, 2, 3, 4: the serial restatement of the reference's path (1 core, what the
    Swift reference is) and the same with OpenMP over rows; bounded samples, extrapolation stated.  Also checks the full-size
    lm_head token of the device against the CPU."""
    import importlib
    from oracle import tfo
    tfk = importlib.import_module("turbo-fieldfare_amd")
    cores = max(1, min(os.cpu_count() or 1, 16))

    def med_time(fn, reps):
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    to_np16 = lambda t: t.cpu().numpy().view(np.uint16)
    # configs[0]: 2112 x 2816 GEMV
    W, S, B = make_int4(torch, gen, F_SHARED, D)
    Wn, Sn, Bn = W.cpu().numpy(), to_np16(S), to_np16(B)
    x = np.random.default_rng(5).standard_normal(D).astype(np.float16).astype(np.float32)
    nbytes0 = int4_matrix_bytes(F_SHARED, D) + D * 2 + F_SHARED * 2
    t1 = med_time(lambda: tfo.int4_gemv_ref(Wn, Sn, Bn, x, threads=1), 5)
    tn = med_time(lambda: tfo.int4_gemv_ref(Wn, Sn, Bn, x, threads=cores), 5)
    extras_out["gemv_2112x2816"]["cpu"] = {"kind": "port", "sample": "the whole GEMV, median of 5", "ms_1_core": round(t1 * 1e3, 3),
                                           "GBps_1_core": round(nbytes0 / t1 / 1e9, 3), "cores": cores, "ms_openmp": round(tn * 1e3, 3),
                                           "GBps_openmp": round(nbytes0 / tn / 1e9, 3)}
    # configs[2]: the full head on the device against the CPU (token), CPU timed on a row subset (1 core) and in full (OpenMP)
    W, S, B = make_int4(torch, gen, VOCAB, D)
    hid = torch.randn(D, device="cuda", generator=gen).to(torch.float16)
    norm_w = bf16_bits_cuda(torch.rand(D, device="cuda", generator=gen) + 0.5)
    tok = torch.zeros(1, dtype=torch.int32, device="cuda")
    k = tfk.Context(0)
    k.lm_head_greedy(hid, norm_w, W, S, B, tok, D, VOCAB)
    torch.cuda.synchronize()
    Wn, Sn, Bn, hn, nn = W.cpu().numpy(), to_np16(S), to_np16(B), to_np16(hid.view(torch.int16)), to_np16(norm_w)
    del W, S, B
    t0 = time.perf_counter()
    cpu_tok = tfo.lm_head_cpu_greedy(hn, nn, Wn, Sn, Bn, threads=cores)
    t_full_n = time.perf_counter() - t0
    sub = 16384
    t_sub_1 = med_time(lambda: tfo.lm_head_cpu_greedy(hn, nn, Wn[:sub], Sn[:sub], Bn[:sub], threads=1), 3)
    extras_out["lm_head_greedy"]["cpu"] = {"kind": "port", "sample": f"1 core: the first {sub} of {VOCAB} rows, x{VOCAB // sub} extrapolated; OpenMP: all rows",
                                           "ms_1_core_extrapolated": round(t_sub_1 * (VOCAB // sub) * 1e3, 1),
                                           "GBps_1_core": round(LM_HEAD_BYTES / (t_sub_1 * (VOCAB // sub)) / 1e9, 3), "cores": cores,
                                           "ms_openmp": round(t_full_n * 1e3, 1), "GBps_openmp": round(LM_HEAD_BYTES / t_full_n / 1e9, 3)}
    extras_out["lm_head_greedy"]["token_equals_cpu_at_full_size"] = bool(int(tok.item()) == cpu_tok)
    del Wn, Sn, Bn
    k.close()
    # configs[3] / configs[4]: the reference's CPU path has no batching: a token costs one routed decode step (router + 8 experts)
    # and, for configs[4], one shared expert; timed on two tokens, multiplied out
    pool, r = layer
    off = tfo.ExpertOffsets(*offs)
    rW, rS, rB = r["W"].cpu().numpy(), to_np16(r["S"]), to_np16(r["B"])
    eff, gain = tfo.bf16_array_to_float(to_np16(r["eff"])), tfo.bf16_array_to_float(to_np16(r["gain"]))
    rng = np.random.default_rng(11)
    per_tok_1, per_tok_n = [], []
    for _ in range(2):
        xt = rng.standard_normal(D).astype(np.float16).astype(np.float32)
        t0 = time.perf_counter()
        ridx, rw, _ = tfo.router_reference(rW, rS, rB, xt, eff, gain)
        t_r = time.perf_counter() - t0
        blobs = [pool[int(e), :payload].cpu().numpy() for e in ridx]
        zero = np.zeros(D, np.float32)
        per_tok_1.append(t_r + med_time(lambda: tfo.moe_apply_streamed_routed(blobs, off, xt, zero, rw, D, F_MOE, threads=1), 1))
        per_tok_n.append(t_r + med_time(lambda: tfo.moe_apply_streamed_routed(blobs, off, xt, zero, rw, D, F_MOE, threads=cores), 1))
    routed_1, routed_n = float(np.mean(per_tok_1)), float(np.mean(per_tok_n))
    if "small_m" in extras_out:
        extras_out["small_m"]["cpu"] = {"kind": "port", "sample": "2 tokens (router + 8 experts each, no sharing of experts between tokens on the CPU path), "
                                        "multiplied by M", "cores": cores,
                                        "ms_per_M_1_core": {m: round(int(m) * routed_1 * 1e3, 1) for m in extras_out["small_m"]["per_M"]},
                                        "ms_per_M_openmp": {m: round(int(m) * routed_n * 1e3, 1) for m in extras_out["small_m"]["per_M"]}}
    g, u, dn = (tuple(a.cpu().numpy() if a.dtype == torch.uint8 else to_np16(a) for a in make_int4(torch, gen, rows, cols))
                for rows, cols in ((F_SHARED, D), (F_SHARED, D), (D, F_SHARED)))
    xt = rng.standard_normal(D).astype(np.float16).astype(np.float32)
    sh_1 = med_time(lambda: tfo.shared_expert_ref(g, u, dn, xt, threads=1), 2)
    sh_n = med_time(lambda: tfo.shared_expert_ref(g, u, dn, xt, threads=cores), 2)
    if "prefill_2048_total" in extras_out:
        flop = extras_out["prefill_2048_total"]["GFLOP"] * 1e9
        extras_out["prefill_2048_total"]["cpu"] = {"kind": "port", "sample": "2 tokens routed + 1 token shared expert, x2048 extrapolated", "cores": cores,
                                                   "s_1_core_extrapolated": round(2048 * (routed_1 + sh_1), 1),
                                                   "GFLOPs_1_core": round(flop / (2048 * (routed_1 + sh_1)) / 1e9, 2),
                                                   "s_openmp_extrapolated": round(2048 * (routed_n + sh_n), 2),
                                                   "GFLOPs_openmp": round(flop / (2048 * (routed_n + sh_n)) / 1e9, 2),
                                                   "tokens_per_s_1_core": round(1.0 / (routed_1 + sh_1), 2)}


if __name__ == "__main__":
    main()

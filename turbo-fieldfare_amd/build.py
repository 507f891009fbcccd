"""Builds libtf_kernels.so (the C-ABI HIP library) for gfx950 with hipcc.

Run as ``python turbo-fieldfare_amd/build.py``; the shared object lands next to this file so that it
travels with the source tree.  Packed-FP32 code generation is switched off for every translation unit.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
OUT = os.path.join(HERE, "libtf_kernels.so")
SOURCES = ["tf_context.hip", "tf_gemv.hip", "tf_moe.hip", "tf_lmhead.hip", "tf_prefill.hip", "tf_prefill_quad.hip", "tf_prefill_few.hip", "tf_qmm.hip", "tf_glue.hip", "tf_sampling.hip", "tf_loader.hip", "tf_attention.hip", "tf_rope.hip", "tf_bench.hip"]
FLAGS = ["-O3", "--offload-arch=gfx950", "-fPIC", "-std=c++17", "-Wall", "-Wno-unused-function",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
# Kernel-argument preloading: gfx950 can hand the leading scalar arguments to a wave in registers at launch instead of through
# a scalar load that heads every kernel's dependency chain (the code keeps a prologue that loads them itself where the firmware
# does not preload).  The decode kernels are a launch and two or three memory round trips long, so that load is on the critical
# path: 0.15 us of the three-launch decode step, 0.4 us of the eight-launch decoder layer.
FLAGS += ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
# tf_prefill_quad.hip: the scheduler's register-pressure trackers let the 8-pair gate / up quad kernel fit three blocks a CU (165
# registers, no spill; without them 168 and one spill).  Only that file: the other kernels measured slightly slower with them.
EXTRA_FLAGS: dict = {"tf_prefill_quad.hip": ["-mllvm", "-amdgpu-use-amdgpu-trackers=1"]}


def _hipcc() -> str:
    for cand in (os.environ.get("HIPCC"), "/opt/rocm/bin/hipcc", "hipcc"):
        if cand and (os.path.sep not in cand or os.path.exists(cand)):
            return cand
    return "hipcc"


def _compile(src: str) -> str:
    obj = os.path.join(CSRC, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *FLAGS, *EXTRA_FLAGS.get(src, []), "-c", os.path.join(CSRC, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature and says so; that line is noise
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(verbose: bool = False) -> str:
    sources = [s for s in SOURCES if os.path.exists(os.path.join(CSRC, s))]
    with ThreadPoolExecutor(max_workers=min(8, len(sources))) as pool:
        objs = list(pool.map(_compile, sources))
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", OUT, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    if verbose:
        print(f"built {OUT}")
    return OUT


if __name__ == "__main__":
    build(verbose=True)

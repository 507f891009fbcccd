"""The C++ host mirror compiles against the C ABI header and its CPU-only parts behave like the reference's
(PrefillMoEGroupingTests.swift:6-56, :137-152)."""
import pathlib
import shutil
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parents[1]
PKG = ROOT / "turbo-fieldfare_amd"


@pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
def test_host_mirror_compiles_and_groups(tmp_path):
    lib = PKG / "libtf_kernels.so"
    if not lib.exists():
        pytest.skip("libtf_kernels.so not built")
    exe = tmp_path / "host_mirror_check"
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-o", str(exe), str(ROOT / "tests" / "host_mirror_check.cpp"),
           f"-L{PKG}", "-ltf_kernels", f"-Wl,-rpath,{PKG}"]
    subprocess.run(cmd, check=True, cwd=ROOT)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True)
    assert "host mirror ok" in out.stdout

"""The packed-experts layout reader of the C++ host mirror (tf_gturbo.hpp) on hand-written layouts: the toy layout of the
reference's PackedExpertsLayoutTests.swift:21-87, a production-shaped one with permuted physical ranks, and the
rejections of GTurboV1StructuralValidator (GTurboPackedExpertsLayoutV1.swift:88-180).  CPU only."""
import copy
import json
import pathlib
import shutil
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parents[1]
PKG = ROOT / "turbo-fieldfare_amd"
pytestmark = pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    lib = PKG / "libtf_kernels.so"
    if not lib.exists():
        pytest.skip("libtf_kernels.so not built")
    exe = tmp_path_factory.mktemp("gturbo") / "gturbo_layout_check"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-o", str(exe), str(ROOT / "tests" / "gturbo_layout_check.cpp"), f"-L{PKG}",
                    "-ltf_kernels", f"-Wl,-rpath,{PKG}"], check=True, cwd=ROOT)
    return exe


def run(checker, tmp_path, layout, raw=None):
    d = tmp_path / "model"
    (d / "packed_experts").mkdir(parents=True, exist_ok=True)
    (d / "packed_experts" / "layout.json").write_text(raw if raw is not None else json.dumps(layout, indent=1))
    out = subprocess.run([str(checker), str(d)], capture_output=True, text=True)
    return out.returncode, out.stdout


def routed_tensors(d=2816, f=704):
    """The nine sub-tensors of a routed expert at 64-byte aligned offsets (RepackPlanner.swift:337-415)."""
    out, pos = {}, 0
    for role, rows, cols in (("gate", f, d), ("up", f, d), ("down", d, f)):
        for name, size, dtype, shape, bits in ((role, rows * cols // 2, "U32", [rows, cols // 8], 4),
                                               (role + "_scales", rows * (cols // 64) * 2, "BF16", [rows, cols // 64], None),
                                               (role + "_biases", rows * (cols // 64) * 2, "BF16", [rows, cols // 64], None)):
            entry = {"offset": pos, "size": size, "dtype": dtype, "shape": shape}
            if bits:
                entry["bits"] = bits
            out[name] = entry
            pos = (pos + size + 63) // 64 * 64
    return out, pos


def production_layout(experts=8, layers=2, stride=3358720, ranks=None):
    tensors, _ = routed_tensors()
    out = {"expertStride": stride, "numLayers": layers, "expertsPerLayer": experts, "layers": []}
    for layer in reversed(range(layers)):                       # listed out of order on purpose
        perm = ranks or list(range(experts))
        out["layers"].append({"layer": layer, "file": f"layer_{layer:02d}.bin",
                              "experts": [{"expert": e, "physicalRank": perm[e], "offset": perm[e] * stride, "size": stride,
                                           "tensors": copy.deepcopy(tensors)} for e in range(experts)]})
    return out


def test_toy_layout_of_the_reference_test(checker, tmp_path):
    tensors = {"gate": {"offset": 0, "size": 4096, "dtype": "U32", "shape": [64, 64], "bits": 4},
               "gate_scales": {"offset": 4096, "size": 256, "dtype": "BF16", "shape": [64, 1]}}
    layout = {"expertStride": 16384, "numLayers": 1, "expertsPerLayer": 2,
              "layers": [{"layer": 0, "file": "layer_00.bin",
                          "experts": [{"expert": 0, "offset": 0, "size": 16384, "tensors": tensors},
                                      {"expert": 1, "physicalRank": 1, "offset": 16384, "size": 16384, "tensors": tensors}]}]}
    rc, out = run(checker, tmp_path, layout)
    assert rc == 0
    assert "stride 16384 layers 1 experts 2" in out and "layer 0 file layer_00.bin ranks 0 1" in out
    assert "tensor gate 0 4096 U32 bits 4" in out and "tensor gate_scales 4096 256 BF16 bits 0" in out
    assert "offsets-error" in out and "missing role gate_biases" in out        # a toy expert is not a complete routed expert


def test_production_shaped_layout_with_permuted_ranks(checker, tmp_path):
    ranks = [3, 0, 7, 1, 6, 2, 5, 4]
    rc, out = run(checker, tmp_path, production_layout(ranks=ranks))
    assert rc == 0
    lines = out.splitlines()
    assert lines[0] == "stride 3358720 layers 2 experts 8"
    assert lines[1] == "layer 0 file layer_00.bin ranks 3 0 7 1 6 2 5 4" and lines[3].startswith("layer 1 file layer_01.bin")   # sorted by layer
    tensors, end = routed_tensors()
    want = [tensors[n]["offset"] for n in ("gate", "gate_scales", "gate_biases", "up", "up_scales", "up_biases", "down", "down_scales", "down_biases")]
    assert lines[2] == "offsets " + " ".join(str(v) for v in want)
    assert end == 3345408                                                       # the payload of a production expert blob
    positional = production_layout()
    for layer in positional["layers"]:
        for e in layer["experts"]:
            del e["expert"], e["physicalRank"]
    assert run(checker, tmp_path, positional)[0] == 0                           # ids may be positional


def mutate(fn):
    layout = production_layout(experts=4, layers=1)
    fn(layout)
    return layout


@pytest.mark.parametrize("change,needle", [
    (lambda l: l.update(expertStride=3358721), "invalid dimensions or stride"),                       # not a multiple of 16384
    (lambda l: l.update(numLayers=2), "invalid dimensions or stride"),                                # layer count mismatch
    (lambda l: l["layers"][0].update(layer=1), "duplicate or invalid layer"),
    (lambda l: l["layers"][0].update(file="../layer_00.bin"), "not a plain file name"),
    (lambda l: l["layers"][0].update(file="Layout.JSON"), "reserved packed-expert filename"),
    (lambda l: l["layers"][0]["experts"].pop(), "wrong expert count"),
    (lambda l: l["layers"][0]["experts"][1].pop("expert"), "either all explicit or all positional"),
    (lambda l: l["layers"][0]["experts"][1].update(expert=0), "duplicate or invalid expert mapping"),
    (lambda l: l["layers"][0]["experts"][1].update(physicalRank=2, offset=3358720 * 2), "duplicate or invalid expert mapping"),
    (lambda l: l["layers"][0]["experts"][1].update(physicalRank=2), "offset or size does not match physical rank"),
    (lambda l: l["layers"][0]["experts"][2].update(offset=3358720 * 3), "offset or size does not match physical rank"),
    (lambda l: l["layers"][0]["experts"][2].update(size=16384), "offset or size does not match physical rank"),
    (lambda l: l["layers"][0]["experts"][0]["tensors"]["gate"].update(dtype="F16"), "invalid dtype or shape"),
    (lambda l: l["layers"][0]["experts"][0]["tensors"]["gate"].update(shape=[]), "invalid dtype or shape"),
    (lambda l: l["layers"][0]["experts"][0]["tensors"]["gate"].update(bits=33), "invalid dtype or shape"),
    (lambda l: l["layers"][0]["experts"][0]["tensors"]["down_biases"].update(offset=3358720 - 8), "range exceeds expert blob"),
    (lambda l: l["layers"][0]["experts"][0]["tensors"]["up"].update(offset=100), "overlapping ranges"),
])
def test_structural_validator_rejections(checker, tmp_path, change, needle):
    rc, out = run(checker, tmp_path, mutate(change))
    assert rc == 1 and out.startswith("error:") and needle in out, out


def test_metadata_must_agree_across_experts_and_json_must_be_sound(checker, tmp_path):
    layout = production_layout(experts=4, layers=1)
    layout["layers"][0]["experts"][3]["tensors"]["up_scales"]["offset"] += 64
    layout["layers"][0]["experts"][3]["tensors"]["up_scales"]["size"] -= 64
    rc, out = run(checker, tmp_path, layout)
    assert rc == 0 and "offsets-error" in out and "differs across experts" in out                    # Model.swift:714-720
    for raw in ("", "{", '{"expertStride": 16384,}', '{"expertStride": -16384}', '{"expertStride": 1.5e4}', "[1, 2]",
                '{"expertStride": 16384, "expertStride": 16384}', '{"expertStride": 99999999999999999999}'):
        rc, out = run(checker, tmp_path, None, raw=raw)
        assert rc == 1 and out.startswith("error:"), (raw, out)
    rc, out = subprocess.run([str(checker), str(tmp_path / "nowhere")], capture_output=True, text=True).returncode, None
    assert rc == 1

"""The resident-index reader of the C++ host mirror (tf_gturbo.hpp) on hand-written index regions: the two-entry file of
the reference's ResidentIndexTests.swift:17-102, its size and cap checks (:104-160), the codec's rejections
(GTurboFormatCodecTests.swift:231-280; GTurboResidentIndexV1.swift:57-171) and Model.resident's offset arithmetic
(Model.swift:186-227).  The wire layout is written here from the format description (24-byte header of three
little-endian u64; 72-byte entries: name offset u32, name length u16, dtype u8, reserved u8, weights offset and size u64,
four u32 dimensions, scale offset/size and bias offset/size u64; names in a string table behind the entries).  CPU only."""
import pathlib
import shutil
import struct
import subprocess

import pytest

ROOT = pathlib.Path(__file__).resolve().parents[1]
PKG = ROOT / "turbo-fieldfare_amd"
pytestmark = pytest.mark.skipif(shutil.which("g++") is None, reason="needs g++")
ALIGN = 16384
HEADER, ENTRY = 24, 72


@pytest.fixture(scope="module")
def checker(tmp_path_factory):
    lib = PKG / "libtf_kernels.so"
    if not lib.exists():
        pytest.skip("libtf_kernels.so not built")
    exe = tmp_path_factory.mktemp("gturbo") / "gturbo_resident_check"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-Werror", "-o", str(exe), str(ROOT / "tests" / "gturbo_resident_check.cpp"), f"-L{PKG}",
                    "-ltf_kernels", f"-Wl,-rpath,{PKG}"], check=True, cwd=ROOT)
    return exe


def entry_bytes(name_offset, name_len, dtype, weights, shape, scales=(0, 0), biases=(0, 0), reserved=0):
    return struct.pack("<IHBBQQ4IQQQQ", name_offset, name_len, dtype, reserved, weights[0], weights[1], *shape, scales[0], scales[1],
                       biases[0], biases[1])


def index_file(entries, index_size=ALIGN, resident_size=96, payload=True, name_bytes=None, name_offsets=None, entry_count=None):
    """entries: dicts with name, dtype, weights (offset, size), shape, scales, biases."""
    names = [e["name"].encode() if name_bytes is None else name_bytes for e in entries]
    table_base = HEADER + len(entries) * ENTRY
    out = bytearray(index_size + (resident_size if payload else 0))
    struct.pack_into("<QQQ", out, 0, index_size, resident_size, len(entries) if entry_count is None else entry_count)
    cursor = table_base
    for i, e in enumerate(entries):
        off = cursor if name_offsets is None else name_offsets[i]
        out[HEADER + i * ENTRY: HEADER + (i + 1) * ENTRY] = entry_bytes(off, len(names[i]), e.get("dtype", 0), e["weights"], e["shape"],
                                                                        e.get("scales", (0, 0)), e.get("biases", (0, 0)), e.get("reserved", 0))
        if name_offsets is None:
            out[cursor: cursor + len(names[i])] = names[i]
            cursor += len(names[i])
    return bytes(out)


def run(checker, tmp_path, data, *names):
    path = tmp_path / "model_weights.bin"
    path.write_bytes(data)
    out = subprocess.run([str(checker), str(path), *names], capture_output=True, text=True)
    return out.returncode, out.stdout


TWO = [dict(name="embedding.weight", weights=(ALIGN, 32), shape=(1024, 64, 0, 0), scales=(ALIGN + 32, 16), biases=(ALIGN + 48, 16)),
       dict(name="layer.0.q_proj.weight", weights=(ALIGN + 64, 32), shape=(256, 64, 0, 0))]


def test_round_trip_of_the_reference_two_entry_file(checker, tmp_path):
    # ResidentIndexTests.swift:17-102
    rc, out = run(checker, tmp_path, index_file(TWO), "embedding.weight", "layer.0.q_proj.weight", "missing.weight")
    assert rc == 0, out
    lines = out.splitlines()
    assert lines[0] == f"header {ALIGN} 96 2"
    assert f"entry embedding.weight dtype 0 weights {ALIGN}+32 shape 1024 64 0 0 scales {ALIGN + 32}+16 biases {ALIGN + 48}+16" in lines
    assert f"entry layer.0.q_proj.weight dtype 0 weights {ALIGN + 64}+32 shape 256 64 0 0 scales 0+0 biases 0+0" in lines
    # Model.resident: absolute file offsets become offsets inside the payload (Model.swift:213-227)
    assert "view embedding.weight 0 32 32 16 48 16" in lines
    assert "view layer.0.q_proj.weight 64 32 0 0 0 0" in lines
    assert any(line.startswith("view-error 1: tensor not found: missing.weight") for line in lines)


def test_named_accessors_build_the_writer_s_tensor_names(checker, tmp_path):
    # Model.swift:88-183: shared expert without a `.shared_expert.` segment, router as `.router.proj.weight`, tied lm_head
    entries = [dict(name="language_model.model.embed_tokens.weight", weights=(ALIGN, 16), shape=(8, 4, 0, 0)),
               dict(name="language_model.model.layers.0.mlp.gate_proj.weight", weights=(ALIGN + 16, 16), shape=(8, 4, 0, 0),
                    scales=(ALIGN + 32, 8), biases=(ALIGN + 40, 8)),
               dict(name="language_model.model.layers.1.router.proj.weight", weights=(ALIGN + 48, 16), shape=(8, 4, 0, 0))]
    rc, out = run(checker, tmp_path, index_file(entries), "@sharedExpertGate0", "@router1", "@lmHead")
    assert rc == 0, out
    assert "view @sharedExpertGate0 16 16 32 8 40 8" in out
    assert "view @router1 48 16 0 0 0 0" in out
    assert "view @lmHead 0 16 0 0 0 0" in out


def test_short_file_and_size_checks(checker, tmp_path):
    # ResidentIndexTests.swift:104-190
    rc, out = run(checker, tmp_path, bytes(8))
    assert rc == 1 and out.startswith("error 0: short read for IndexHeader")
    cap = 16 * 1024 * 1024
    rc, out = run(checker, tmp_path, index_file([], index_size=cap, resident_size=0))
    assert rc == 0 and out.splitlines()[0] == f"header {cap} 0 0"
    over = bytearray(HEADER)
    struct.pack_into("<QQQ", over, 0, cap + 1, 0, 0)
    rc, out = run(checker, tmp_path, bytes(over))
    assert rc == 1 and "metadata cap" in out
    small = bytearray(HEADER)
    struct.pack_into("<QQQ", small, 0, HEADER - 1, 0, 0)
    rc, out = run(checker, tmp_path, bytes(small))
    assert rc == 1 and "smaller than the header" in out
    beyond = bytearray(HEADER)
    struct.pack_into("<QQQ", beyond, 0, ALIGN, 0, 0)
    rc, out = run(checker, tmp_path, bytes(beyond))
    assert rc == 1 and "exceeds file size" in out


@pytest.mark.parametrize("mutate,needle", [
    (lambda e: e.__setitem__("reserved", 1), "reserved: must be zero"),                                 # GTurboFormatCodecTests.swift:274-280
    (lambda e: e.__setitem__("scales", (ALIGN + 16, 32)), "overlaps"),                                  # :242-253
    (lambda e: e.__setitem__("dtype", 4), "dtype: unknown dtype"),
    (lambda e: e.__setitem__("shape", (0, 64, 0, 0)), "shape: first dimension must be positive"),
    (lambda e: e.__setitem__("shape", (4, 0, 2, 0)), "shape: zero dimensions must be trailing"),
    (lambda e: e.__setitem__("weights", (ALIGN, 0)), "weights: primary payload is empty"),
    (lambda e: e.__setitem__("weights", (ALIGN - 16, 32)), "weights: range outside resident payload"),
    (lambda e: e.__setitem__("weights", (ALIGN + 80, 32)), "weights: range outside resident payload"),
    (lambda e: e.__setitem__("biases", (ALIGN + 48, 0)), "biases: absent payload offset must be zero"),
])
def test_codec_rejections(checker, tmp_path, mutate, needle):
    e = dict(name="t", weights=(ALIGN, 32), shape=(4, 4, 0, 0))
    mutate(e)
    rc, out = run(checker, tmp_path, index_file([e]))
    assert rc == 1 and needle in out, out


def test_name_table_rejections(checker, tmp_path):
    e = dict(name="t", weights=(ALIGN, 32), shape=(4, 4, 0, 0))
    # a name that points into the entry table (GTurboFormatCodecTests.swift:255-263)
    rc, out = run(checker, tmp_path, index_file([e], name_offsets=[HEADER]))
    assert rc == 1 and "name: range outside string table" in out
    # invalid UTF-8 (:265-272)
    rc, out = run(checker, tmp_path, index_file([e], name_bytes=b"\xff"))
    assert rc == 1 and "invalid UTF-8 or duplicate" in out
    # overlong and truncated sequences, a surrogate
    for bad in (b"\xc0\x80", b"\xe2\x82", b"\xed\xa0\x80"):
        rc, out = run(checker, tmp_path, index_file([e], name_bytes=bad))
        assert rc == 1 and "invalid UTF-8 or duplicate" in out, bad
    # a duplicate name
    dup = [dict(name="same", weights=(ALIGN, 16), shape=(4, 0, 0, 0)), dict(name="same", weights=(ALIGN + 16, 16), shape=(4, 0, 0, 0))]
    rc, out = run(checker, tmp_path, index_file(dup))
    assert rc == 1 and "invalid UTF-8 or duplicate" in out
    # multi-byte UTF-8 is fine
    ok = dict(name="té中", weights=(ALIGN, 32), shape=(4, 4, 0, 0))
    rc, out = run(checker, tmp_path, index_file([ok]))
    assert rc == 0, out
    # an index size that is not a multiple of the 16 KiB alignment, an entry table larger than the index
    rc, out = run(checker, tmp_path, index_file([e], index_size=ALIGN + 64))
    assert rc == 1 and "resident.index: truncated" in out
    rc, out = run(checker, tmp_path, index_file([], entry_count=1000))
    assert rc == 1 and "entryTable: outside index" in out

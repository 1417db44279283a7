"""CPU: the GGUF reader (host logic of the weight loader) on files written by tests/gguf_writer.py, its size formula on
the reference's own tensor list, and its rejection of malformed files.  No GPU call is made here."""
import ctypes as C
import json
import os
import re
import struct

import numpy as np
import pytest

import gguf_writer as W

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden", "q8_0_layout_fixtures.json")


@pytest.fixture(scope="module")
def gguf():
    from nihilus_amd import gguf as G

    return G


def model_file(tmp_path, oracle, alignment=32):
    k, rows = 256, 64
    embd = oracle.fill_weights(1, rows, k).tobytes()
    attn = oracle.fill_weights(2, 32, 128).tobytes()
    norm = W.f32_bytes(np.arange(128) * 0.5)
    meta = [
        ("general.architecture", W.STRING, "llama"),
        ("general.alignment", W.U32, alignment),
        ("llama.block_count", W.U32, 2),
        ("llama.attention.layer_norm_rms_epsilon", W.F32, 1e-5),
        ("llama.context_length", W.U64, 8192),
        ("some.negative", W.I16, -7),
        ("some.flag", W.BOOL, 1),
        ("some.double", W.F64, 2.5),
        ("tokenizer.ggml.tokens", W.ARRAY, (W.STRING, ["<s>", "hello", "wor ld", ""])),
        ("tokenizer.ggml.token_type", W.ARRAY, (W.I32, [3, 1, 1, 6])),
    ]
    tensors = [
        ("token_embd.weight", [k, rows], 8, embd),
        ("blk.0.attn_norm.weight", [128], 0, norm),
        ("blk.1.attn_q.weight", [128, 32], 8, attn),
        ("output_norm.weight", [128], 0, norm),
    ]
    path = str(tmp_path / "tiny.gguf")
    where = W.write_gguf(path, meta, tensors, alignment=alignment)
    return path, where, {n: raw for n, _, _, raw in tensors}


def test_header_exports_every_declared_symbol(gguf):
    from nihilus_amd import _lib

    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "nihilus_amd", "gguf_q8_0.h")).read(), flags=re.S)
    names = sorted(set(re.findall(r"\b(nh_g[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 15 and sorted(gguf.SIGNATURES) == names
    for n in names:
        assert hasattr(_lib.lib(), n), n


@pytest.mark.parametrize("alignment", [32, 64, 4096])
def test_parse_tensors_and_metadata(gguf, oracle, tmp_path, alignment):
    path, where, raws = model_file(tmp_path, oracle, alignment)
    with gguf.GGUFFile(path) as f:
        assert f.version == 3 and f.alignment == alignment and f.tensor_count == 4 and f.metadata_count == 10
        assert f.data_offset % alignment == 0
        names = [f.tensor_at(i).name.decode() for i in range(4)]
        assert names == ["token_embd.weight", "blk.0.attn_norm.weight", "blk.1.attn_q.weight", "output_norm.weight"]
        t = f.find("token_embd.weight")
        assert (t.n_dims, t.ggml_type, list(t.dims), t.layer) == (2, 8, [256, 64, 1, 1], -1)
        assert t.byte_size == 64 * 8 * 34 and t.file_offset == where["token_embd.weight"] and t.file_offset == f.data_offset + t.offset
        q = f.find("blk.1.attn_q.weight")
        assert (q.layer, q.byte_size, q.offset % alignment) == (1, 32 * 4 * 34, 0)
        n = f.find("blk.0.attn_norm.weight")
        assert (n.layer, n.ggml_type, n.byte_size, list(n.dims)) == (0, 0, 512, [128, 1, 1, 1])
        for name, raw in raws.items():
            assert f.data(f.find(name)) == raw, name
        assert f.string("general.architecture") == "llama"
        assert f.u64("llama.block_count") == 2 and f.u64("llama.context_length") == 8192 and f.u64("some.flag") == 1
        assert f.i64("some.negative") == -7
        assert f.f64("llama.attention.layer_norm_rms_epsilon") == float(np.float32(1e-5)) and f.f64("some.double") == 2.5
        et, cnt, addr = f.array("tokenizer.ggml.token_type")
        assert (et, cnt) == (W.I32, 4) and list(struct.unpack("<4i", C.string_at(addr, 16))) == [3, 1, 1, 6]
        et, cnt, addr = f.array("tokenizer.ggml.tokens")
        assert (et, cnt) == (W.STRING, 4) and struct.unpack("<Q", C.string_at(addr, 8))[0] == 3 and C.string_at(addr + 8, 3) == b"<s>"
        with pytest.raises(Exception) as e:
            f.find("blk.7.attn_q.weight")
        assert e.value.status == -9
        with pytest.raises(Exception) as e:
            f.u64("general.architecture")  # a string, not an integer
        assert e.value.status == -6
        with pytest.raises(Exception) as e:
            f.string("no.such.key")
        assert e.value.status == -9


def test_tensor_byte_sizes_of_the_reference_model(gguf):
    # every Q8_0 tensor of the reference's own dump (dims + byte_size) through the loader's size formula
    with open(GOLDEN) as fh:
        tensors = json.load(fh)["q8_0_tensors"]
    assert len(tensors) == 226
    for t in tensors:
        assert gguf.tensor_bytes(8, t["dims"]) == t["byte_size"], t["name"]
    assert gguf.tensor_bytes(0, [4096]) == 16384 and gguf.tensor_bytes(1, [64, 3]) == 384 and gguf.tensor_bytes(26, [2]) == 8
    assert gguf.tensor_bytes(8, [100, 4]) == -3  # a row must be whole blocks
    assert gguf.tensor_bytes(12, [256, 4]) == 0  # a K-quant: size not known to this loader


def test_rejects_malformed_files(gguf, oracle, tmp_path):
    def status_of(path):
        with pytest.raises(Exception) as e:
            gguf.GGUFFile(path)
        return e.value.status

    assert status_of(str(tmp_path / "missing.gguf")) == -7
    path, _, _ = model_file(tmp_path, oracle)
    good = open(path, "rb").read()

    def variant(name, data):
        p = str(tmp_path / name)
        open(p, "wb").write(data)
        return p

    assert status_of(variant("magic.gguf", b"GGML" + good[4:])) == -8
    assert status_of(variant("version.gguf", good[:4] + struct.pack("<I", 1) + good[8:])) == -8
    assert status_of(variant("tensors.gguf", good[:8] + struct.pack("<Q", 100001) + good[16:])) == -8
    assert status_of(variant("kv.gguf", good[:16] + struct.pack("<Q", 10001) + good[24:])) == -8
    assert status_of(variant("short.gguf", good[:10])) == -8
    assert status_of(variant("cut_in_metadata.gguf", good[:60])) == -8
    assert status_of(variant("cut_in_data.gguf", good[:-100])) == -8  # the last tensor no longer fits in the file
    # five dimensions, an oversized dimension, a misaligned offset, a duplicate name
    blocks = oracle.fill_weights(1, 1, 32).tobytes()
    p = str(tmp_path / "dims5.gguf")
    W.write_gguf(p, [], [("t", [32, 1, 1, 1, 1], 8, blocks)])
    assert status_of(p) == -8
    p = str(tmp_path / "dup.gguf")
    W.write_gguf(p, [], [("t", [32], 8, blocks), ("t", [32], 8, blocks)])
    assert status_of(p) == -8
    p = str(tmp_path / "ragged.gguf")
    W.write_gguf(p, [], [("t", [48], 8, blocks)])
    assert status_of(p) == -8
    p = str(tmp_path / "align0.gguf")
    W.write_gguf(p, [("general.alignment", W.U32, 48)], [("t", [32], 8, blocks)], alignment=48)
    assert status_of(p) == -8  # not a power of two
    # an offset just below 2^64 wraps to a small file offset when added to the data start: the tensor would alias the header
    p = str(tmp_path / "wrap.gguf")
    W.write_gguf(p, [], [("t", [32], 8, blocks)])
    raw = bytearray(open(p, "rb").read())
    at = 24 + (8 + 1) + 4 + 8 + 4  # header, name, n_dims, one dim, type: the record's offset field
    assert struct.unpack_from("<Q", raw, at)[0] == 0
    struct.pack_into("<Q", raw, at, 2**64 - 64)  # data starts at byte 64 of this file: 64 + (2^64 - 64) = 0
    assert status_of(variant("wrap_patched.gguf", bytes(raw))) == -8
    # a v2 file and a file with no tensors are fine
    p = str(tmp_path / "v2.gguf")
    W.write_gguf(p, [("a", W.U8, 5)], [("t", [32], 8, blocks)], version=2)
    with gguf.GGUFFile(p) as f:
        assert f.version == 2 and f.u64("a") == 5 and f.data(f.find("t")) == blocks
    p = str(tmp_path / "empty.gguf")
    W.write_gguf(p, [("a", W.U8, 5)], [])
    with gguf.GGUFFile(p) as f:
        assert f.tensor_count == 0


def test_mutated_files_under_sanitizers(oracle, tmp_path):
    # 6000 mutants of a valid file (truncated, flipped bytes and bits, overwritten counts / lengths / offsets) through every query of the
    # reader, in a build of its source with AddressSanitizer and UBSan: no report, and no accepted tensor may reach past the end of its file
    import subprocess
    import sys

    sys.path.insert(0, os.path.join(ROOT, "tests", "cpp"))
    import build_host_tests as B

    if not os.path.exists(B.FUZZ_BIN) or os.path.getmtime(B.FUZZ_BIN) < max(os.path.getmtime(B.FUZZ_SRC), os.path.getmtime(os.path.join(ROOT, "nihilus_amd", "csrc", "gguf_q8_0.cpp"))):
        B.build_gguf_fuzz()
    path, _, _ = model_file(tmp_path, oracle)
    for seed in (1, 2):
        res = subprocess.run([B.FUZZ_BIN, path, "3000", str(seed), str(tmp_path / "mutant.gguf")], capture_output=True, text=True, timeout=240)
        assert res.returncode == 0, (res.stdout + res.stderr)[-3000:]
        assert "3000 mutants" in res.stdout and "ERROR" not in res.stderr
        assert int(res.stdout.split(",")[1].split()[0]) > 300  # a fair share of the mutants still parses: the queries really ran

"""CPU: pins the checker's fp16 conversions and its reading of the block layout.

fp16: exhaustive over all 65536 halves, every midpoint between neighbouring halves (ties-to-even), numpy's
float16 as an independent converter, F16C hardware as a third.  Layout: the reference's own tensor dumps
(tests/golden/q8_0_layout_fixtures.json, extracted from Leaf_Data_0.json / Node_Data_0.json).
"""
import json
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "q8_0_layout_fixtures.json")


def test_fp16_to_fp32_exhaustive(oracle):
    h = np.arange(65536, dtype=np.uint16)
    ref = h.view(np.float16).astype(np.float32)
    for i in range(65536):
        got = np.float32(oracle.fp16_to_fp32(i))
        hw = np.float32(oracle.fp16_to_fp32_f16c(i))
        if np.isnan(ref[i]):
            assert np.isnan(got) and np.isnan(hw)
        else:
            assert got.tobytes() == ref[i].tobytes() == hw.tobytes(), hex(i)


def test_fp32_to_fp16_roundtrip_and_midpoints(oracle):
    h = np.arange(65536, dtype=np.uint16)
    f = h.view(np.float16).astype(np.float32)
    finite = np.isfinite(f)
    for i in np.nonzero(finite)[0]:
        assert oracle.fp32_to_fp16(f[i]) == i
    # midpoints between neighbouring positive halves go to the even one; a hair either side goes to the nearer
    pos = np.arange(0, 0x7C00, dtype=np.uint16)  # +0 .. largest finite; pos+1 may be inf
    lo = pos.view(np.float16).astype(np.float64)
    hi_bits = (pos + 1).astype(np.uint16)
    hi = np.where(hi_bits == 0x7C00, 65536.0, hi_bits.view(np.float16).astype(np.float64))
    mid = ((lo + hi) / 2).astype(np.float32)  # exactly representable in fp32
    assert np.array_equal(mid.astype(np.float64), (lo + hi) / 2)
    for i in range(0, len(pos), 1):
        even = pos[i] if pos[i] % 2 == 0 else hi_bits[i]
        m = mid[i]
        assert oracle.fp32_to_fp16(m) == even, hex(pos[i])
        assert oracle.fp32_to_fp16_f16c(m) == even
        assert oracle.fp32_to_fp16(np.nextafter(m, np.float32(0))) == pos[i]
        assert oracle.fp32_to_fp16(np.nextafter(m, np.float32(1e9))) == hi_bits[i]
        assert oracle.fp32_to_fp16(-m) == (even | 0x8000)


def test_fp32_to_fp16_random_against_numpy_and_f16c(oracle):
    rng = np.random.default_rng(0)
    mags = 2.0 ** rng.uniform(-30, 17, size=40000)
    f = (rng.standard_normal(40000) * mags).astype(np.float32)
    f = np.concatenate([f, np.float32([0.0, -0.0, 65504, 65519.99, 65520, 65536, 1e30, -1e30, np.inf, -np.inf, 5.96e-8, 2.98e-8, 2.9802322e-8, 1e-10, 1e-45])])
    with np.errstate(over="ignore"):
        ref = f.astype(np.float16).view(np.uint16)
    for v, r in zip(f, ref):
        assert oracle.fp32_to_fp16(v) == r, v
        assert oracle.fp32_to_fp16_f16c(v) == r, v
    assert oracle.fp32_to_fp16(np.float32(np.nan)) & 0x7C00 == 0x7C00 and oracle.fp32_to_fp16(np.float32(np.nan)) & 0x3FF


# ------------------------------------------------------------------ layout against the reference's dumps


@pytest.fixture(scope="module")
def golden():
    with open(GOLDEN) as f:
        return json.load(f)


def test_byte_size_formula_on_all_reference_q8_0_tensors(oracle, golden):
    tensors = golden["q8_0_tensors"]
    assert len(tensors) == 226
    for t in tensors:
        k, rows = t["dims"][0], t["dims"][1]  # ggml order: dim0 = K (fastest), dim1 = rows
        assert t["dims"][2:] == [1, 1]
        assert oracle.q8_0_bytes(rows, k) == t["byte_size"], t["name"]
    sizes = {t["name"]: t["byte_size"] for t in tensors}
    assert sizes["blk.0.attn_q.weight"] == 17825792
    assert sizes["blk.0.ffn_down.weight"] == 62390272
    assert sizes["token_embd.weight"] == 558170112


def test_block_field_positions_on_real_blocks(oracle, golden):
    # Real blocks come out of ggml's quantizer, so each has max|q| == 127 and a small positive finite scale.
    # Reading d or qs from the wrong offset breaks this on the spot.
    seen = 0
    for t in golden["q8_0_tensors"]:
        if "first_bytes" not in t:
            continue
        raw = np.array(t["first_bytes"], dtype=np.uint8)
        assert raw.size == 128
        d, qs = oracle.split_blocks(raw[:102])  # three whole blocks
        for b in range(3):
            scale = oracle.fp16_to_fp32(int(d[b]))
            assert 0.0 < scale < 0.1, (t["name"], b, scale)
            assert np.abs(qs[b].astype(np.int32)).max() == 127, (t["name"], b)
            # quantize(dequantize(block)) reproduces a real block byte for byte
            y = oracle.dequantize_row(raw[34 * b : 34 * b + 34], 32)
            assert np.array_equal(y, np.float32(scale) * qs[b].astype(np.float32))
            assert np.array_equal(oracle.quantize_rows(y)[0], raw[34 * b : 34 * b + 34]), (t["name"], b)
            assert np.array_equal(oracle.quantize_rows(y, avx2=True)[0], raw[34 * b : 34 * b + 34])
            seen += 1
    assert seen == 21
    first = next(t for t in golden["q8_0_tensors"] if t["name"] == "blk.0.attn_q.weight")["first_bytes"]
    assert first[0] | (first[1] << 8) == 0x0BBF and np.array(first[2:5], dtype=np.uint8).view(np.int8).tolist() == [22, -124, -27]


def test_quantize_on_embedding_row_from_reference_graph_dump(oracle, golden):
    # inp_embd (first 32 floats of the embedded first prompt token) is, in the dump, q * d for integers q with
    # max|q| == 127 and one fp32 scale d = amax / 127 (d is NOT fp16-representable there, so this row does not pin
    # the dequantizer; it is real data with a known integer structure, which pins the quantizer): quantizing it
    # must give exactly those integers and the fp16 rounding of that d.
    e = golden["inp_embd"]
    assert e["dims"][0] == 4096 and e["type"] == 0
    y = np.array(e["first_bytes"], dtype=np.uint8).view(np.float32)
    d = np.float32(np.abs(y).max() / np.float32(127.0))
    q = y / d
    assert np.array_equal(q, np.rint(q)) and np.abs(q).max() == 127
    assert np.array_equal(d * q.astype(np.float32), y)
    for avx2 in (False, True):
        dd, qs = oracle.split_blocks(oracle.quantize_rows(y, avx2=avx2)[0])
        assert np.array_equal(qs[0], q.astype(np.int8))
        assert dd[0] == d.astype(np.float16).view(np.uint16)

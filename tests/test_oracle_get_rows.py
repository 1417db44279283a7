"""CPU: the checker's token-embedding lookup (get_rows) against what fixes it independently.

out[t][j] = f32(d[ids[t]][j/32]) * f32(q[ids[t]][j]) (cpu/avx_2.hpp:40-66 under the per-token loops :80-103 and
:112-135).  Pinned by an independent numpy evaluation (numpy's own float16), by real blocks out of the reference's
tensor dumps used as an embedding table, and by a table whose row r decodes to the constant r, so that an
off-by-one or transposed index shows as a wrong constant.
"""
import json
import os

import numpy as np
import pytest

from helpers import random_blocks

GOLDEN = os.path.join(os.path.dirname(__file__), "golden", "q8_0_layout_fixtures.json")


def numpy_get_rows(blocks, ids, n_rows, k):
    b = blocks.reshape(n_rows, k // 32, 34)
    d = b[:, :, :2].copy().view(np.float16).astype(np.float32)  # [rows, nb, 1]
    q = b[:, :, 2:].view(np.int8).astype(np.float32)
    table = (d * q).reshape(n_rows, k)
    out = np.zeros((len(ids), k), dtype=np.float32)
    ok = (ids >= 0) & (ids < n_rows)
    out[ok] = table[ids[ok]]
    return out, int((~ok).sum())


@pytest.mark.parametrize("n_rows,k,n_tokens", [(1, 32, 1), (7, 96, 5), (300, 4096, 64), (128, 128, 1)])
def test_get_rows_against_numpy(oracle, n_rows, k, n_tokens):
    rng = np.random.default_rng(n_rows * 7 + k)
    w = random_blocks(rng, n_rows, k)
    ids = rng.integers(0, n_rows, size=n_tokens, dtype=np.int32)
    ids[0] = n_rows - 1
    ids[-1] = 0
    got, bad = oracle.get_rows(w, ids, n_rows, k)
    want, _ = numpy_get_rows(w, ids, n_rows, k)
    assert bad == 0 and np.array_equal(got, want)


def test_get_rows_row_indexing(oracle):
    # row r: every block d = 1.0, every quant r - 50  ->  the row decodes to the constant r - 50
    n_rows, k = 101, 64
    w = np.empty((n_rows, k // 32, 34), dtype=np.uint8)
    w[:, :, 0], w[:, :, 1] = 0x00, 0x3C  # fp16 1.0
    w[:, :, 2:] = (np.arange(n_rows, dtype=np.int16) - 50).astype(np.int8).view(np.uint8)[:, None, None]
    ids = np.array([100, 0, 50, 7, 7, 99], dtype=np.int32)
    got, bad = oracle.get_rows(w.reshape(-1), ids, n_rows, k)
    assert bad == 0
    for t, r in enumerate(ids):
        assert np.all(got[t] == np.float32(r - 50)), (t, r)


def test_get_rows_out_of_range_ids_give_zero_rows(oracle):
    rng = np.random.default_rng(3)
    n_rows, k = 10, 64
    w = random_blocks(rng, n_rows, k)
    ids = np.array([3, -1, 10, 9, 2**31 - 1, -(2**31)], dtype=np.int32)
    got, bad = oracle.get_rows(w, ids, n_rows, k)
    want, wbad = numpy_get_rows(w, ids, n_rows, k)
    assert bad == wbad == 4 and np.array_equal(got, want)
    assert not got[1].any() and not got[2].any() and got[0].any()


def test_get_rows_on_real_blocks_from_reference_dumps(oracle):
    # 21 dumped tensors x their first three whole blocks = a 21-row, 96-wide embedding table of real ggml blocks
    with open(GOLDEN) as f:
        tensors = [t for t in json.load(f)["q8_0_tensors"] if "first_bytes" in t]
    table = np.stack([np.array(t["first_bytes"], dtype=np.uint8)[:102] for t in tensors])
    n_rows = table.shape[0]
    ids = np.arange(n_rows - 1, -1, -1, dtype=np.int32)
    got, bad = oracle.get_rows(table.reshape(-1), ids, n_rows, 96)
    want, _ = numpy_get_rows(table.reshape(-1), ids, n_rows, 96)
    assert bad == 0 and np.array_equal(got, want)
    # a real block dequantizes to values whose largest magnitude is 127 * d
    d0 = table[ids[0], :2].copy().view(np.float16).astype(np.float32)[0]
    assert np.abs(got[0, :32]).max() == np.float32(127.0) * d0

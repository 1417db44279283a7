"""GPU: token-embedding lookup through the C ABI, bit-exact against the CPU checker, both weight layouts."""
import numpy as np
import pytest

from helpers import random_blocks, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("tiled", [False, True])
@pytest.mark.parametrize("n_rows,k,n_tokens", [(1, 128, 1), (33, 128, 7), (1000, 4096, 1), (1000, 4096, 512), (77, 14336, 9), (40, 1024, 70000)])
def test_get_rows_bit_exact(q8, oracle, tiled, n_rows, k, n_tokens):
    rng = np.random.default_rng(n_rows + k + n_tokens)
    w = random_blocks(rng, n_rows, k)
    ids = rng.integers(0, n_rows, size=n_tokens, dtype=np.int32)
    ids[0], ids[-1] = n_rows - 1, 0
    want, _ = oracle.get_rows(w, ids, n_rows, k)
    wd = to_dev(w)
    if tiled:
        wd = q8.tile(wd, n_rows, k)
    got, bad = q8.get_rows(wd, to_dev(ids), n_rows, k, tiled, count_invalid=True)
    assert bad == 0
    assert np.array_equal(to_host(got), want)


def test_get_rows_blocks_layout_k_multiple_of_32_only(q8, oracle):
    rng = np.random.default_rng(5)
    n_rows, k = 19, 96
    w = random_blocks(rng, n_rows, k)
    ids = rng.integers(0, n_rows, size=11, dtype=np.int32)
    want, _ = oracle.get_rows(w, ids, n_rows, k)
    assert np.array_equal(to_host(q8.get_rows(to_dev(w), to_dev(ids), n_rows, k, False)), want)


@pytest.mark.parametrize("tiled", [False, True])
def test_get_rows_out_of_range_ids(q8, oracle, tiled):
    rng = np.random.default_rng(6)
    n_rows, k = 50, 256
    w = random_blocks(rng, n_rows, k)
    ids = np.array([3, -1, 50, 49, 2**31 - 1, -(2**31), 0], dtype=np.int32)
    want, wbad = oracle.get_rows(w, ids, n_rows, k)
    wd = q8.tile(to_dev(w), n_rows, k) if tiled else to_dev(w)
    got, bad = q8.get_rows(wd, to_dev(ids), n_rows, k, tiled, count_invalid=True)
    assert bad == wbad == 4
    assert np.array_equal(to_host(got), want)
    # without a counter the rows are still zero
    assert np.array_equal(to_host(q8.get_rows(wd, to_dev(ids), n_rows, k, tiled)), want)


def test_get_rows_is_the_dequantized_weight(q8, oracle):
    # ids = 0..n-1 returns the whole matrix dequantized: ties this row to the mat-vec's weights (same bytes, same layout)
    rng = np.random.default_rng(8)
    n_rows, k = 64, 512
    w = random_blocks(rng, n_rows, k)
    ids = np.arange(n_rows, dtype=np.int32)
    got = to_host(q8.get_rows(q8.tile(to_dev(w), n_rows, k), to_dev(ids), n_rows, k, True))
    for r in (0, 31, 32, 63):
        assert np.array_equal(got[r], oracle.dequantize_row(w.reshape(n_rows, -1)[r], k))


def test_get_rows_empty_and_errors(q8):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()

    w = torch.zeros(34 * 4, dtype=torch.uint8, device="cuda")
    ids = torch.zeros(0, dtype=torch.int32, device="cuda")
    assert q8.get_rows(w, ids, 1, 128, False).shape == (0, 128)
    out = torch.zeros(128, dtype=torch.float32, device="cuda")
    one = torch.zeros(1, dtype=torch.int32, device="cuda")
    assert lib.nh_q8_0_get_rows(w.data_ptr(), one.data_ptr(), out.data_ptr(), None, 1, 1, 100, None) == -3  # K % 32
    assert lib.nh_q8_0_get_rows_tiled(w.data_ptr(), one.data_ptr(), out.data_ptr(), None, 1, 1, 96, None) == -3  # K % 128
    assert lib.nh_q8_0_get_rows(w.data_ptr(), None, out.data_ptr(), None, 1, 1, 128, None) == -1
    assert lib.nh_q8_0_get_rows(w.data_ptr(), one.data_ptr(), None, None, 1, 1, 128, None) == -1
    assert lib.nh_q8_0_get_rows(w.data_ptr(), one.data_ptr(), out.data_ptr() + 4, None, 1, 1, 128, None) == -2
    assert lib.nh_q8_0_get_rows(w.data_ptr(), one.data_ptr(), out.data_ptr(), None, -1, 1, 128, None) == -3

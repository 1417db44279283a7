"""GPU: layout conversion is a lossless byte permutation; the device generator equals the CPU one."""
import numpy as np
import pytest

from helpers import random_blocks, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,k", [(32, 128), (1, 128), (33, 256), (4096, 4096), (100, 14336)])
def test_tile_untile_roundtrip(q8, rows, k):
    rng = np.random.default_rng(rows + k)
    w = random_blocks(rng, rows, k)
    t = q8.tile(to_dev(w), rows, k)
    assert t.numel() == ((rows + 31) // 32) * (k // 128) * 4352
    assert np.array_equal(to_host(q8.untile(t, rows, k)), w)


def test_tiled_layout_definition(q8):
    # spot-check the documented address formula against a host-side permutation
    rows, k = 64, 256
    rng = np.random.default_rng(1)
    w = random_blocks(rng, rows, k).reshape(rows, k // 32, 34)
    t = to_host(q8.tile(to_dev(w.reshape(-1)), rows, k))
    groups = k // 128
    for row, b, q in [(0, 0, 0), (5, 3, 17), (37, 6, 31), (63, 7, 15), (32, 4, 16)]:
        macro = ((row // 32) * groups + b // 4) * 4352
        lane = row % 32 + 32 * (q // 16)
        assert t[macro + (b % 4) * 1024 + 16 * lane + q % 16] == w[row, b, 2 + q]
        assert t[macro + 4096 + 8 * (row % 32) + 2 * (b % 4)] == w[row, b, 0]
        assert t[macro + 4096 + 8 * (row % 32) + 2 * (b % 4) + 1] == w[row, b, 1]


def test_device_generator_matches_cpu(q8, oracle):
    for seed, n, k, first in [(0, 64, 4096, 0), (12345, 3, 96, 77), (2**63 + 5, 16, 128, 10**9)]:
        got = to_host(q8.fill_weight_blocks(seed, n, k, first_block=first))
        assert np.array_equal(got, oracle.fill_weights(seed, n, k, first_block=first))
        x = to_host(q8.fill_activations(seed, 4097))
        assert np.array_equal(x, oracle.fill_activations(seed, 4097))

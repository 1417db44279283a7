"""GPU parity: prefill int8-MFMA mat-mat vs the CPU restatement."""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def _inputs(oracle, m, n, k, seed):
    w = oracle.fill_weights(seed, n, k)
    x = oracle.fill_activations(seed, m * k).reshape(m, k)
    return w, x, oracle.quantize_rows(x)


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (128, 14336, 4096), (32, 128, 128), (1, 128, 128), (8, 96, 256), (33, 65, 384), (130, 257, 512), (64, 4096, 14336)])
def test_gemm_tiled_and_blocks(q8, oracle, m, n, k):
    w, x, aq = _inputs(oracle, m, n, k, seed=m + n + k)
    want = oracle.gemm(w, aq, m, n, k, threads=8) if (k // 32) % 16 == 0 else oracle.gemm(w, aq, m, n, k)
    wd, aqd = to_dev(w), to_dev(aq.reshape(-1))
    c_blocks = to_host(q8.gemm(wd, aqd, m, n, k, tiled=False))
    c_tiled = to_host(q8.gemm(q8.tile(wd, n, k), q8.tile(aqd, m, k), m, n, k, tiled=True))
    assert rel_l2(c_blocks, want) <= REL_L2_TOL
    assert rel_l2(c_tiled, want) <= REL_L2_TOL
    assert rel_l2(c_blocks, c_tiled) < 2e-6  # different kernels, different fp32 order, same exact block sums
    # every row separately, so one bad row cannot hide in the norm of the rest
    for i in range(0, m, max(1, m // 7)):
        assert rel_l2(c_tiled[i], want[i]) <= REL_L2_TOL


@pytest.mark.parametrize("m,n,k", [(64, 96, 256), (33, 65, 160), (1, 32, 32), (128, 128, 4096)])
def test_gemm_block_sums_exact(q8, oracle, m, n, k):
    w, x, aq = _inputs(oracle, m, n, k, seed=9)
    got = to_host(q8.debug_block_sums(to_dev(w), to_dev(aq.reshape(-1)), m, n, k, path=1))
    for i in range(m):
        assert np.array_equal(got[i], oracle.block_sums_gemv(w, aq[i], n, k)), i
    if k % 128 == 0:
        wd, aqd = to_dev(w), to_dev(aq.reshape(-1))
        got_t = to_host(q8.debug_block_sums(q8.tile(wd, n, k), q8.tile(aqd, m, k), m, n, k, path=3))
        assert np.array_equal(got_t, got)


def test_gemm_equals_gemvs(q8, oracle):
    # the mat-mat must be M independent mat-vecs on the same quantized rows
    m, n, k = 16, 512, 1024
    w, x, aq = _inputs(oracle, m, n, k, seed=21)
    wd = to_dev(w)
    wt = q8.tile(wd, n, k)
    c = to_host(q8.gemm(wt, q8.tile(to_dev(aq.reshape(-1)), m, k), m, n, k, tiled=True))
    for i in range(m):
        y = to_host(q8.gemv(wt, to_dev(aq[i]), n, k, tiled=True))
        assert rel_l2(c[i], y) < 2e-6


def test_mul_mat_fused(q8, oracle):
    for m, n, k in [(1, 4096, 4096), (512, 4096, 4096), (5, 160, 256)]:
        w, x, aq = _inputs(oracle, m, n, k, seed=33 + m)
        want = oracle.gemm(w, aq, m, n, k, threads=8) if (k // 32) % 16 == 0 else oracle.gemm(w, aq, m, n, k)
        wt = q8.tile(to_dev(w), n, k)
        got = to_host(q8.mul_mat(wt, to_dev(x), n, k))
        assert rel_l2(got, want) <= REL_L2_TOL


def test_gemm_extreme_quants(q8, oracle):
    m, n, k = 32, 32, 128
    nb = k // 32
    one = np.float16(1.0).view(np.uint16)
    a = oracle.pack_blocks(np.full(m * nb, one), np.full((m, k), -127, dtype=np.int8))
    w = oracle.pack_blocks(np.full(n * nb, one), np.full((n, k), 127, dtype=np.int8))
    c = to_host(q8.gemm(to_dev(w), to_dev(a), m, n, k, tiled=False))
    assert np.array_equal(c, np.full((m, n), -127.0 * 127.0 * k, dtype=np.float32))

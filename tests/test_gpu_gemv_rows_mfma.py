"""GPU: four to sixteen activation rows on small matrices -- the streaming mat-vec with the rows as an MFMA operand, the activation
quantize inside the kernel (q8_0_gemv_rows_mfma.hip), reached through nh_q8_0_mul_mat.

Checked against the CPU checker's quantize + mat-mat (1e-4 relative L2 overall and row by row), for every row count the kernel
takes, whole and ragged strips, one and two groups per wave, K over one, two and four workgroups per strip, the chunked walk a
capturing stream gets, with and without a residual; runs of the same call are bit-identical, and rows do not leak into each
other (a row's result does not depend on what the other rows hold).
"""
import numpy as np
import pytest
import torch

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

# (N, K): whole strips / a ragged last strip / few strips (K split over workgroups) / long K (K split, two groups per wave)
SHAPES = [(4096, 4096), (100, 128), (33, 256), (1024, 8192), (4096, 14336), (2048, 512), (6000, 1024), (32, 2048)]


def _want(oracle, w, x, n, k):
    aq = oracle.quantize_rows(x)
    return oracle.gemm(w, aq, x.shape[0], n, k)


@pytest.mark.parametrize("n,k", SHAPES, ids=[f"{n}x{k}" for n, k in SHAPES])
def test_rows_on_the_matrix_cores_match_the_checker(q8, oracle, n, k):
    rng = np.random.default_rng(n + k)
    w = random_blocks(rng, n, k, 0.02)
    wt = q8.tile(to_dev(w), n, k)
    for m in ((4, 5, 6, 7, 8, 9, 11, 16) if n * (k // 32) * 34 <= 40 << 20 else (4,)):  # above 40 MB the kernel takes four rows only
        assert q8.plan_mul_mat(m, n, k)["kernel"] == "gemv_rows_mfma"
        x = rng.standard_normal((m, k)).astype(np.float32)
        x[m - 1, : k // 2] *= 37.0  # rows of different magnitude: every row has its own block scales
        res = rng.standard_normal((m, n)).astype(np.float32)
        y = to_host(q8.mul_mat(wt, to_dev(x), n, k))
        want = _want(oracle, w, x, n, k)
        assert np.isfinite(y).all()
        assert rel_l2(y, want) <= REL_L2_TOL
        assert max(rel_l2(y[i], want[i]) for i in range(m)) <= REL_L2_TOL
        assert np.array_equal(to_host(q8.mul_mat(wt, to_dev(x), n, k)), y)  # run-to-run bit-stable
        yr = to_host(q8.mul_mat(wt, to_dev(x), n, k, residual=to_dev(res)))
        assert np.array_equal(yr, y + res)  # one fp32 add after the sum
        # a row's result is its own: the same row among other rows, and at another position, gives the same bits
        x2 = rng.standard_normal((m, k)).astype(np.float32)
        x2[0] = x[m - 1]
        y2 = to_host(q8.mul_mat(wt, to_dev(x2), n, k))
        assert np.array_equal(y2[0], y[m - 1])


def test_rows_of_zeros_and_an_absent_scale(q8, oracle):
    n, k = 256, 512
    rng = np.random.default_rng(5)
    w = random_blocks(rng, n, k, 0.02)
    wt = q8.tile(to_dev(w), n, k)
    x = rng.standard_normal((11, k)).astype(np.float32)
    x[9] = 0.0
    x[2] = 0.0  # amax = 0: scale 0, quants 0 (the reference's guard against 127 / 0)
    x[4, 32:64] = 0.0  # one block of zeros inside a row
    y = to_host(q8.mul_mat(wt, to_dev(x), n, k))
    assert np.array_equal(y[2], np.zeros(n, dtype=np.float32)) and np.array_equal(y[9], np.zeros(n, dtype=np.float32))
    assert rel_l2(y, _want(oracle, w, x, n, k)) <= REL_L2_TOL


@pytest.mark.parametrize("m", [8, 16])
def test_captured_stream_takes_the_unsplit_walk(q8, oracle, m):
    # under capture the K split's hand-off (an epoch per launch) cannot be used: the same kernel walks K in chunks instead
    from nihilus_amd import _lib

    _lib.check("nh_q8_0_prepare", _lib.lib().nh_q8_0_prepare())
    n, k = 1024, 8192
    assert q8.plan_mul_mat(m, n, k)["k_splits"] == 4
    rng = np.random.default_rng(9)
    w = random_blocks(rng, n, k, 0.02)
    wt = q8.tile(to_dev(w), n, k)
    x_d = torch.zeros((m, k), dtype=torch.float32, device="cuda")
    q8.mul_mat(wt, x_d, n, k)  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y_d = q8.mul_mat(wt, x_d, n, k)
    for rep in range(3):
        x = rng.standard_normal((m, k)).astype(np.float32)
        x_d.copy_(to_dev(x))
        graph.replay()
        torch.cuda.synchronize()
        got = to_host(y_d).copy()
        eager = to_host(q8.mul_mat(wt, x_d, n, k))  # the split form, with a fresh epoch, between the replays
        assert rel_l2(got, eager) < 2e-6, rep  # same arithmetic, another cut of K
        assert rel_l2(got, _want(oracle, w, x, n, k)) <= REL_L2_TOL, rep

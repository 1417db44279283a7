"""GPU: one parity case per route of nh_q8_0_mul_mat, with the route asserted.

Each case names the kernel (and the part of its cut) it means to cover; the test first asks the library's plan function that
the shape really takes that route -- the launchers execute exactly that plan -- and then compares the result with the CPU
checker.  A threshold that moves a shape onto another kernel fails here by name instead of silently changing what is covered.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

# (M, N, K, kernel, the plan entries that must hold)
ROUTES = [
    (1, 4096, 14336, "gemv", {"k_splits": 4, "row_parts": 1}),  # K over four workgroups per strip, tagged hand-off
    (1, 1024, 4096, "gemv", {"k_splits": 1, "row_parts": 4}),  # 32 strips cut into four row parts each
    (1, 4096, 4096, "gemv", {"k_splits": 1, "row_parts": 2}),
    (1, 14336, 4096, "gemv", {"k_splits": 1, "row_parts": 1}),
    (3, 14336, 4096, "gemv_rows", {}),
    (5, 1024, 8192, "gemv_rows_mfma", {"k_splits": 4}),  # the rows as an MFMA operand, quantize inside; few strips: K over four workgroups
    (8, 4096, 4096, "gemv_rows_mfma", {"k_splits": 2, "groups_per_wave": 1}),
    (16, 4096, 4096, "gemv_rows_mfma", {"k_splits": 2, "groups_per_wave": 1}),  # the sixteen-row form of the operand tile
    (13, 1024, 14336, "gemv_rows_mfma", {"k_splits": 8, "groups_per_wave": 1}),
    (4, 14336, 4096, "gemv_rows_mfma", {"k_splits": 1, "groups_per_wave": 2}),
    (8, 14336, 4096, "gemm_skinny", {"activation_strips": 1, "k_splits": 1}),
    (32, 4096, 14336, "gemm_skinny", {"activation_strips": 1, "k_splits": 2}),  # K over two workgroups per strip, arrival counter
    (128, 4096, 4096, "gemm_skinny", {"activation_strips": 2, "k_splits": 1}),  # more than 64 rows walked in groups of 64
    (64, 20480, 4096, "gemm_skinny", {"activation_strips": 2}),  # 160 column blocks whose K the tile kernel could not split
    (64, 14336, 4096, "gemm_tile_stream", {"activation_strips": 2, "k_sets": 4, "k_splits": 2}),
    (16, 8192, 8192, "gemm_tile_stream", {"activation_strips": 1, "k_sets": 4, "k_splits": 4}),
    (64, 4096, 14336, "gemm_tile_stream", {"activation_strips": 2, "k_sets": 4, "k_splits": 4}),
    (24, 24576, 1024, "gemm_tile_stream", {"activation_strips": 1, "k_splits": 1}),  # 192 column blocks: the tile kernel from seventeen rows on
    (512, 4096, 4096, "gemm_tile", {"activation_strips": 2, "k_sets": 4}),
    (128, 20480, 4096, "gemm_tile", {"activation_strips": 2, "k_sets": 2}),
    (512, 14336, 4096, "gemm_tile", {"activation_strips": 2, "k_sets": 1}),
    (70, 16384, 1024, "gemm_tile", {"activation_strips": 2}),  # a ragged last activation strip
]


@pytest.mark.parametrize("m,n,k,kernel,cut", ROUTES, ids=[f"{r[3]}-{r[0]}x{r[1]}x{r[2]}" for r in ROUTES])
def test_route_runs_and_matches_the_checker(q8, oracle, m, n, k, kernel, cut):
    plan = q8.plan_mul_mat(m, n, k)
    assert plan["kernel"] == kernel, plan
    for key, value in cut.items():
        assert plan[key] == value, (key, plan)
    w = oracle.fill_weights(1000 + m + n % 89, n, k)
    x = oracle.fill_activations(m + k, m * k).reshape(m, k)
    aq = oracle.quantize_rows(x)
    want = oracle.gemm(w, aq, m, n, k, threads=8)
    got = to_host(q8.mul_mat(q8.tile(to_dev(w), n, k), to_dev(x), n, k)).reshape(m, n)
    assert np.isfinite(got).all()
    assert rel_l2(got, want) <= REL_L2_TOL
    worst = max(rel_l2(got[i], want[i]) for i in range(m))  # row by row: a wrong row must not hide in the norm of the others
    assert worst <= REL_L2_TOL, worst

"""GPU: seeded random shapes through every mat-vec / small-M entry point, each result against the CPU checker.

The named tests pin the shapes of the benchmark configurations; this one walks the space between them (ragged row counts,
K from one group to 120, every cut the planner can choose: row parts, K splits, chunked walks, grouped launches of mixed
shapes, 2- and 3-row forms, the MFMA streaming kernel from M = 4) so that a shape-dependent mistake in a path the named
tests do not happen to take shows up here.  Seeds are fixed: a failure names its case and can be rerun.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def _shape(rng):
    n = int(rng.choice([rng.integers(1, 64), rng.integers(64, 700), rng.integers(700, 3000)]))
    k = 128 * int(rng.choice([rng.integers(1, 5), rng.integers(5, 40), rng.integers(40, 121)]))
    return n, k


def _want(oracle, w, x, n, k):
    aq = oracle.quantize_rows(np.ascontiguousarray(x.reshape(-1, k)))
    return oracle.gemm(w, aq, aq.shape[0], n, k)


@pytest.mark.parametrize("seed", range(12))
def test_random_single_and_residual_mat_vecs(q8, oracle, seed):
    rng = np.random.default_rng(1000 + seed)
    for case in range(4):
        n, k = _shape(rng)
        w = random_blocks(rng, n, k)
        x = rng.standard_normal(k).astype(np.float32)
        r = rng.standard_normal(n).astype(np.float32)
        wt = q8.tile(to_dev(w), n, k)
        want = _want(oracle, w, x, n, k)[0]
        assert rel_l2(to_host(q8.gemv_f32(wt, to_dev(x), n, k)), want) <= REL_L2_TOL, (seed, case, n, k)
        assert rel_l2(to_host(q8.gemv_residual_f32(wt, to_dev(x), to_dev(r), n, k)), want + r) <= REL_L2_TOL, (seed, case, n, k, "residual")
        xq = q8.quantize_row_q8_0(to_dev(x))
        assert rel_l2(to_host(q8.gemv(wt, xq, n, k, tiled=True)), want) <= REL_L2_TOL, (seed, case, n, k, "blocks in")


@pytest.mark.parametrize("seed", range(8))
def test_random_shared_x_and_grouped_launches(q8, oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    # up to three matrices that share x and K
    k = 128 * int(rng.integers(1, 60))
    ns = [int(rng.integers(1, 1500)) for _ in range(int(rng.integers(2, 4)))]
    ws = [random_blocks(rng, n, k) for n in ns]
    x = rng.standard_normal(k).astype(np.float32)
    ys = q8.gemv_f32([q8.tile(to_dev(w), n, k) for w, n in zip(ws, ns)], to_dev(x), ns, k)
    for i, (w, n) in enumerate(zip(ws, ns)):
        assert rel_l2(to_host(ys[i]), _want(oracle, w, x, n, k)[0]) <= REL_L2_TOL, (seed, "shared", i, n, k)
    # two to eleven independent ones of unrelated shapes
    shapes = [_shape(rng) for _ in range(int(rng.integers(2, 12)))]
    ws = [random_blocks(rng, n, k) for n, k in shapes]
    xs = [rng.standard_normal(k).astype(np.float32) for _, k in shapes]
    rs = [rng.standard_normal(n).astype(np.float32) if rng.integers(0, 2) else None for n, _ in shapes]
    ys = q8.gemv_group_f32([q8.tile(to_dev(w), n, k) for w, (n, k) in zip(ws, shapes)], [to_dev(x) for x in xs], [n for n, _ in shapes], [k for _, k in shapes],
                           residuals=[None if r is None else to_dev(r) for r in rs])
    for i, (n, k) in enumerate(shapes):
        want = _want(oracle, ws[i], xs[i], n, k)[0] + (0 if rs[i] is None else rs[i])
        assert rel_l2(to_host(ys[i]), want) <= REL_L2_TOL, (seed, "group", i, n, k)


@pytest.mark.parametrize("seed", range(8))
def test_random_small_m_mul_mat(q8, oracle, seed):
    rng = np.random.default_rng(3000 + seed)
    for case in range(3):
        n, k = _shape(rng)
        m = int(rng.choice([2, 3, 4, 5, 8, 17, 33, 64, 70]))
        w = random_blocks(rng, n, k)
        x = rng.standard_normal((m, k)).astype(np.float32)
        r = rng.standard_normal((m, n)).astype(np.float32)
        wt = q8.tile(to_dev(w), n, k)
        want = _want(oracle, w, x, n, k)
        assert rel_l2(to_host(q8.mul_mat(wt, to_dev(x), n, k)), want) <= REL_L2_TOL, (seed, case, m, n, k)
        assert rel_l2(to_host(q8.mul_mat(wt, to_dev(x), n, k, residual=to_dev(r))), want + r) <= REL_L2_TOL, (seed, case, m, n, k, "residual")

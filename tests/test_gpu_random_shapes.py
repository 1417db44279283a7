"""GPU: seeded random shapes through every mat-vec / small-M entry point, each result against the CPU checker.

The named tests pin the shapes of the benchmark configurations; this one walks the space between them (ragged row counts,
K from one group to 299, every cut the planner can choose: row parts, K splits, chunked walks, grouped launches of mixed
shapes, 2- and 3-row forms, the MFMA streaming kernel from M = 4) so that a shape-dependent mistake in a path the named
tests do not happen to take shows up here.  Seeds are fixed: a failure names its case and can be rerun.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def _shape(rng):
    n = int(rng.choice([rng.integers(1, 64), rng.integers(64, 700), rng.integers(700, 3000)]))
    k = 128 * int(rng.choice([rng.integers(1, 5), rng.integers(5, 40), rng.integers(40, 121), rng.integers(121, 300)]))
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
        nw = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        want_n = oracle.gemv(w, oracle.rms_norm_quantize_rows(x[None, :], nw, 1e-5)[0], n, k)
        assert rel_l2(to_host(q8.gemv_f32(wt, to_dev(x), n, k, norm_weight=to_dev(nw), eps=1e-5)), want_n) <= REL_L2_TOL, (seed, case, n, k, "norm inside")


def test_norm_inside_with_waves_of_unequal_group_counts(q8, oracle):
    # K = 5120 is 40 groups: in an unsplit launch eight waves own three and eight own two, in the four-group kernel variant.
    # The quantizer's wait for the activation slice must name a register that a load fills for every count
    # (a wave with two groups has none in the upper half of the slice registers).
    rng = np.random.default_rng(77)
    for n, k in ((8192, 5120), (600, 5120), (3000, 2560 + 128)):
        w = random_blocks(rng, n, k)
        x = rng.standard_normal(k).astype(np.float32)
        nw = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
        wt = q8.tile(to_dev(w), n, k)
        want = oracle.gemv(w, oracle.rms_norm_quantize_rows(x[None, :], nw, 1e-5)[0], n, k)
        for rep in range(3):
            assert rel_l2(to_host(q8.gemv_f32(wt, to_dev(x), n, k, norm_weight=to_dev(nw), eps=1e-5)), want) <= REL_L2_TOL, (n, k, rep)


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


@pytest.mark.parametrize("seed", range(8))
def test_random_one_launch_ffn(q8, oracle, seed):
    # the stages of the one-launch FFN against the checker: gate / up from the launch's own inspection copies, the down stage
    # re-derived from them (so its activation quantize is checked bit for bit in effect), with and without norm and residual
    rng = np.random.default_rng(4000 + seed)
    n_ff = 128 * int(rng.choice([rng.integers(1, 9), rng.integers(9, 60)]))
    k = 128 * int(rng.choice([rng.integers(1, 9), rng.integers(9, 48)]))
    n_out = int(rng.choice([rng.integers(1, 100), rng.integers(100, 2500)]))
    sg, sd = 1.0 / (58.0 * np.sqrt(k)), 1.0 / (58.0 * np.sqrt(n_ff))
    wg, wu, wd = random_blocks(rng, n_ff, k, sg), random_blocks(rng, n_ff, k, sg), random_blocks(rng, n_out, n_ff, sd)
    wg_t, wu_t, wd_t = (q8.tile(to_dev(w), r, c) for w, r, c in ((wg, n_ff, k), (wu, n_ff, k), (wd, n_out, n_ff)))
    x = rng.standard_normal(k).astype(np.float32)
    res = rng.standard_normal(n_out).astype(np.float32)
    nw = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    for use_norm, use_res in ((False, False), (True, True)):
        y = q8.ffn(wg_t, wu_t, wd_t, to_dev(x), n_ff, k, n_out, residual=to_dev(res) if use_res else None, norm_weight=to_dev(nw) if use_norm else None, eps=1e-5)
        g, u = (to_host(t) for t in q8.debug_ffn_gate_up(n_ff))
        xq = oracle.rms_norm_quantize_rows(x[None, :], nw, 1e-5)[0] if use_norm else oracle.quantize_rows(x[None, :])[0]
        tag = (seed, n_ff, k, n_out, use_norm)
        assert rel_l2(g, oracle.gemv(wg, xq, n_ff, k)) <= REL_L2_TOL and rel_l2(u, oracle.gemv(wu, xq, n_ff, k)) <= REL_L2_TOL, tag
        want = oracle.gemv(wd, oracle.silu_mul_quantize_rows(g, u)[0], n_out, n_ff) + (res if use_res else 0)
        assert rel_l2(to_host(y), want) <= REL_L2_TOL, tag


@pytest.mark.parametrize("seed", range(8))
def test_random_prefill_path(q8, oracle, seed):
    # quantizers bit for bit (blocks and tiled), then the mat-mat on the tile kernel's side of the routing (M > 64) and
    # the raw-blocks twin, with ragged M and N
    rng = np.random.default_rng(5000 + seed)
    m = int(rng.choice([rng.integers(65, 130), rng.integers(130, 400)]))
    n = int(rng.choice([rng.integers(1, 200), rng.integers(200, 2500)]))
    k = 128 * int(rng.choice([rng.integers(1, 6), rng.integers(6, 33)]))
    w = random_blocks(rng, n, k)
    x = (rng.standard_normal((m, k)) * rng.choice([1e-3, 1.0, 300.0])).astype(np.float32)
    tag = (seed, m, n, k)
    aq_cpu = oracle.quantize_rows(x)
    aq = q8.quantize_row_q8_0(to_dev(x))
    assert np.array_equal(to_host(aq).reshape(m, -1), aq_cpu), tag
    aq_t = q8.quantize_row_q8_0(to_dev(x), tiled=True)
    assert np.array_equal(to_host(q8.untile(aq_t, m, k)).reshape(m, -1), aq_cpu), tag
    nw = (1.0 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    an_t = q8.rms_norm_quantize(to_dev(x), to_dev(nw), 1e-5, tiled=True)
    assert np.array_equal(to_host(q8.untile(an_t, m, k)).reshape(m, -1), oracle.rms_norm_quantize_rows(x, nw, 1e-5)), tag
    g, u = rng.standard_normal((m, k)).astype(np.float32) * 3, rng.standard_normal((m, k)).astype(np.float32)
    as_t = q8.silu_mul_quantize(to_dev(g), to_dev(u), tiled=True)
    assert np.array_equal(to_host(q8.untile(as_t, m, k)).reshape(m, -1), oracle.silu_mul_quantize_rows(g, u)), tag
    want = oracle.gemm(w, aq_cpu, m, n, k, threads=4) if (k // 32) % 16 == 0 else oracle.gemm(w, aq_cpu, m, n, k)
    wt = q8.tile(to_dev(w), n, k)
    r = rng.standard_normal((m, n)).astype(np.float32)
    assert rel_l2(to_host(q8.gemm(wt, aq_t, m, n, k, tiled=True)), want) <= REL_L2_TOL, tag
    assert rel_l2(to_host(q8.gemm_residual(wt, aq_t, to_dev(r), m, n, k)), want + r) <= REL_L2_TOL, tag
    assert rel_l2(to_host(q8.gemm(to_dev(w), aq, m, n, k, tiled=False)), want) <= REL_L2_TOL, tag
    assert rel_l2(to_host(q8.mul_mat(wt, to_dev(x), n, k)), want) <= REL_L2_TOL, tag
    # token rows out of the same matrix, some ids out of range
    ids = rng.integers(-2, n + 2, size=37).astype(np.int32)
    got = q8.get_rows(wt, to_dev(ids), n, k, tiled=True)
    want_rows = oracle.get_rows(w, ids, n, k)[0]
    assert np.array_equal(to_host(got), want_rows), tag


@pytest.mark.parametrize("seed", range(8))
def test_random_blocks_layout_and_block_sums(q8, oracle, seed):
    # the reference's packed blocks as they come (K any multiple of 32): quantize, mat-vec, mat-mat, get_rows; and the int32
    # block sums of all four kernel families, bit for bit
    rng = np.random.default_rng(6000 + seed)
    n = int(rng.choice([rng.integers(1, 40), rng.integers(40, 900)]))
    k = 32 * int(rng.choice([rng.integers(1, 9), rng.integers(9, 200)]))
    m = int(rng.choice([1, 2, 7, 33, 90]))
    tag = (seed, m, n, k)
    w = random_blocks(rng, n, k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    aq_cpu = oracle.quantize_rows(x)
    aq = q8.quantize_row_q8_0(to_dev(x))
    assert np.array_equal(to_host(aq).reshape(m, -1), aq_cpu), tag
    want = oracle.gemm(w, aq_cpu, m, n, k)
    wd = to_dev(w)
    assert rel_l2(to_host(q8.gemv(wd, aq.reshape(m, -1)[0].contiguous(), n, k, tiled=False)), want[0]) <= REL_L2_TOL, tag
    assert rel_l2(to_host(q8.gemm(wd, aq, m, n, k, tiled=False)), want) <= REL_L2_TOL, tag
    sums = np.stack([oracle.block_sums_gemv(w, aq_cpu[i], n, k) for i in range(m)])
    assert np.array_equal(to_host(q8.debug_block_sums(wd, aq.reshape(m, -1)[0].contiguous(), 1, n, k, path=0))[0], sums[0]), tag
    assert np.array_equal(to_host(q8.debug_block_sums(wd, aq, m, n, k, path=1)), sums), tag
    ids = rng.integers(0, n, size=11).astype(np.int32)
    assert np.array_equal(to_host(q8.get_rows(wd, to_dev(ids), n, k, tiled=False)), oracle.get_rows(w, ids, n, k)[0]), tag
    if k % 128 == 0:
        wt = q8.tile(wd, n, k)
        assert np.array_equal(to_host(q8.debug_block_sums(wt, aq.reshape(m, -1)[0].contiguous(), 1, n, k, path=2))[0], sums[0]), tag
        assert np.array_equal(to_host(q8.debug_block_sums(wt, q8.tile(aq, m, k), m, n, k, path=3)), sums), tag

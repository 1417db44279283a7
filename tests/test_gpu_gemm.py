"""GPU parity: prefill int8-MFMA mat-mat vs the CPU restatement."""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def _inputs(oracle, m, n, k, seed):
    w = oracle.fill_weights(seed, n, k)
    x = oracle.fill_activations(seed, m * k).reshape(m, k)
    return w, x, oracle.quantize_rows(x)


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (512, 14336, 4096), (128, 14336, 4096), (32, 128, 128), (1, 128, 128), (8, 96, 256), (33, 65, 384), (130, 257, 512), (64, 4096, 14336), (75, 1100, 4096), (75, 1100, 2048), (20, 1000, 4096), (40, 4100, 12288), (20, 8200, 8192), (64, 8192, 8192)])
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


@pytest.mark.parametrize("m,n,k", [(512, 4096, 4096), (40, 512, 1024), (16, 2048, 14336), (64, 4096, 4096), (130, 257, 512), (8, 96, 256), (256, 14336, 4096), (75, 1100, 4096), (75, 1100, 2048), (20, 1000, 4096), (40, 4100, 12288), (20, 8200, 8192), (64, 4096, 14336)])
def test_gemm_residual(q8, oracle, m, n, k):
    # C = W . Aq + residual: exactly one fp32 add per element after its sum, in the MFMA tile kernel (one and two row strips, K
    # sets) and in the streaming kernel (one and two row strips, K split over workgroups), also in place
    w, x, aq = _inputs(oracle, m, n, k, seed=m * 7 + n)
    res = oracle.fill_activations(m + n, m * n).reshape(m, n)
    wt, at = q8.tile(to_dev(w), n, k), q8.tile(to_dev(aq.reshape(-1)), m, k)
    plain = to_host(q8.gemm(wt, at, m, n, k, tiled=True))
    got = to_host(q8.gemm_residual(wt, at, to_dev(res), m, n, k))
    assert np.array_equal(got, plain + res)
    acc = to_dev(res.copy())
    q8.gemm_residual(wt, at, acc, m, n, k, out=acc)
    assert np.array_equal(to_host(acc), got)


def test_mul_mat_residual_every_row_count(q8, oracle):
    # y = mul_mat(W, x) + residual through one entry point whatever M picks underneath: mat-vec, 2- and 3-row form, streaming and
    # tile mat-mat; one fp32 add per element after its sum
    n, k = 384, 1024
    w = oracle.fill_weights(3, n, k)
    wt = q8.tile(to_dev(w), n, k)
    for m in (1, 2, 3, 4, 40, 200):
        x = to_dev(oracle.fill_activations(m, m * k).reshape(m, k))
        res = oracle.fill_activations(100 + m, m * n).reshape(m, n)
        plain = to_host(q8.mul_mat(wt, x, n, k)).reshape(m, n)
        got = to_host(q8.mul_mat(wt, x, n, k, residual=to_dev(res))).reshape(m, n)
        assert np.array_equal(got, plain + res), m


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


@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 14336), (14336, 4096), (33, 128), (100, 1024), (8192, 28672), (1024, 8192), (1024, 4096), (512, 2048), (40000, 8192), (64, 128 * 70)])
def test_mul_mat_few_rows(q8, oracle, n, k):
    # 2 or 3 activation rows: the streaming mat-vec with one dot product per row and weight tile, quantize inside the kernel
    # (unsplit, K split over workgroups, chunked walk, ragged N); no workspace is needed there.  4 and 5 rows: the same kernel on
    # matrices up to 40 MB, quantize + the MFMA kernel on larger ones.  6 rows: the MFMA kernel.
    w = oracle.fill_weights(n + k, n, k)
    wt = q8.tile(to_dev(w), n, k)
    for m in (2, 3, 4, 5, 6):
        assert (q8._lib.lib().nh_q8_0_mul_mat_workspace_bytes(m, k) == 0) == (m <= 3)
        x = oracle.fill_activations(m + n, m * k).reshape(m, k)
        if m == 3:
            x[1] = 0.0  # an all-zero row: d = 0, every quant 0
            x[2, ::2] *= 1e-3
        aq = oracle.quantize_rows(x)
        want = oracle.gemm(w, aq, m, n, k, threads=8) if (k // 32) % 16 == 0 else oracle.gemm(w, aq, m, n, k)
        got = to_host(q8.mul_mat(wt, to_dev(x), n, k))
        assert got.shape == (m, n)
        for i in range(m):
            assert rel_l2(got[i], want[i]) <= REL_L2_TOL, (m, i)
        # each row is the mat-vec of that row: same kernel family, same fixed order -> same bits when the K cut is the same
        y0 = to_host(q8.gemv_f32(wt, to_dev(x[0]), n, k))
        assert rel_l2(got[0], y0) < 2e-6


@pytest.mark.parametrize("m,n,k", [(6, 24577, 256), (33, 24640, 384), (64, 24576 + 96, 128), (40, 30000, 640)])
def test_few_rows_on_a_wide_matrix(q8, oracle, m, n, k):
    # >= 192 column blocks of 128 rows: the tile kernel takes the batched-decode shapes too (activation tiles shared through
    # LDS, weight loads that bypass the caches); ragged N (a last column block with one to three strips, a last strip with
    # one row), one and two activation strips with padding rows, K sets of one, two and four groups, integer sums and fp32
    w, x, aq = _inputs(oracle, m, n, k, seed=m + n)
    wt, aqt = q8.tile(to_dev(w), n, k), q8.tile(to_dev(aq.reshape(-1)), m, k)
    sums = to_host(q8.debug_block_sums(wt, aqt, m, n, k, path=3))
    for i in range(m):
        assert np.array_equal(sums[i], oracle.block_sums_gemv(w, aq[i], n, k)), i
    got = to_host(q8.gemm(wt, aqt, m, n, k, tiled=True))
    assert rel_l2(got, oracle.gemm(w, aq, m, n, k)) <= REL_L2_TOL
    for i in range(m):
        assert rel_l2(got[i], oracle.gemv(w, aq[i], n, k)) <= REL_L2_TOL, i
    res = oracle.fill_activations(7, m * n).reshape(m, n)
    got_r = to_host(q8.gemm_residual(wt, aqt, to_dev(res), m, n, k))
    assert np.array_equal(got_r, got + res)


def test_mul_mat_batch_mixed_rows(q8, oracle):
    # one native call, seven projections: two mat-vecs sharing x (one launch), a 3-row op and two 8-row ops with no workspace use (the
    # quantize happens inside their kernels), two 24-row ops sharing the quantized x in the workspace
    import torch

    from nihilus_amd import _lib

    k, shapes = 1024, [(1, 256), (1, 96), (3, 160), (8, 256), (8, 64), (24, 256), (24, 64)]
    x1 = oracle.fill_activations(1, k).reshape(1, k)
    x3 = oracle.fill_activations(3, 3 * k).reshape(3, k)
    x8 = oracle.fill_activations(8, 8 * k).reshape(8, k)
    x24 = oracle.fill_activations(24, 24 * k).reshape(24, k)
    xs = {1: x1, 3: x3, 8: x8, 24: x24}
    xd = {m: to_dev(v) for m, v in xs.items()}
    ops = (_lib.MulMatOp * len(shapes))()
    keep, want = [], []
    for i, (m, n) in enumerate(shapes):
        w = oracle.fill_weights(40 + i, n, k)
        wt = q8.tile(to_dev(w), n, k)
        y = torch.full((m, n), float("nan"), dtype=torch.float32, device="cuda")
        keep += [wt, y]
        ops[i] = _lib.MulMatOp(wt.data_ptr(), xd[m].data_ptr(), y.data_ptr(), m, n, k, 1 if i in (1, 4, 6) else 0, 0)
        want.append(oracle.gemm(w, oracle.quantize_rows(xs[m]), m, n, k, threads=4))
    need = q8._lib.lib().nh_q8_0_mul_mat_workspace_bytes(24, k)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    assert [q8.plan_mul_mat(m, n, k)["quantize_launch"] for m, n in shapes] == [False] * 5 + [True] * 2
    _lib.check("nh_q8_0_mul_mat_batch", q8._lib.lib().nh_q8_0_mul_mat_batch(ops, len(shapes), ws.data_ptr(), need, torch.cuda.current_stream().cuda_stream))
    for i in range(len(shapes)):
        assert rel_l2(to_host(keep[2 * i + 1]), want[i]) <= REL_L2_TOL, i


def test_gemm_extreme_quants(q8, oracle):
    m, n, k = 32, 32, 128
    nb = k // 32
    one = np.float16(1.0).view(np.uint16)
    a = oracle.pack_blocks(np.full(m * nb, one), np.full((m, k), -127, dtype=np.int8))
    w = oracle.pack_blocks(np.full(n * nb, one), np.full((n, k), 127, dtype=np.int8))
    c = to_host(q8.gemm(to_dev(w), to_dev(a), m, n, k, tiled=False))
    assert np.array_equal(c, np.full((m, n), -127.0 * 127.0 * k, dtype=np.float32))

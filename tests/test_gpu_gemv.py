"""GPU parity: decode mat-vec vs the CPU restatement.

int32 block sums bit-exact; fp32 y within 1e-4 relative L2 of vec_dot_q8_0_q8_0<K/32> in the reference's
summation order (the GPU sums in a different order).
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

SHAPES = [(4096, 4096), (14336, 4096), (4096, 14336), (1024, 4096), (128256, 4096), (96, 512), (33, 128), (1, 128), (31, 256), (257, 8192), (8192, 28672), (1024, 8192), (100, 40960)]


def _inputs(oracle, n, k, seed):
    w = oracle.fill_weights(seed, n, k)
    x = oracle.fill_activations(seed, k)
    return w, x, oracle.quantize_rows(x)[0]


@pytest.mark.parametrize("n,k", SHAPES)
def test_gemv_tiled_and_blocks(q8, oracle, n, k):
    w, x, xq = _inputs(oracle, n, k, seed=n * 131 + k)
    want = oracle.gemv(w, xq, n, k)
    wd, xqd = to_dev(w), to_dev(xq)
    y_blocks = to_host(q8.gemv(wd, xqd, n, k, tiled=False))
    y_tiled = to_host(q8.gemv(q8.tile(wd, n, k), xqd, n, k, tiled=True))
    assert rel_l2(y_blocks, want) <= REL_L2_TOL
    assert rel_l2(y_tiled, want) <= REL_L2_TOL
    # the two kernels sum in different orders; they agree far inside the contract
    assert rel_l2(y_blocks, y_tiled) < 2e-6
    # far tighter than the contract in practice
    assert rel_l2(y_tiled, oracle.gemv_f64(w, xq, n, k)) < 5e-6


@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 14336), (96, 512), (33, 160), (5, 32), (64, 28672), (40, 128)])
def test_gemv_block_sums_exact(q8, oracle, n, k):
    w, x, xq = _inputs(oracle, n, k, seed=5)
    want = oracle.block_sums_gemv(w, xq, n, k)
    got = to_host(q8.debug_block_sums(to_dev(w), to_dev(xq), 1, n, k, path=0))[0]
    assert np.array_equal(got, want)
    if k % 128 == 0:  # the streaming kernel on the tiled layout
        got = to_host(q8.debug_block_sums(q8.tile(to_dev(w), n, k), to_dev(xq), 1, n, k, path=2))[0]
        assert np.array_equal(got, want)


def test_gemv_ragged_k_blocks_layout(q8, oracle):
    # K a multiple of 32 but not of 128: only the blocks layout takes it
    rng = np.random.default_rng(3)
    for n, k in [(40, 32), (40, 96), (7, 608)]:
        w = random_blocks(rng, n, k)
        xq = oracle.quantize_rows(rng.standard_normal(k).astype(np.float32))[0]
        got = to_host(q8.gemv(to_dev(w), to_dev(xq), n, k, tiled=False))
        assert rel_l2(got, oracle.gemv(w, xq, n, k)) <= REL_L2_TOL


def test_gemv_extreme_quants_and_unit_scales(q8, oracle):
    n, k = 64, 256
    nb = k // 32
    one = np.float16(1.0).view(np.uint16)
    # all +-127 against all 127, d = 1: y is an exact integer, 127*127*k (with sign)
    sign = np.where(np.arange(n) % 2 == 0, 127, -127).astype(np.int8)
    w = oracle.pack_blocks(np.full(n * nb, one), np.repeat(sign[:, None], k, axis=1))
    xq = oracle.pack_blocks(np.full(nb, one), np.full(k, 127, dtype=np.int8))
    y = to_host(q8.gemv(to_dev(w), to_dev(xq), n, k, tiled=False))
    assert np.array_equal(y, sign.astype(np.float32) * 127.0 * k)
    sums = to_host(q8.debug_block_sums(to_dev(w), to_dev(xq), 1, n, k, path=0))[0]
    assert np.array_equal(sums, np.repeat((sign.astype(np.int32) * 127 * 32)[:, None], nb, axis=1))


def test_gemv_errors(q8):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    w = torch.zeros(34 * 4 * 32, dtype=torch.uint8, device="cuda")
    xq = torch.zeros(34 * 4, dtype=torch.uint8, device="cuda")
    y = torch.full((32,), 7.0, dtype=torch.float32, device="cuda")
    assert lib.nh_q8_0_gemv(w.data_ptr(), xq.data_ptr(), y.data_ptr(), 0, 128, None) == 0
    assert lib.nh_q8_0_gemv(w.data_ptr(), xq.data_ptr(), y.data_ptr(), 32, 100, None) == -3
    assert lib.nh_q8_0_gemv_tiled(w.data_ptr(), xq.data_ptr(), y.data_ptr(), 32, 96, None) == -3
    assert lib.nh_q8_0_gemv(None, xq.data_ptr(), y.data_ptr(), 32, 128, None) == -1
    assert lib.nh_q8_0_gemv(w.data_ptr() + 2, xq.data_ptr(), y.data_ptr(), 32, 128, None) == -2
    assert lib.nh_q8_0_gemv(w.data_ptr(), xq.data_ptr(), y.data_ptr(), 32, 1 << 20, None) == -5  # blocks-layout mat-vec: K bounded by LDS
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())  # rejected calls wrote nothing
    assert lib.nh_q8_0_gemv(w.data_ptr(), xq.data_ptr(), y.data_ptr(), 32, 0, None) == 0  # empty dot product
    torch.cuda.synchronize()
    assert bool((y == 0.0).all())


def test_gemv_split_k_is_deterministic_and_reusable(q8, oracle):
    # few rows, long K: K is split over several workgroups whose partial sums are added by the last arriver in a
    # fixed order -- repeated launches must give identical bits, and the arrival counters must be left ready
    n, k = 4096, 14336
    w, x, xq = _inputs(oracle, n, k, seed=77)
    wt, xqd = q8.tile(to_dev(w), n, k), to_dev(xq)
    first = to_host(q8.gemv(wt, xqd, n, k, tiled=True))
    for _ in range(20):
        assert np.array_equal(to_host(q8.gemv(wt, xqd, n, k, tiled=True)), first)
    assert rel_l2(first, oracle.gemv(w, xq, n, k)) <= REL_L2_TOL


def test_split_k_back_to_back_with_changing_inputs(q8, oracle):
    # launches that share the K-split scratch queued without a sync in between, inputs alternating: a stale partial sum of
    # the previous launch must never be taken for a share of the current one (mat-vec, 3-row form, MFMA streaming kernel)
    import torch

    n, k = 2048, 14336
    w = oracle.fill_weights(5, n, k)
    wt = q8.tile(to_dev(w), n, k)
    xs = [to_dev(oracle.fill_activations(40 + i, 8 * k).reshape(8, k)) for i in range(2)]
    solo = []
    for x in xs:
        solo.append((to_host(q8.gemv_f32(wt, x[0], n, k)), to_host(q8.mul_mat(wt, x[:3], n, k)), to_host(q8.mul_mat(wt, x, n, k))))
        torch.cuda.synchronize()
    outs = []
    for i in range(12):
        x = xs[i & 1]
        outs.append((q8.gemv_f32(wt, x[0], n, k), q8.mul_mat(wt, x[:3], n, k), q8.mul_mat(wt, x, n, k)))
    torch.cuda.synchronize()
    for i, got in enumerate(outs):
        for g, want in zip(got, solo[i & 1]):
            assert np.array_equal(to_host(g), want), i


@pytest.mark.parametrize("k", [128, 4096, 14336, 28672, 512 * 128])
def test_fused_quantize_stage_is_bit_exact(q8, oracle, k):
    # the quantize inside the mat-vec kernel must stage exactly the bytes the stand-alone quantizer writes
    rng = np.random.default_rng(k)
    for x in (oracle.fill_activations(k, k), (rng.standard_normal(k) * 2.0 ** rng.integers(-30, 30, size=k)).astype(np.float32)):
        got = to_host(q8.debug_fused_quantize(to_dev(x)))
        assert np.array_equal(got, oracle.quantize_rows(x)[0])


@pytest.mark.parametrize("n,k", [(4096, 4096), (14336, 4096), (4096, 14336), (33, 128), (8192, 28672)])
def test_gemv_fused_f32_equals_two_step(q8, oracle, n, k):
    w, x, xq = _inputs(oracle, n, k, seed=n + 3 * k)
    wt = q8.tile(to_dev(w), n, k)
    fused = to_host(q8.gemv_f32(wt, to_dev(x), n, k))
    two_step = to_host(q8.gemv(wt, to_dev(xq), n, k, tiled=True))
    assert np.array_equal(fused, two_step)  # same staged bytes, same kernel, same order
    assert rel_l2(fused, oracle.gemv(w, xq, n, k)) <= REL_L2_TOL


@pytest.mark.parametrize("n,k", [(4096, 4096), (4096, 14336), (100, 1024), (33, 128), (128256, 4096)])
def test_gemv_residual(q8, oracle, n, k):
    # y = W . Q(x) + residual: exactly one fp32 add after the row's sum, in every form of the kernel (unsplit, row parts, K split),
    # and in place
    w, x, xq = _inputs(oracle, n, k, seed=n + 3 * k)
    res = oracle.fill_activations(n, n)
    wt, xd = q8.tile(to_dev(w), n, k), to_dev(x)
    plain = to_host(q8.gemv_f32(wt, xd, n, k))
    got = to_host(q8.gemv_residual_f32(wt, xd, to_dev(res), n, k))
    assert np.array_equal(got, plain + res)
    acc = to_dev(res.copy())
    q8.gemv_residual_f32(wt, xd, acc, n, k, out=acc)
    assert np.array_equal(to_host(acc), got)
    assert rel_l2(got, oracle.gemv(w, xq, n, k) + res) <= REL_L2_TOL


def test_gemv_multi_segment(q8, oracle):
    # q/k/v-shaped and gate/up-shaped groups as one launch each; results equal the single launches bit for bit
    for ns, k in [([4096, 1024, 1024], 4096), ([14336, 14336], 4096), ([40, 33, 1], 256), ([96], 128)]:
        x = oracle.fill_activations(9, k)
        ws = [oracle.fill_weights(50 + i, n, k) for i, n in enumerate(ns)]
        wts = [q8.tile(to_dev(w), n, k) for w, n in zip(ws, ns)]
        xd = to_dev(x)
        ys = q8.gemv_f32(wts, xd, ns, k)
        xq = oracle.quantize_rows(x)[0]
        for w, wt, n, y in zip(ws, wts, ns, ys):
            assert rel_l2(to_host(y), oracle.gemv(w, xq, n, k)) <= REL_L2_TOL
            if sum((m + 31) // 32 for m in ns) >= 256 or len(ns) == 1:  # same K split as the single launch
                assert np.array_equal(to_host(y), to_host(q8.gemv_f32(wt, xd, n, k)))


def test_gemv_long_k_many_rows_chunked_walk(q8, oracle):
    # many strips AND a K too long for one pass per wave: the kernel walks its K range in chunks
    n, k = 16416, 16384  # 513 strips (> split limit), 128 groups -> 8 groups per wave
    w, x, xq = _inputs(oracle, n, k, seed=4)
    wt = q8.tile(to_dev(w), n, k)
    want = oracle.gemm(w, xq[None, :], 1, n, k, threads=8)[0]
    assert rel_l2(to_host(q8.gemv(wt, to_dev(xq), n, k, tiled=True)), want) <= REL_L2_TOL
    assert rel_l2(to_host(q8.gemv_f32(wt, to_dev(x), n, k)), want) <= REL_L2_TOL

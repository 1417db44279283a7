"""GPU: every class of fp16 block scale READ on the device (reference conversion: cpu/common.hpp:215-221, vcvtph2ps, exact).

The other parity inputs draw scales from |N(0,1)| * 0.01 or 1.0, which never produces an fp16 subnormal or a value near the
top of the range.  A kernel that flushed subnormal halves (a float mode, or a matrix-pipe instruction that ignores the mode)
would pass them all.  Here the scales are the edge patterns themselves:

  * get_rows over a table whose block scales are all 63 488 finite fp16 bit patterns, both signs: bit-exact;
  * the v_dot4 mat-vec (blocks layout, tiled layout, tiled with the quantize inside) and the two MFMA kernels (streaming and
    tile form, whose scale product is a v_mfma_f32_32x32x8_f16 on the stored halves) with weight AND activation scales from
    {smallest subnormal, 2 x it, largest subnormal, smallest normal, the next one, largest finite, a typical value}.  Every
    weight row has ONE non-zero quant, so its output is a single product s * dW * dX: two 11-bit significands and a small
    integer, rounded once whatever the summation order.  The expectation is that closed form in float64 rounded to fp32,
    and the CPU checker must give the same bits.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, rel_l2, to_dev, to_host

gpu = pytest.mark.gpu  # one test below checks the construction itself and runs without a GPU

# fp16 bit patterns: 2^-24, 2^-23, largest subnormal, smallest normal, the next normal, 65504, ~0.0123
SCALE_CLASSES = np.array([0x0001, 0x0002, 0x03FF, 0x0400, 0x0401, 0x7BFF, 0x224C], dtype=np.uint16)
NC = len(SCALE_CLASSES)


def _f64(bits: np.ndarray) -> np.ndarray:
    return np.asarray(bits, dtype=np.uint16).view(np.float16).astype(np.float64)


@gpu
def test_get_rows_every_finite_fp16_scale(q8, oracle):
    finite = np.array([h for h in range(1 << 16) if (h >> 10) & 31 != 31], dtype=np.uint16)
    assert finite.size == 63488
    rng = np.random.default_rng(1)
    qs = rng.integers(-127, 128, size=(finite.size, 32), dtype=np.int8)
    qs[:, 0], qs[:, 1], qs[:, 2] = 1, -128, 127
    # independent expectation: numpy's float16 -> float32 (exact) times the quant, one fp32 multiply
    want = (finite.view(np.float16).astype(np.float32)[:, None] * qs.astype(np.float32)).astype(np.float32)
    for tiled, k in ((False, 32), (True, 128)):
        n_rows = finite.size * 32 // k
        w = oracle.pack_blocks(finite, qs)
        ids = np.arange(n_rows, dtype=np.int32)
        ref, bad = oracle.get_rows(w, ids, n_rows, k)
        assert bad == 0 and np.array_equal(ref.view(np.uint32), want.reshape(n_rows, k).view(np.uint32))
        wd = to_dev(w)
        if tiled:
            wd = q8.tile(wd, n_rows, k)
        got = to_host(q8.get_rows(wd, to_dev(ids), n_rows, k, tiled))
        assert np.array_equal(got.view(np.uint32), want.reshape(n_rows, k).view(np.uint32)), ("tiled" if tiled else "blocks")


def _one_hot_case(oracle, m, n, k, seed):
    """Weights [n x k]: row r has one non-zero quant (1, 2 or 3) in block r % nb, scale class (r // nb) % NC; every other block of
    the row is all-zero quants under an arbitrary class.  Activations [m x k]: block b of row i has scale class (b + i) % NC and
    quants in {-2, -1, 1, 2}.  Returns packed blocks and the closed-form fp32 outputs."""
    nb = k // 32
    rng = np.random.default_rng(seed)
    r = np.arange(n)
    w_d = SCALE_CLASSES[rng.integers(0, NC, size=(n, nb))]
    w_d[r, r % nb] = SCALE_CLASSES[(r // nb) % NC]
    w_q = np.zeros((n, nb, 32), dtype=np.int8)
    pos = rng.integers(0, 32, size=n)
    w_val = rng.integers(1, 4, size=n).astype(np.int8)
    w_q[r, r % nb, pos] = w_val
    a_cls = (np.arange(nb)[None, :] + np.arange(m)[:, None]) % NC
    a_d = SCALE_CLASSES[a_cls]
    a_q = rng.choice(np.array([-2, -1, 1, 2], dtype=np.int8), size=(m, nb, 32))
    s = w_val[None, :].astype(np.int64) * a_q[:, r % nb, pos].astype(np.int64)  # [m, n]: the one block sum that is not zero
    want = (s.astype(np.float64) * _f64(w_d[r, r % nb])[None, :] * _f64(a_d[:, r % nb])).astype(np.float32)
    assert np.all(np.isfinite(want)) and np.count_nonzero(want) == want.size  # nothing under- or overflows in fp32
    return oracle.pack_blocks(w_d, w_q), oracle.pack_blocks(a_d, a_q).reshape(m, -1), want


def test_one_hot_case_covers_every_scale_pair(oracle):
    # the construction reaches all NC x NC (weight class, activation class) pairs, and the CPU checker agrees with the closed form
    n, k = 7 * 8 * 2, 256
    w, aq, want = _one_hot_case(oracle, 1, n, k, seed=2)
    d_w, _ = oracle.split_blocks(w)
    d_a, _ = oracle.split_blocks(aq[0])
    nb = k // 32
    pairs = {(int(d_w.reshape(n, nb)[r, r % nb]), int(d_a[r % nb])) for r in range(n)}
    assert len(pairs) == NC * NC
    assert np.array_equal(oracle.gemv(w, aq[0], n, k).view(np.uint32), want[0].view(np.uint32))


@gpu
@pytest.mark.parametrize("n,k", [(112, 256), (4096, 4096), (4096, 14336), (160, 8192)])
def test_mat_vec_reads_extreme_scales(q8, oracle, n, k):
    # v_dot4 path: blocks layout, tiled layout (unsplit, row split, K split over workgroups)
    w, aq, want = _one_hot_case(oracle, 1, n, k, seed=n + k)
    assert np.array_equal(oracle.gemv(w, aq[0], n, k).view(np.uint32), want[0].view(np.uint32))
    wd, xd = to_dev(w), to_dev(aq[0])
    got_b = to_host(q8.gemv(wd, xd, n, k, tiled=False))
    got_t = to_host(q8.gemv(q8.tile(wd, n, k), xd, n, k, tiled=True))
    assert np.array_equal(got_b.view(np.uint32), want[0].view(np.uint32))
    assert np.array_equal(got_t.view(np.uint32), want[0].view(np.uint32))


@gpu
@pytest.mark.parametrize("n,k", [(112, 256), (4096, 4096), (4096, 14336)])
def test_fused_mat_vec_writes_and_reads_extreme_scales(q8, oracle, n, k):
    # quantize inside the mat-vec: activations built so that every block quantizes to a chosen edge scale (x = q * d with
    # the block's largest |q| = 127), then read back by the dot product
    nb = k // 32
    rng = np.random.default_rng(k)
    w, _, _ = _one_hot_case(oracle, 1, n, k, seed=n)
    cls = SCALE_CLASSES[np.arange(nb) % NC]
    q = rng.integers(-126, 127, size=(nb, 32)).astype(np.float64)
    q[np.arange(nb), rng.integers(0, 32, size=nb)] = 127.0
    x = (q * _f64(cls)[:, None]).astype(np.float32).reshape(k)
    xq = oracle.quantize_rows(x)[0]
    d_x, q_x = oracle.split_blocks(xq)
    assert np.array_equal(d_x, cls) and np.array_equal(q_x, q.astype(np.int8))  # the quantizer reproduces the construction
    want = oracle.gemv(w, xq, n, k)
    assert np.array_equal(to_host(q8.quantize_row_q8_0(to_dev(x)))[0], xq)
    got = to_host(q8.gemv_f32(q8.tile(to_dev(w), n, k), to_dev(x), n, k))
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))
    # the 2-row form of the same kernel
    got2 = to_host(q8.mul_mat(q8.tile(to_dev(w), n, k), to_dev(np.stack([x, -x])), n, k))
    assert np.array_equal(got2[0].view(np.uint32), want.view(np.uint32))
    assert np.array_equal(got2[1], -want)  # by value: a row whose one product is zero gives +0 for either sign of x


@gpu
@pytest.mark.parametrize("m,n,k", [(4, 112, 256), (16, 4096, 1024), (64, 2048, 4096), (40, 8192, 512), (512, 4096, 256), (512, 2176, 1024), (130, 14336, 512), (96, 257, 384)])
def test_mfma_kernels_read_extreme_scales(q8, oracle, m, n, k):
    # the scale product dA * dW comes from a v_mfma_f32_32x32x8_f16 on the halves as stored: streaming kernel (m <= 64 or a
    # small grid), tile kernel (one and two activation strips per wave, K sets), and the kernel on the packed-blocks layout
    w, aq, want = _one_hot_case(oracle, m, n, k, seed=m * 3 + n)
    wd, ad = to_dev(w), to_dev(aq.reshape(-1))
    got_b = to_host(q8.gemm(wd, ad, m, n, k, tiled=False))
    assert np.array_equal(got_b.view(np.uint32), want.view(np.uint32))
    if k % 128 == 0:
        got_t = to_host(q8.gemm(q8.tile(wd, n, k), q8.tile(ad, m, k), m, n, k, tiled=True))
        assert np.array_equal(got_t.view(np.uint32), want.view(np.uint32))
    for i in (0, m - 1):
        assert np.array_equal(oracle.gemv(w, aq[i], n, k).view(np.uint32), want[i].view(np.uint32))


@gpu
@pytest.mark.parametrize("m", [8, 32])
@pytest.mark.parametrize("n,k", [(4096, 4096), (14336, 4096)])
def test_crossover_rows_at_the_prefill_weights(q8, oracle, m, n, k):
    # the mat-vec -> mat-mat crossover points of the prefill configuration (M = 8 and 32 against W [4096 x 4096] and
    # [14336 x 4096], weights and activations from seed 0) through the fused entry point, against the CPU checker
    w = oracle.fill_weights(0, n, k)
    x = oracle.fill_activations(0, 512 * k).reshape(512, k)[:m]
    aq = oracle.quantize_rows(x)
    want = oracle.gemm(w, aq, m, n, k, threads=8)
    got = to_host(q8.mul_mat(q8.tile(to_dev(w), n, k), to_dev(x), n, k))
    assert rel_l2(got, want) <= REL_L2_TOL
    for i in range(m):
        assert rel_l2(got[i], want[i]) <= REL_L2_TOL, i

"""CPU: pins the checker's quantize, integer block dot and fp32 accumulation by what the arithmetic itself fixes:
closed forms, invariants, brute force, float64, special cases -- each chosen so a plausible slip (wrong sign,
dropped term, roundf instead of round-half-even, transposed operands) fails at least one."""
import numpy as np
import pytest

from helpers import random_blocks, rel_l2


def _numpy_quantize(x: np.ndarray) -> np.ndarray:
    """Independent evaluation of the same closed form with numpy fp32 arithmetic (np.rint is half-to-even)."""
    x = np.asarray(x, dtype=np.float32).reshape(-1, 32)
    amax = np.abs(x).max(axis=1)
    with np.errstate(divide="ignore", invalid="ignore", over="ignore"):
        d = (amax / np.float32(127.0)).astype(np.float32)
        inv = np.where(amax != 0, np.float32(127.0) / amax, np.float32(0.0)).astype(np.float32)
        q = np.rint((x * inv[:, None]).astype(np.float32))
    out = np.empty((x.shape[0], 34), dtype=np.uint8)
    dh = d.astype(np.float16).view(np.uint16)
    out[:, 0], out[:, 1] = dh & 0xFF, dh >> 8
    out[:, 2:] = q.astype(np.int8).view(np.uint8)
    return out.reshape(-1)


def test_quantize_matches_independent_numpy_form_and_avx2(oracle):
    rng = np.random.default_rng(1)
    for scale in (1.0, 1e-3, 37.0, 1e4):
        x = (rng.standard_normal((64, 4096)) * scale).astype(np.float32)
        got = oracle.quantize_rows(x)
        assert np.array_equal(got.reshape(-1), _numpy_quantize(x))
        assert np.array_equal(got, oracle.quantize_rows(x, avx2=True))


def test_quantize_invariants(oracle):
    rng = np.random.default_rng(2)
    x = rng.standard_normal((200, 32)).astype(np.float32)
    blk = oracle.quantize_rows(x)
    d, qs = oracle.split_blocks(blk)
    # the element of largest magnitude maps to +-127 with its sign
    j = np.abs(x).argmax(axis=1)
    assert np.array_equal(qs[np.arange(200), j], (np.sign(x[np.arange(200), j]) * 127).astype(np.int8))
    # d = fp16(amax / 127)
    assert np.array_equal(d, (np.abs(x).max(axis=1) / np.float32(127)).astype(np.float16).view(np.uint16))
    # odd symmetry: q(-x) = -q(x), same d
    d2, qs2 = oracle.split_blocks(oracle.quantize_rows(-x))
    assert np.array_equal(d2, d) and np.array_equal(qs2, -qs)
    # scaling by a power of two leaves q unchanged and scales d exactly
    for e in (-3, 7):  # d stays in the normal fp16 range
        d3, qs3 = oracle.split_blocks(oracle.quantize_rows(x * np.float32(2.0**e)))
        assert np.array_equal(qs3, qs)
        assert np.array_equal(d3.view(np.float16).astype(np.float32), d.view(np.float16).astype(np.float32) * np.float32(2.0**e))
    # all-zero block (and negative zeros): d = 0, q = 0
    z = oracle.quantize_rows(np.zeros((1, 64), dtype=np.float32))
    assert not z.any()
    assert not oracle.quantize_rows(np.full((1, 32), -0.0, dtype=np.float32)).any()


def test_quantize_ties_go_to_even(oracle):
    # amax = 127 makes id = 127/127 = 1 exactly, so x = j + 0.5 is an exact tie: half-to-even gives j or j+1,
    # whichever is even -- roundf (half away from zero) would give j+1 always.  The reference rounds with
    # _mm256_round_ps(NEAREST) (cpu/avx_2.hpp:4470-4473), i.e. to even.
    j = np.arange(31, dtype=np.float32)
    x = np.concatenate([[127.0], j + 0.5]).astype(np.float32)
    want = np.concatenate([[127], np.where(j % 2 == 0, j, j + 1)]).astype(np.int8)
    for sign in (1.0, -1.0):
        d, qs = oracle.split_blocks(oracle.quantize_rows((sign * x)[None, :]))
        assert np.array_equal(qs[0], (sign * want).astype(np.int8))
        assert d[0] == np.float16(1.0).view(np.uint16)
        d, qs = oracle.split_blocks(oracle.quantize_rows((sign * x)[None, :], avx2=True))
        assert np.array_equal(qs[0], (sign * want).astype(np.int8))


def test_quantize_ignores_ragged_tail_and_handles_edges(oracle):
    rng = np.random.default_rng(3)
    x = rng.standard_normal((3, 100)).astype(np.float32)
    full = oracle.quantize_rows(x, k=100)  # nb = k / 32 = 3: the last 4 values are dropped (cpu/avx_2.hpp:4440)
    assert full.shape == (3, 3 * 34)
    assert np.array_equal(full, oracle.quantize_rows(np.ascontiguousarray(x[:, :96])))
    assert oracle.quantize_rows(x, k=31).shape == (3, 0)
    # scale overflow / underflow edges of the fp16 scale
    big = np.full((1, 32), 70000.0 * 127, dtype=np.float32)
    d, qs = oracle.split_blocks(oracle.quantize_rows(big))
    assert d[0] == 0x7C00 and (qs == 127).all()  # d rounds to fp16 inf, quants are still +-127
    tiny = np.full((1, 32), 1e-12, dtype=np.float32)
    d, qs = oracle.split_blocks(oracle.quantize_rows(tiny))
    assert d[0] == 0 and (qs == 127).all()
    sub = np.full((1, 32), 1e-6, dtype=np.float32)  # d = 7.87e-9 -> fp16 subnormal range: kept, not flushed
    d, _ = oracle.split_blocks(oracle.quantize_rows(sub))
    assert d[0] == np.float32(1e-6 / 127).astype(np.float16).view(np.uint16) == 0  # below half the smallest subnormal
    sub = np.full((1, 32), 1e-4, dtype=np.float32)  # d = 7.87e-7: a proper fp16 subnormal
    d, _ = oracle.split_blocks(oracle.quantize_rows(sub))
    assert 0 < d[0] < 0x0400 and d[0] == (np.float32(1e-4) / np.float32(127)).astype(np.float16).view(np.uint16)
    # 127/amax overflowing to inf: inf and 0*inf = NaN both become -128, as x86 cvtps_epi32 + saturating packs do
    weird = np.concatenate([[1e-45], np.zeros(31)]).astype(np.float32)[None, :]
    _, qs = oracle.split_blocks(oracle.quantize_rows(weird))
    assert (qs == -128).all()
    assert np.array_equal(oracle.quantize_rows(weird), oracle.quantize_rows(weird, avx2=True))


# ------------------------------------------------------------------ integer block dot


def test_block_sums_brute_force_and_extremes(oracle):
    rng = np.random.default_rng(4)
    n, k = 37, 256
    w = random_blocks(rng, n, k)
    x = random_blocks(rng, 1, k)
    got = oracle.block_sums_gemv(w, x, n, k)
    _, wq = oracle.split_blocks(w)
    _, xq = oracle.split_blocks(x)
    want = (wq.reshape(n, k // 32, 32).astype(np.int64) * xq.reshape(1, k // 32, 32).astype(np.int64)).sum(axis=2)
    assert np.array_equal(got.astype(np.int64), want)
    one = np.float16(1).view(np.uint16)
    for a, b, s in ((127, 127, 516128), (-127, 127, -516128), (-127, -127, 516128), (-128, 127, -520192)):
        wa = oracle.pack_blocks([one], np.full(32, a, dtype=np.int8))
        xb = oracle.pack_blocks([one], np.full(32, b, dtype=np.int8))
        assert oracle.block_sums_gemv(wa, xb, 1, 32)[0, 0] == s
    # not symmetric-by-accident: a one-hot against a ramp picks out the right element
    ramp = np.arange(-16, 16, dtype=np.int8)
    for j in (0, 5, 31):
        hot = np.zeros(32, dtype=np.int8)
        hot[j] = 3
        assert oracle.block_sums_gemv(oracle.pack_blocks([one], hot), oracle.pack_blocks([one], ramp), 1, 32)[0, 0] == 3 * int(ramp[j])


# ------------------------------------------------------------------ fp32 accumulation


@pytest.mark.parametrize("nb", list(range(1, 40)) + [128, 448, 256, 896])
def test_vec_dot_all_branches_against_float64(oracle, nb):
    # every branch of vec_dot_q8_0_q8_0<n> (n<4 scalar, 4, 5..7, 8, 9..15, 16, >16 with and without remainder)
    rng = np.random.default_rng(nb)
    x, y = random_blocks(rng, 1, nb * 32), random_blocks(rng, 1, nb * 32, scale_sigma=1.0)
    ref = oracle.vec_dot_f64(nb, x, y)
    got = float(oracle.vec_dot(nb, x, y))
    rt = float(oracle.vec_dot_rt(nb * 32, x, y))
    scale = np.sqrt(nb) * 2.0e4 * 0.01  # typical magnitude of the sum; guards the ref == 0 case
    assert abs(got - ref) <= 2e-6 * max(abs(ref), scale)
    assert abs(rt - ref) <= 2e-6 * max(abs(ref), scale)
    if nb % 16 == 0:
        assert oracle.vec_dot_avx2(nb, x, y) == oracle.vec_dot(nb, x, y)  # same operations, same order: same bits


def test_vec_dot_unit_scales_give_exact_integers(oracle):
    rng = np.random.default_rng(6)
    one = np.float16(1).view(np.uint16)
    for nb in (1, 3, 4, 7, 8, 16, 23, 128):
        qa = rng.integers(-127, 128, size=nb * 32, dtype=np.int8)
        qb = rng.integers(-127, 128, size=nb * 32, dtype=np.int8)
        a, b = oracle.pack_blocks(np.full(nb, one), qa), oracle.pack_blocks(np.full(nb, one), qb)
        exact = int((qa.astype(np.int64) * qb.astype(np.int64)).sum())
        assert abs(exact) < 2**24
        assert float(oracle.vec_dot(nb, a, b)) == float(exact)
        assert float(oracle.vec_dot_rt(nb * 32, a, b)) == float(exact)


def test_vec_dot_tiny_hand_checked(oracle):
    # one block, d_x = 0.5, d_y = 2, quants x = [1,2,3,0...], y = [4,5,6,0...]: (4+10+18) * 0.5 * 2 = 32
    qx = np.zeros(32, dtype=np.int8)
    qy = np.zeros(32, dtype=np.int8)
    qx[:3], qy[:3] = [1, 2, 3], [4, 5, 6]
    x = oracle.pack_blocks([np.float16(0.5).view(np.uint16)], qx)
    y = oracle.pack_blocks([np.float16(2.0).view(np.uint16)], qy)
    assert float(oracle.vec_dot(1, x, y)) == 32.0
    # scales multiply per block, not once for the row: two blocks with different scales
    x2 = oracle.pack_blocks([np.float16(0.5).view(np.uint16), np.float16(4.0).view(np.uint16)], np.concatenate([qx, qx]))
    y2 = oracle.pack_blocks([np.float16(2.0).view(np.uint16), np.float16(0.25).view(np.uint16)], np.concatenate([qy, qy]))
    assert float(oracle.vec_dot(2, x2, y2)) == 32.0 + 32.0
    assert oracle.vec_dot_f64(2, x2, y2) == 64.0


def test_gemv_gemm_orientation_and_consistency(oracle):
    rng = np.random.default_rng(7)
    m, n, k = 5, 48, 512
    w = random_blocks(rng, n, k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    aq = oracle.quantize_rows(x)
    c = oracle.gemm(w, aq, m, n, k)
    assert c.shape == (m, n)
    for i in range(m):
        assert np.array_equal(c[i], oracle.gemv(w, aq[i], n, k))  # C[m][n]: n fastest, row m = activation row m
    assert np.array_equal(c, oracle.gemm(w, aq, m, n, k, threads=3))
    # against a dequantize-then-float64 product: both the weight row and the activation row are the right ones
    wd = np.stack([oracle.dequantize_row(w.reshape(n, -1)[j], k) for j in range(n)]).astype(np.float64)
    xd = np.stack([oracle.dequantize_row(aq[i], k) for i in range(m)]).astype(np.float64)
    assert rel_l2(c, xd @ wd.T) < 1e-6
    assert rel_l2(oracle.gemv_f64(w, aq[2], n, k), (xd @ wd.T)[2]) < 1e-12


def test_generator_statistics_and_determinism(oracle):
    w = oracle.fill_weights(0, 64, 4096)
    d, qs = oracle.split_blocks(w)
    assert qs.min() == -127 and qs.max() == 127 and abs(qs.astype(np.float64).mean()) < 0.5
    scales = d.view(np.float16).astype(np.float64)
    assert 0.0075 < scales.mean() < 0.0085  # E|N(0,1)| * 0.01 = 0.00798
    x = oracle.fill_activations(0, 1 << 16)
    assert abs(x.mean()) < 0.02 and 0.98 < x.std() < 1.02
    assert np.array_equal(w, oracle.fill_weights(0, 64, 4096))
    assert np.array_equal(oracle.fill_weights(0, 32, 4096, first_block=32 * 128), w[32 * 128 * 34 :])
    assert not np.array_equal(w, oracle.fill_weights(1, 64, 4096))


def test_division_by_127_through_the_rounded_reciprocal_is_exact(tmp_path):
    """The device quantizer's short route: amax / 127 as reciprocal multiply + one fma correction.  Checked on the host against the
    correctly rounded division for every fp32 mantissa (tests/cpp/divide_by_127_check.c)."""
    import os
    import subprocess

    src = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cpp", "divide_by_127_check.c")
    exe = str(tmp_path / "divide_by_127_check")
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-mfma", "-o", exe, src, "-lm"], check=True)
    res = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout
    assert "mismatches 0" in res.stdout

"""CPU: the checker's RMS norm (fixed-order sum of squares, IEEE sqrt and divide, then the norm weight) against what
fixes it.  The reference has no live body for rms_norm and its dead one calls an ISA-dependent sqrtf_fast
(cpu/avx_2.hpp:5331-5347, cpu/common.hpp:310/448), so nothing of it can be replayed: the scale and the normalised row are
pinned against float64, by exact invariances, and by rows whose answer is known in closed form."""
import numpy as np
import pytest


@pytest.mark.parametrize("k", [128, 384, 4096, 8192, 14336, 2176])
def test_scale_against_float64(oracle, k):
    rng = np.random.default_rng(k)
    x = (rng.standard_normal(k) * 3).astype(np.float32)
    for eps in (0.0, 1e-5, 1e-6):
        want = 1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2) + np.float64(np.float32(eps)))
        assert abs(oracle.rms_norm_scale(x, eps) - want) / want <= 3e-7


def test_scale_invariances_and_closed_forms(oracle):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(4096).astype(np.float32)
    s = oracle.rms_norm_scale(x, 0.0)
    for e in (-20, -3, 1, 7, 30):  # powers of two commute with every rounding on the way
        assert oracle.rms_norm_scale(np.ldexp(x, e), 0.0) == float(np.ldexp(np.float32(s), -e))
    assert oracle.rms_norm_scale(-x, 0.0) == s
    assert oracle.rms_norm_scale(x[::-1].copy(), 1e-5) != 0  # order matters only in the last bits
    assert abs(oracle.rms_norm_scale(x[::-1].copy(), 1e-5) - oracle.rms_norm_scale(x, 1e-5)) <= 2e-7 * s
    # constant rows: mean(x^2) = c^2 exactly when c^2 and the partial sums are exact
    assert oracle.rms_norm_scale(np.full(4096, 2.0, np.float32), 0.0) == 0.5
    assert oracle.rms_norm_scale(np.full(1024, 0.25, np.float32), 0.0) == 4.0
    assert oracle.rms_norm_scale(np.full(128 * 19, 0.5, np.float32), 0.0) == 2.0  # ragged cut: 3 runs of 2 groups, 13 of 1
    one = np.zeros(4096, np.float32)
    one[1234] = 64.0  # mean = 64^2 / 4096 = 1
    assert oracle.rms_norm_scale(one, 0.0) == 1.0
    assert oracle.rms_norm_scale(np.zeros(128, np.float32), 0.25) == 2.0  # 1 / sqrt(eps)
    # a dropped element changes the answer: every element takes part
    y = np.ones(8192, np.float32)
    y[8191] = 300.0
    assert oracle.rms_norm_scale(y, 0.0) < oracle.rms_norm_scale(np.ones(8192, np.float32), 0.0) * 0.5


def test_normalised_row_and_quantize_composition(oracle):
    rng = np.random.default_rng(2)
    k, m = 4096, 3
    x = (rng.standard_normal((m, k)) * 5).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    for r in range(m):
        y = oracle.rms_norm_mul(x[r], w, 1e-5)
        want = x[r].astype(np.float64) / np.sqrt(np.mean(x[r].astype(np.float64) ** 2) + 1e-5) * w
        assert np.abs(y - want).max() <= 4e-7 * np.abs(want).max()
        s = np.float32(oracle.rms_norm_scale(x[r], 1e-5))
        assert np.array_equal(y, (x[r] * s) * w)  # two separately rounded multiplies, in that order
    rows = np.stack([oracle.rms_norm_mul(x[r], w, 1e-5) for r in range(m)])
    assert np.array_equal(oracle.rms_norm_quantize_rows(x, w, 1e-5), oracle.quantize_rows(rows))

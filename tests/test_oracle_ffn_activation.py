"""CPU: the checker's FFN activation (fixed-sequence fp32 exp, SiLU(g) * u, quantize of that) against what fixes it.

The reference has no body for silu or mul (cpu/avx_2.hpp:1946-2075), so nothing of it can be replayed: the exp is
pinned against the correctly rounded double-precision value, the SiLU against its closed form in float64, and the
fused quantize against the composition of the already pinned parts.
"""
import numpy as np


def ulp_error(got: np.ndarray, ref64: np.ndarray) -> np.ndarray:
    ulp = np.spacing(np.abs(ref64).astype(np.float32)).astype(np.float64)
    return np.abs(got.astype(np.float64) - ref64) / ulp


def test_expf_within_two_ulp_over_the_clamped_range(oracle):
    x = np.concatenate([np.linspace(-87.0, 88.0, 400001), np.linspace(-1.0, 1.0, 100001), np.linspace(-1e-3, 1e-3, 2001)]).astype(np.float32)
    err = ulp_error(oracle.expf(x), np.exp(x.astype(np.float64)))
    assert err.max() <= 2.0, (err.max(), x[err.argmax()])


def test_expf_special_points(oracle):
    e = oracle.expf(np.array([0.0, -0.0, 1.0, -1.0, 88.0, -87.0, 1000.0, -1000.0, np.log(2.0)], dtype=np.float32))
    assert e[0] == 1.0 and e[1] == 1.0
    assert abs(float(e[2]) - np.e) <= 2 * np.spacing(np.float32(np.e))
    assert abs(float(e[3]) - 1 / np.e) <= 2 * np.spacing(np.float32(1 / np.e))
    assert e[6] == e[4] and e[7] == e[5]  # clamped, finite, normal
    assert np.isfinite(e).all() and (e >= np.finfo(np.float32).tiny).all()
    assert abs(float(e[8]) - 2.0) <= 2 * np.spacing(np.float32(2.0))
    # monotone over a fine sweep around a reduction boundary (n changes at x = 0.5 * ln 2)
    x = np.linspace(0.3465, 0.3467, 2001).astype(np.float32)
    y = oracle.expf(x)
    assert (np.diff(y) >= 0).all()


def test_silu_mul_closed_form(oracle):
    rng = np.random.default_rng(0)
    g = np.concatenate([rng.standard_normal(20000) * 4, [0.0, 30.0, -30.0, 100.0, -100.0, 1e-20, -1e-20]]).astype(np.float32)
    u = np.concatenate([rng.standard_normal(20000) * 2, [3.0, 2.0, 2.0, 1.0, 1.0, 5.0, 5.0]]).astype(np.float32)
    got = oracle.silu_mul(g, u).astype(np.float64)
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64
    big = np.abs(g) <= 80  # beyond the clamp the value is below 1e-30 in magnitude either way
    rel = np.abs(got[big] - want[big]) / np.maximum(np.abs(want[big]), 1e-30)
    assert rel.max() <= 4e-7, rel.max()
    assert np.all(np.abs(got[~big] - want[~big]) <= 1e-30 + 1e-6 * np.abs(want[~big]))
    assert oracle.silu_mul(np.float32([0.0]), np.float32([7.0]))[0] == 0.0
    assert oracle.silu_mul(np.float32([100.0]), np.float32([1.0]))[0] == 100.0  # 1 + exp(-100) rounds to 1


def test_silu_mul_quantize_is_the_composition(oracle):
    rng = np.random.default_rng(1)
    m, k = 5, 256
    g = (rng.standard_normal((m, k)) * 3).astype(np.float32)
    u = (rng.standard_normal((m, k)) * 2).astype(np.float32)
    act = oracle.silu_mul(g, u).reshape(m, k)
    assert np.array_equal(oracle.silu_mul_quantize_rows(g, u), oracle.quantize_rows(act))

"""GPU: SiLU(gate) * up fused into the quantizer, byte-exact against the CPU checker (same fixed-sequence exp)."""
import numpy as np
import pytest

from helpers import to_dev, to_host

pytestmark = pytest.mark.gpu


def inputs(seed, m, k, scale):
    rng = np.random.default_rng(seed)
    g = (rng.standard_normal((m, k)) * scale).astype(np.float32)
    u = (rng.standard_normal((m, k)) * 2).astype(np.float32)
    return g, u


@pytest.mark.parametrize("m,k,scale", [(1, 128, 3.0), (1, 14336, 3.0), (7, 4096, 1.0), (33, 256, 30.0), (512, 1024, 5.0)])
def test_silu_mul_quantize_bit_exact(q8, oracle, m, k, scale):
    g, u = inputs(m + k, m, k, scale)
    g[0, :8] = [0.0, -0.0, 100.0, -100.0, 87.5, -87.5, 1e-30, -1e-30]
    want = oracle.silu_mul_quantize_rows(g, u)
    got = to_host(q8.silu_mul_quantize(to_dev(g), to_dev(u)))
    assert np.array_equal(got, want)
    tiled = q8.silu_mul_quantize(to_dev(g), to_dev(u), tiled=True)
    assert np.array_equal(to_host(q8.untile(tiled, m, k)).reshape(m, -1), want)


def test_silu_mul_quantize_whole_exponent_range(q8, oracle):
    # gate values sweeping every binade where exp(-g) matters, and the clamp edges
    g = np.concatenate([np.linspace(-90, 90, 4096 - 64), np.ldexp(1.0, np.arange(-40, 24))]).astype(np.float32).reshape(1, 4096)
    u = np.ones_like(g)
    assert np.array_equal(to_host(q8.silu_mul_quantize(to_dev(g), to_dev(u))), oracle.silu_mul_quantize_rows(g, u))


def test_silu_mul_quantize_errors(q8):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    g = torch.zeros(128, dtype=torch.float32, device="cuda")
    out = torch.zeros(4 * 34, dtype=torch.uint8, device="cuda")
    assert lib.nh_q8_0_silu_mul_quantize(g.data_ptr(), g.data_ptr(), out.data_ptr(), 1, 100, None) == -3
    assert lib.nh_q8_0_silu_mul_quantize_tiled(g.data_ptr(), g.data_ptr(), out.data_ptr(), 1, 96, None) == -3
    assert lib.nh_q8_0_silu_mul_quantize(None, g.data_ptr(), out.data_ptr(), 1, 128, None) == -1
    assert lib.nh_q8_0_silu_mul_quantize(g.data_ptr(), g.data_ptr() + 4, out.data_ptr(), 1, 96, None) == -2
    assert lib.nh_q8_0_silu_mul_quantize(g.data_ptr(), g.data_ptr(), out.data_ptr(), 0, 128, None) == 0

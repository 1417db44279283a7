"""GPU: the fp32-activation mul_mat (no activation quantize) through the C ABI against the checker's restatement of the
reference's two leaves (eval_time order for one row, prompt_eval_time order for several), fp32 contract 1e-4 relative L2."""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (1, 1000, 14336), (1, 33, 128), (3, 257, 1024), (40, 96, 512), (2, 14336, 4096), (1, 64, 0), (2, 160, 5120), (1, 96, 8192), (1, 64, 28672), (1, 40, 4224), (2, 96, 14336), (3, 64, 28672)])
def test_matches_checker(q8, oracle, m, n, k):
    rng = np.random.default_rng(m + n + k)
    w = random_blocks(rng, n, k) if k else np.zeros(0, dtype=np.uint8)
    x = rng.standard_normal((m, k)).astype(np.float32)
    got = to_host(q8.mul_mat_f32_activations(q8.tile(to_dev(w), n, k), to_dev(x), n, k))
    if k == 0:
        assert got.shape == (m, n) and (got == 0).all()
        return
    want = oracle.mul_mat_f32_activations(w, x, n, k, prompt_order=m > 1)
    assert rel_l2(got, want) <= REL_L2_TOL
    assert rel_l2(got, oracle.mul_mat_f32_activations_f64(w, x, n, k)) < 2e-6


def test_unit_scales_and_integer_activations_are_exact(q8, oracle):
    rng = np.random.default_rng(3)
    n, k = 100, 1024
    one = np.float16(1.0).view(np.uint16)
    qs = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    w = oracle.pack_blocks(np.full(n * (k // 32), one), qs)
    x = rng.integers(-8, 9, size=(3, k)).astype(np.float32)
    got = to_host(q8.mul_mat_f32_activations(q8.tile(to_dev(w), n, k), to_dev(x), n, k))
    assert np.array_equal(got.astype(np.int64), x.astype(np.int64) @ qs.astype(np.int64).T)


def test_differs_from_the_quantized_path_as_expected(q8, oracle):
    # the same operands through the model's path (activations quantized to Q8_0 first): close, but not the same numbers --
    # the quantization error of the activations is ~0.5 % here, far above the fp32 contract
    rng = np.random.default_rng(4)
    n, k = 512, 4096
    w = random_blocks(rng, n, k)
    x = rng.standard_normal(k).astype(np.float32)
    wt = q8.tile(to_dev(w), n, k)
    a = to_host(q8.mul_mat_f32_activations(wt, to_dev(x), n, k))[0]
    b = to_host(q8.gemv_f32(wt, to_dev(x), n, k))
    assert 1e-3 < rel_l2(b, a) < 3e-2

"""The checker's restatement of the reference's fp32-activation mul_mat (no activation quantize; cpu/avx_2.hpp:4782-5004),
pinned without running the reference: against a float64 evaluation, against dequantize-then-dot (an independent route through
the layout and the fp16 decode), by cases whose answer is an exact integer, and by the two reference summation orders agreeing
to rounding."""
import numpy as np

from helpers import random_blocks, rel_l2


def test_orders_agree_with_float64_and_with_dequantized_weights(oracle):
    rng = np.random.default_rng(21)
    for n, k, m in ((7, 32, 1), (33, 96, 3), (100, 4096, 2), (5, 14336, 1)):
        w = random_blocks(rng, n, k)
        x = rng.standard_normal((m, k)).astype(np.float32)
        ref = oracle.mul_mat_f32_activations_f64(w, x, n, k)
        deq = np.stack([oracle.dequantize_row(w.reshape(n, -1)[i], k) for i in range(n)]).astype(np.float64)
        assert rel_l2(ref, x.astype(np.float64) @ deq.T) < 1e-12  # same products, float64 both ways
        for prompt in (False, True):
            got = oracle.mul_mat_f32_activations(w, x, n, k, prompt_order=prompt)
            # fp32 sums in element order: the rounding error grows with the number of terms (a dropped term or a wrong
            # index is three orders of magnitude above this bound)
            assert got.shape == (m, n) and rel_l2(got, ref) < 2e-6 * max(1.0, (k / 1024) ** 0.5) * 4, (n, k, m, prompt)


def test_unit_scales_and_integer_activations_are_exact(oracle):
    # d == 1 and small integer activations: every product and partial sum is an integer below 2^24, so fp32 is exact in any order
    rng = np.random.default_rng(22)
    n, k = 12, 256
    one = np.float16(1.0).view(np.uint16)
    qs = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    w = oracle.pack_blocks(np.full(n * (k // 32), one), qs)
    x = rng.integers(-8, 9, size=(2, k)).astype(np.float32)
    want = x.astype(np.int64) @ qs.astype(np.int64).T
    for prompt in (False, True):
        assert np.array_equal(oracle.mul_mat_f32_activations(w, x, n, k, prompt_order=prompt).astype(np.int64), want)


def test_a_dropped_scale_or_transposed_operand_would_show(oracle):
    # scales that differ per block and per row, activations that differ per row: the answer changes if a scale is skipped,
    # taken from the wrong block, or if rows and columns are swapped
    n, k = 3, 64
    d = np.array([0.5, 2.0, 1.0, 4.0, 0.25, 8.0], dtype=np.float16).view(np.uint16)
    qs = np.zeros((n, k), dtype=np.int8)
    qs[0, 0], qs[0, 32], qs[1, 1], qs[1, 33], qs[2, 2], qs[2, 34] = 1, 2, 3, 4, 5, 6
    w = oracle.pack_blocks(d, qs)
    x = np.zeros((2, k), dtype=np.float32)
    x[0, [0, 1, 2, 32, 33, 34]] = [1, 10, 100, 1000, 10000, 100000]
    x[1, [0, 32]] = [-1, 1]
    want = np.array([[1 * 0.5 + 2000 * 2.0, 30 * 1.0 + 40000 * 4.0, 500 * 0.25 + 600000 * 8.0], [-0.5 + 4.0, 0.0, 0.0]], dtype=np.float32)
    assert np.array_equal(oracle.mul_mat_f32_activations(w, x, n, k), want)
    assert np.array_equal(oracle.mul_mat_f32_activations(w, x, n, k, prompt_order=True), want)

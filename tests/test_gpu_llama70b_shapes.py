"""GPU parity at the LLaMA-3-70B projection shapes, batched decode M in {1, 4, 16, 64}.

Shapes follow the reference's model constants (infra/model_traits.hpp:49-83, infra/core_traits.hpp:145-182):
q/o [8192x8192], k/v [1024x8192], gate/up [28672x8192], down [8192x28672], lm_head [128256x8192].
Everything goes through nh_q8_0_mul_mat (fp32 activations in, quantize included), which picks the
mat-vec for M = 1 and the weight-streaming mat-mat above it; the expected values come from the CPU
restatement on the same seeded bytes.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

PROJECTIONS = {"q_o": (8192, 8192), "k_v": (1024, 8192), "gate_up": (28672, 8192), "down": (8192, 28672)}
BATCHES = [1, 4, 16, 64]


@pytest.mark.parametrize("name", list(PROJECTIONS))
def test_llama70b_projection(q8, oracle, name):
    n, k = PROJECTIONS[name]
    w = oracle.fill_weights(70 + n % 97, n, k)
    wt = q8.tile(to_dev(w), n, k)
    for m in BATCHES:
        x = oracle.fill_activations(m, m * k).reshape(m, k)
        aq = oracle.quantize_rows(x)
        want = oracle.gemm(w, aq, m, n, k, threads=8)
        got = to_host(q8.mul_mat(wt, to_dev(x), n, k)).reshape(m, n)
        assert rel_l2(got, want) <= REL_L2_TOL, (name, m)
        for i in range(m):  # row by row: a wrong row must not hide in the norm of the others
            assert rel_l2(got[i], want[i]) <= REL_L2_TOL, (name, m, i)
        if m == 1:
            # the activation bytes the fused launch quantized itself are the checker's, bit for bit
            assert np.array_equal(to_host(q8.debug_fused_quantize(to_dev(x[0]))), aq.reshape(-1))


def test_llama70b_lm_head(q8, oracle):
    n, k = 128256, 8192
    w = oracle.fill_weights(7, n, k)
    wt = q8.tile(to_dev(w), n, k)
    row_bytes = (k // 32) * 34
    # the checker runs on three row windows (first, an unaligned middle one, the last rows): rows are independent
    windows = [(0, 256), (64001, 64001 + 223), (n - 200, n)]
    for m in BATCHES:
        x = oracle.fill_activations(100 + m, m * k).reshape(m, k)
        aq = oracle.quantize_rows(x)
        got = to_host(q8.mul_mat(wt, to_dev(x), n, k)).reshape(m, n)
        assert np.isfinite(got).all()
        for r0, r1 in windows:
            want = oracle.gemm(w[r0 * row_bytes : r1 * row_bytes], aq, m, r1 - r0, k, threads=8)
            assert rel_l2(got[:, r0:r1], want) <= REL_L2_TOL, (m, r0)
    # whole output at M = 64 against the checker on every row
    want = oracle.gemm(w, aq, 64, n, k, threads=8)
    assert rel_l2(got, want) <= REL_L2_TOL

"""GPU: size-independent properties at the full benchmark sizes (no CPU work beyond generating inputs).

* scaling the activation by a power of two scales every block scale exactly and leaves the quants unchanged, so the
  output scales exactly (bit for bit), through the fused quantizer of the mat-vec and through the stand-alone one;
* rows are independent: a mat-mat equals the mat-vecs of its rows (same exact block sums, fp32 order differs);
* the tiled copy of a weight is a permutation: tile -> untile gives the bytes back.
"""
import numpy as np
import pytest

from helpers import rel_l2, to_host

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("n,k", [(128256, 4096), (14336, 4096), (4096, 14336), (28672, 8192), (8192, 28672)])
def test_power_of_two_scaling_is_exact(q8, n, k):
    w = q8.fill_weight_blocks(n, n, k)
    wt = q8.tile(w, n, k)
    assert (q8.untile(wt, n, k) == w).all()
    del w
    x = q8.fill_activations(k, k)
    y = q8.gemv_f32(wt, x, n, k)
    for s in (0.25, 8.0):
        assert (q8.gemv_f32(wt, x * s, n, k) == y * s).all()
    # two-step form: the stand-alone quantizer's blocks differ from the unscaled ones only in their scale fields
    a, b = to_host(q8.quantize_row_q8_0(x)).reshape(-1, 34), to_host(q8.quantize_row_q8_0(x * 4.0)).reshape(-1, 34)
    assert np.array_equal(a[:, 2:], b[:, 2:])
    da, db = a[:, :2].copy().view(np.float16).astype(np.float32), b[:, :2].copy().view(np.float16).astype(np.float32)
    assert np.array_equal(db, da * 4.0)


@pytest.mark.parametrize("m,n,k", [(512, 14336, 4096), (64, 28672, 8192), (16, 128256, 4096), (3, 4096, 14336)])
def test_mat_mat_rows_equal_mat_vecs(q8, m, n, k):
    wt = q8.tile(q8.fill_weight_blocks(m + n, n, k), n, k)
    x = q8.fill_activations(m, m * k).reshape(m, k)
    c = q8.mul_mat(wt, x, n, k)
    for i in sorted({0, 1, m // 2, m - 1}):
        assert rel_l2(to_host(c[i]), to_host(q8.gemv_f32(wt, x[i].contiguous(), n, k))) < 2e-6, i

"""GPU parity: fused activation quantize vs the CPU restatement -- bit-exact bytes."""
import numpy as np
import pytest

from helpers import to_dev, to_host

pytestmark = pytest.mark.gpu


def _check(q8, oracle, x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    want = oracle.quantize_rows(x)
    got = to_host(q8.quantize_row_q8_0(to_dev(x)))
    assert got.shape == want.shape
    if not np.array_equal(got, want):
        bad = np.argwhere(got != want)
        raise AssertionError(f"{len(bad)} bytes differ, first at {bad[0]}: got {got[tuple(bad[0])]} want {want[tuple(bad[0])]}")


@pytest.mark.parametrize("m,k", [(1, 4096), (1, 14336), (1, 32), (3, 96), (7, 8192), (512, 4096), (33, 28672)])
def test_quantize_normal_inputs(q8, oracle, m, k):
    rng = np.random.default_rng(1000 + m + k)
    _check(q8, oracle, rng.standard_normal((m, k)))


def test_quantize_generator_inputs(q8, oracle):
    # config 1's activation vector, drawn by the CPU generator
    _check(q8, oracle, oracle.fill_activations(0, 4096)[None, :])


def test_quantize_adversarial_blocks(q8, oracle):
    rng = np.random.default_rng(7)
    rows = []
    rows.append(np.zeros(32))  # all-zero block: d = 0, q = 0
    rows.append(np.full(32, -0.0))
    r = np.arange(32, dtype=np.float64) - 15.5  # exact .5 ties after scaling by 127/amax with amax = 127
    r = np.concatenate([[127.0], np.arange(31) + 0.5])
    rows.append(r)
    rows.append(-r)
    rows.append(r * 2.0**-20)
    rows.append(r * 2.0**20)
    rows.append(np.full(32, 65504.0 * 127))  # d overflows nothing: amax/127 = 65504 = fp16 max
    rows.append(np.full(32, 70000.0 * 127))  # d rounds to fp16 inf
    rows.append(np.full(32, 1e-8))  # d in the fp16 subnormal range
    rows.append(np.full(32, 5.96e-8 * 127))  # d near the smallest fp16 subnormal
    rows.append(np.full(32, 1e-12))  # d underflows to 0 while quants stay +-127
    rows.append(np.full(32, 1e-40))  # fp32 subnormal inputs
    rows.append(np.concatenate([[1e-45], np.zeros(31)]))  # smallest fp32 subnormal: 127/amax overflows to inf
    rows.append(np.concatenate([[3.4e38], rng.standard_normal(31) * 1e37]))
    x = np.stack(rows).astype(np.float32)
    _check(q8, oracle, x)
    # heavy-tailed magnitudes over the whole exponent range
    e = rng.integers(-120, 120, size=(64, 1)).astype(np.float64)
    _check(q8, oracle, (rng.standard_normal((64, 256)) * 2.0**e).astype(np.float32))


def test_quantize_tiled_matches_blocks(q8, oracle):
    rng = np.random.default_rng(11)
    for m, k in [(1, 128), (33, 256), (512, 4096), (70, 14336)]:
        x = rng.standard_normal((m, k)).astype(np.float32)
        want = oracle.quantize_rows(x).reshape(-1)
        tiled = q8.quantize_row_q8_0(to_dev(x), tiled=True)
        got = to_host(q8.untile(tiled, m, k))
        assert np.array_equal(got, want), (m, k)
        # padding rows of the last strip must be zero blocks
        pad_rows = (-m) % 32
        if pad_rows:
            full = to_host(q8.untile(tiled, m + pad_rows, k)).reshape(m + pad_rows, -1)
            assert not full[m:].any()


@pytest.mark.parametrize("m,k", [(1030, 4096), (8200, 512), (2048, 8192)])
def test_quantize_two_blocks_per_thread(q8, oracle, m, k):
    # from 2^20 float4s on a thread takes two, a grid's worth of threads apart: same bytes, both layouts, ragged last strip included
    rng = np.random.default_rng(m + k)
    x = rng.standard_normal((m, k)).astype(np.float32)
    x[m // 2] = 0.0
    want = oracle.quantize_rows(x)
    assert np.array_equal(to_host(q8.quantize_row_q8_0(to_dev(x))), want)
    tiled = q8.quantize_row_q8_0(to_dev(x), tiled=True)
    rows = (m + 31) // 32 * 32
    full = to_host(q8.untile(tiled, rows, k)).reshape(rows, -1)
    assert np.array_equal(full[:m], want) and not full[m:].any()


def test_quantize_either_side_of_the_size_where_a_thread_takes_two_blocks(q8, oracle):
    # 2^20 float4s = 2^17 blocks: shapes just below, at and above it, odd row counts, both layouts
    for m, k in [(1023, 4096), (1024, 4096), (1025, 4096), (4097, 1024), (257, 16384)]:
        rng = np.random.default_rng(m + k)
        x = (rng.standard_normal((m, k)) * rng.uniform(0.01, 100.0)).astype(np.float32)
        want = oracle.quantize_rows(x)
        assert np.array_equal(to_host(q8.quantize_row_q8_0(to_dev(x))), want), (m, k)
        rows = (m + 31) // 32 * 32
        full = to_host(q8.untile(q8.quantize_row_q8_0(to_dev(x), tiled=True), rows, k)).reshape(rows, -1)
        assert np.array_equal(full[:m], want) and not full[m:].any(), (m, k)


def test_quantize_empty_and_errors(q8):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    x = torch.zeros(64, dtype=torch.float32, device="cuda")
    out = torch.zeros(128, dtype=torch.uint8, device="cuda")
    assert lib.nh_q8_0_quantize(x.data_ptr(), out.data_ptr(), 0, 32, None) == 0  # empty: no work
    assert lib.nh_q8_0_quantize(x.data_ptr(), out.data_ptr(), 1, 0, None) == 0
    assert lib.nh_q8_0_quantize(x.data_ptr(), out.data_ptr(), 1, 33, None) == -3  # ragged K rejected
    assert lib.nh_q8_0_quantize(x.data_ptr(), out.data_ptr(), -1, 32, None) == -3
    assert lib.nh_q8_0_quantize(None, out.data_ptr(), 1, 32, None) == -1
    assert lib.nh_q8_0_quantize(x.data_ptr() + 4, out.data_ptr(), 1, 32, None) == -2
    assert lib.nh_q8_0_quantize_tiled(x.data_ptr(), out.data_ptr(), 1, 32, None) == -3  # tiled needs K % 128 == 0
    torch.cuda.synchronize()
    assert not out.any()

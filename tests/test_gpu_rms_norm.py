"""GPU: RMS norm * weight fused into the quantizer (stand-alone kernel, inside the mat-vec, inside the one-launch FFN),
byte-exact against the CPU checker, which takes the sum of squares in the same fixed order."""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

EPS = 1e-5


def row_inputs(seed, m, k, scale=3.0):
    rng = np.random.default_rng(seed)
    x = (rng.standard_normal((m, k)) * scale).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    return x, w


@pytest.mark.parametrize("m,k", [(1, 128), (1, 4096), (5, 8192), (33, 1024), (3, 14336), (64, 4096)])
def test_rms_norm_quantize_bit_exact(q8, oracle, m, k):
    x, w = row_inputs(m + k, m, k)
    want = oracle.rms_norm_quantize_rows(x, w, EPS)
    assert np.array_equal(to_host(q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS)), want)
    tiled = q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS, tiled=True)
    assert np.array_equal(to_host(q8.untile(tiled, m, k)).reshape(m, -1), want)


@pytest.mark.parametrize("m,k", [(2048, 4096), (2050, 1664), (2048, 8192), (2100, 128), (2049, 2048), (4096, 640)])
def test_rms_norm_quantize_eight_rows_per_workgroup(q8, oracle, m, k):
    # From 2048 rows on the tiled form takes eight rows per workgroup (whole 128-byte lines of the operand tiles per store, the
    # rows read once): one and two float4s per lane and run, runs of unequal length (13 and 5 groups over 16 runs), a single
    # group, a ragged last strip whose padding rows must come out as zero blocks.  Same bytes as the CPU checker.
    x, w = row_inputs(m + k, m, k)
    x[7] = 0.0
    want = oracle.rms_norm_quantize_rows(x, w, EPS)
    tiled = q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS, tiled=True)
    rows = (m + 31) // 32 * 32
    full = to_host(q8.untile(tiled, rows, k)).reshape(rows, -1)
    assert np.array_equal(full[:m], want)
    assert not full[m:].any()


def test_rms_norm_quantize_either_side_of_the_row_count_where_the_form_changes(q8, oracle):
    # seeded random shapes around 2048 rows (one row per workgroup below, eight from there on) and K up to 8192 and beyond (the
    # eight-row form stops at 8192): both forms and the hand-over between them give the checker's bytes
    rng = np.random.default_rng(2048)
    shapes = [(2047, 384), (2048, 384), (2049, 384)] + [(int(rng.integers(1990, 2120)), 128 * int(rng.integers(1, 65))) for _ in range(5)] + [(2050, 8320)]
    for m, k in shapes:
        x, w = row_inputs(m * 7 + k, m, k, scale=float(rng.uniform(0.1, 30.0)))
        want = oracle.rms_norm_quantize_rows(x, w, EPS)
        rows = (m + 31) // 32 * 32
        full = to_host(q8.untile(q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS, tiled=True), rows, k)).reshape(rows, -1)
        assert np.array_equal(full[:m], want), (m, k)
        assert not full[m:].any(), (m, k)


@pytest.mark.parametrize("k", [128, 1024, 4096, 8192, 14336])
def test_norm_inside_the_mat_vec_stages_the_same_bytes(q8, oracle, k):
    # K <= 8192: the in-chunk reduction (weights already in flight); 14336: the up-front form
    x, w = row_inputs(k, 1, k, scale=0.5)
    want = oracle.rms_norm_quantize_rows(x, w, EPS)[0]
    assert np.array_equal(to_host(q8.debug_fused_quantize(to_dev(x[0]), to_dev(w), EPS)), want)
    assert np.array_equal(to_host(q8.debug_fused_quantize(to_dev(x[0]))), oracle.quantize_rows(x)[0])  # and without a norm, as before


@pytest.mark.parametrize("n,k", [(4096, 4096), (100, 1024), (1024, 8192), (64, 14336), (128256, 4096)])
def test_norm_mat_vec_matches_two_step_form(q8, oracle, n, k):
    x, w = row_inputs(n + k, 1, k)
    wt = q8.tile(q8.fill_weight_blocks(n, n, k), n, k)
    y = q8.gemv_f32(wt, to_dev(x[0]), n, k, norm_weight=to_dev(w), eps=EPS)
    xq = q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS)
    assert np.array_equal(to_host(y), to_host(q8.gemv(wt, xq.reshape(-1), n, k, True)))  # same quantized row, same mat-vec
    if n <= 4096:
        wb = oracle.fill_weights(n, n, k)
        assert rel_l2(to_host(y), oracle.gemv(wb, oracle.rms_norm_quantize_rows(x, w, EPS)[0], n, k)) <= REL_L2_TOL


def test_norm_qkv_as_one_launch(q8, oracle):
    k, ns = 4096, [4096, 1024, 1024]
    x, w = row_inputs(9, 1, k)
    wts = [q8.tile(q8.fill_weight_blocks(20 + i, n, k), n, k) for i, n in enumerate(ns)]
    ys = q8.gemv_f32(wts, to_dev(x[0]), ns, k, norm_weight=to_dev(w), eps=EPS)
    xq = oracle.rms_norm_quantize_rows(x, w, EPS)[0]
    for i, n in enumerate(ns):
        assert rel_l2(to_host(ys[i]), oracle.gemv(oracle.fill_weights(20 + i, n, k), xq, n, k)) <= REL_L2_TOL


def test_norm_inside_the_one_launch_ffn(q8, oracle):
    n_ff, k, n_out = 2048, 1024, 512
    rng = np.random.default_rng(4)
    wg, wu, wd = random_blocks(rng, n_ff, k, 0.02), random_blocks(rng, n_ff, k, 0.02), random_blocks(rng, n_out, n_ff, 0.02)
    x, w = row_inputs(5, 1, k)
    t = [q8.tile(to_dev(b), r, c) for b, r, c in ((wg, n_ff, k), (wu, n_ff, k), (wd, n_out, n_ff))]
    y = q8.ffn(t[0], t[1], t[2], to_dev(x[0]), n_ff, k, n_out, norm_weight=to_dev(w), eps=EPS)
    g, u = q8.debug_ffn_gate_up(n_ff)
    xq = oracle.rms_norm_quantize_rows(x, w, EPS)[0]
    assert rel_l2(to_host(g), oracle.gemv(wg, xq, n_ff, k)) <= REL_L2_TOL and rel_l2(to_host(u), oracle.gemv(wu, xq, n_ff, k)) <= REL_L2_TOL
    aq = oracle.silu_mul_quantize_rows(to_host(g), to_host(u))[0]
    assert rel_l2(to_host(y), oracle.gemv(wd, aq, n_out, n_ff)) <= 2e-6


@pytest.mark.parametrize("ns,k", [([128256], 4096), ([8192], 28672), ([28672, 28672], 8192), ([32768, 1000, 33], 512)])
def test_norm_row_shared_between_the_workgroups_of_a_large_launch(q8, oracle, ns, k):
    # From 1024 workgroups on, only the first strip's workgroups (one per K split) normalise and quantize the row; they publish
    # it and the rest read it.  The result must be the two-step form's (same quantized row, same mat-vec: bit for bit), on an
    # unsplit launch, a K-split one, two and three matrices in one launch with ragged tails, and launch after launch with a new row.
    wts = [q8.tile(q8.fill_weight_blocks(40 + i, n, k), n, k) for i, n in enumerate(ns)]
    for rep in range(3):
        x, w = row_inputs(50 + rep + k, 1, k, scale=1.0 + rep)
        ys = q8.gemv_f32(wts if len(ns) > 1 else wts[0], to_dev(x[0]), ns if len(ns) > 1 else ns[0], k, norm_weight=to_dev(w), eps=EPS)
        ys = ys if len(ns) > 1 else [ys]
        xq = q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS)
        assert np.array_equal(to_host(xq).reshape(-1), oracle.rms_norm_quantize_rows(x, w, EPS)[0].reshape(-1))
        for i, n in enumerate(ns):
            alone = to_host(q8.gemv(wts[i], xq.reshape(-1), n, k, True))
            if len(ns) == 1:
                assert np.array_equal(to_host(ys[i]), alone), (rep, i)  # one matrix: the stand-alone launch cuts K the same way
            else:
                assert rel_l2(to_host(ys[i]), alone) < 2e-6, (rep, i)  # a matrix launched alone may be cut differently: last bits


def test_norm_row_shared_inside_the_one_launch_ffn(q8, oracle):
    # 896 producer workgroups: the first publishes the normalised, quantized row, the others read it
    n_ff, k, n_out = 28672, 1024, 256
    wg_t, wu_t = (q8.tile(q8.fill_weight_blocks(60 + i, n_ff, k), n_ff, k) for i in range(2))
    wd_t = q8.tile(q8.fill_weight_blocks(62, n_out, n_ff), n_out, n_ff)
    for rep in range(3):
        x, w = row_inputs(70 + rep, 1, k, scale=0.5 + rep)
        y = q8.ffn(wg_t, wu_t, wd_t, to_dev(x[0]), n_ff, k, n_out, norm_weight=to_dev(w), eps=EPS)
        g, u = q8.debug_ffn_gate_up(n_ff)
        xq = q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS)
        # gate and up are mat-vecs of the same quantized row: the stand-alone kernel cuts K differently, so last bits may differ
        assert rel_l2(to_host(g), to_host(q8.gemv(wg_t, xq.reshape(-1), n_ff, k, True))) < 2e-6
        assert rel_l2(to_host(u), to_host(q8.gemv(wu_t, xq.reshape(-1), n_ff, k, True))) < 2e-6
        aq = oracle.silu_mul_quantize_rows(to_host(g), to_host(u))[0]
        rows = 64
        assert rel_l2(to_host(y)[:rows], oracle.gemv(oracle.fill_weights(62, rows, n_ff), aq, rows, n_ff)) <= REL_L2_TOL


@pytest.mark.parametrize("n_ff,k,n_out", [(4096, 3072, 256), (2048, 2560, 512), (14336, 4096, 4096)])
def test_norm_ffn_with_producer_waves_on_both_matrices(q8, oracle, n_ff, k, n_out):
    # K of 17..32 groups with a norm: the producer workgroup cuts the row sixteen ways and every wave takes its range of gate AND
    # up against one staged slice (ranges of one and two groups mixed when K / 128 is not a multiple of 16)
    wg_t, wu_t = (q8.tile(q8.fill_weight_blocks(80 + i, n_ff, k), n_ff, k) for i in range(2))
    wd_t = q8.tile(q8.fill_weight_blocks(82, n_out, n_ff), n_out, n_ff)
    x, w = row_inputs(n_ff + k, 1, k, scale=0.7)
    res = np.random.default_rng(1).standard_normal(n_out).astype(np.float32)
    y = q8.ffn(wg_t, wu_t, wd_t, to_dev(x[0]), n_ff, k, n_out, residual=to_dev(res), norm_weight=to_dev(w), eps=EPS)
    g, u = q8.debug_ffn_gate_up(n_ff)
    xq = oracle.rms_norm_quantize_rows(x, w, EPS)[0]
    rows = min(n_ff, 256)
    assert rel_l2(to_host(g)[:rows], oracle.gemv(oracle.fill_weights(80, rows, k), xq, rows, k)) <= REL_L2_TOL
    assert rel_l2(to_host(u)[:rows], oracle.gemv(oracle.fill_weights(81, rows, k), xq, rows, k)) <= REL_L2_TOL
    xq_d = q8.rms_norm_quantize(to_dev(x), to_dev(w), EPS)
    assert rel_l2(to_host(g), to_host(q8.gemv(wg_t, xq_d.reshape(-1), n_ff, k, True))) < 2e-6  # every row, against the stand-alone mat-vec
    assert rel_l2(to_host(u), to_host(q8.gemv(wu_t, xq_d.reshape(-1), n_ff, k, True))) < 2e-6
    aq = oracle.silu_mul_quantize_rows(to_host(g), to_host(u))[0]
    rows_out = min(n_out, 64)
    assert rel_l2(to_host(y)[:rows_out], oracle.gemv(oracle.fill_weights(82, rows_out, n_ff), aq, rows_out, n_ff) + res[:rows_out]) <= REL_L2_TOL
    assert np.array_equal(to_host(q8.ffn(wg_t, wu_t, wd_t, to_dev(x[0]), n_ff, k, n_out, residual=to_dev(res), norm_weight=to_dev(w), eps=EPS)), to_host(y))  # bit-stable


def test_rms_norm_errors(q8):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    x = torch.ones(128, dtype=torch.float32, device="cuda")
    out = torch.zeros(4 * 34, dtype=torch.uint8, device="cuda")
    p = lambda t: t.data_ptr()
    assert lib.nh_q8_0_rms_norm_quantize(p(x), p(x), 1e-5, p(out), 1, 100, None) == -3
    assert lib.nh_q8_0_rms_norm_quantize(p(x), None, 1e-5, p(out), 1, 128, None) == -1
    assert lib.nh_q8_0_rms_norm_quantize(p(x), p(x), -1.0, p(out), 1, 128, None) == -6
    assert lib.nh_q8_0_rms_norm_quantize(p(x), p(x) + 4, 1e-5, p(out), 1, 128, None) == -2
    assert lib.nh_q8_0_rms_norm_quantize(p(x), p(x), 1e-5, p(out), 1, 96, None) == -3  # the sum order is defined on 128-value groups
    assert lib.nh_q8_0_rms_norm_quantize(p(x), p(x), 1e-5, p(out), 0, 128, None) == 0

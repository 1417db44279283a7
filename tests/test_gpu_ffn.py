"""GPU: the decode-time FFN as one launch (gate/up mat-vecs, SiLU*up, down mat-vec) through the C ABI.

Checked against the CPU checker's composition of the same steps (fp32 outputs, 1e-4 relative L2), stage by stage
(the down projection is re-derived from the launch's own gate/up outputs, so its activation quantize is compared
bit for bit in effect: one wrong quant moves y by far more than the fp32 order does), against the library's own
three-launch sequence, and launch after launch with changing inputs (a consumer that read a previous launch's
activation, or woke on a stale flag, would differ).  The fused launch cuts K differently from the stand-alone
mat-vecs, so the gate/up sums differ in the last bits between the two; since a quantizer sits between the stages, a
last-bit difference in an activation that lies on a rounding tie moves one quant by one, which shows in y at the 1e-4
level: end-to-end comparisons across different summation orders therefore use END_TO_END_TOL, the stage-wise ones
the tight bounds.  Runs of the same launch are bit-identical.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

END_TO_END_TOL = 1e-3  # across the intermediate quantizer, see the module docstring


def cpu_ffn(oracle, wg, wu, wd, x, n_ff, k, n_out, residual=None):
    xq = oracle.quantize_rows(x)[0]
    g = oracle.gemv(wg, xq, n_ff, k)
    u = oracle.gemv(wu, xq, n_ff, k)
    aq = oracle.silu_mul_quantize_rows(g, u)[0]
    y = oracle.gemv(wd, aq, n_out, n_ff)
    return (y + residual if residual is not None else y), g, u


def gpu_three_launches(q8, wg_t, wu_t, wd_t, x_d, n_ff, k, n_out):
    g = q8.gemv_f32(wg_t, x_d, n_ff, k)
    u = q8.gemv_f32(wu_t, x_d, n_ff, k)
    aq = q8.silu_mul_quantize(g, u)
    return q8.gemv(wd_t, aq.reshape(-1), n_out, n_ff, True), g, u


def make(seed, n_ff, k, n_out, q8):
    rng = np.random.default_rng(seed)
    wg, wu, wd = random_blocks(rng, n_ff, k, 0.02), random_blocks(rng, n_ff, k, 0.02), random_blocks(rng, n_out, n_ff, 0.02)
    tiled = [q8.tile(to_dev(w), r, c) for w, r, c in ((wg, n_ff, k), (wu, n_ff, k), (wd, n_out, n_ff))]
    return rng, (wg, wu, wd), tiled


@pytest.mark.parametrize("n_ff,k,n_out", [(128, 128, 32), (256, 256, 100), (512, 1024, 64), (2048, 512, 2048), (14336, 4096, 4096), (4096, 2048, 33)])
def test_ffn_matches_checker_and_three_launch_sequence(q8, oracle, n_ff, k, n_out):
    rng, (wg, wu, wd), (wg_t, wu_t, wd_t) = make(n_ff + k + n_out, n_ff, k, n_out, q8)
    x = rng.standard_normal(k).astype(np.float32)
    res = rng.standard_normal(n_out).astype(np.float32)
    x_d = to_dev(x)
    y = q8.ffn(wg_t, wu_t, wd_t, x_d, n_ff, k, n_out)
    g, u = q8.debug_ffn_gate_up(n_ff)
    y3, g3, u3 = gpu_three_launches(q8, wg_t, wu_t, wd_t, x_d, n_ff, k, n_out)
    assert rel_l2(to_host(g), to_host(g3)) <= 2e-6 and rel_l2(to_host(u), to_host(u3)) <= 2e-6
    assert rel_l2(to_host(y), to_host(y3)) <= END_TO_END_TOL
    want, wg_cpu, wu_cpu = cpu_ffn(oracle, wg, wu, wd, x, n_ff, k, n_out)
    assert rel_l2(to_host(g), wg_cpu) <= REL_L2_TOL and rel_l2(to_host(u), wu_cpu) <= REL_L2_TOL
    assert rel_l2(to_host(y), want) <= END_TO_END_TOL
    # the down stage alone, from this launch's own gate/up values: checker-side SiLU*up, quantize and mat-vec
    aq = oracle.silu_mul_quantize_rows(to_host(g), to_host(u))[0]
    assert rel_l2(to_host(y), oracle.gemv(wd, aq, n_out, n_ff)) <= 2e-6
    assert np.array_equal(to_host(q8.ffn(wg_t, wu_t, wd_t, x_d, n_ff, k, n_out)), to_host(y))  # run-to-run bit-stable
    # residual: one fp32 add after the sum
    yr = q8.ffn(wg_t, wu_t, wd_t, x_d, n_ff, k, n_out, residual=to_dev(res))
    assert np.array_equal(to_host(yr), to_host(y) + res)


def test_ffn_llama3_70b_shape(q8, oracle):
    n_ff, k, n_out = 28672, 8192, 8192
    wg_t = q8.tile(q8.fill_weight_blocks(1, n_ff, k), n_ff, k)
    wu_t = q8.tile(q8.fill_weight_blocks(2, n_ff, k), n_ff, k)
    wd_t = q8.tile(q8.fill_weight_blocks(3, n_out, n_ff), n_out, n_ff)
    x_d = q8.fill_activations(4, k)
    y = q8.ffn(wg_t, wu_t, wd_t, x_d, n_ff, k, n_out)
    y3, _, _ = gpu_three_launches(q8, wg_t, wu_t, wd_t, x_d, n_ff, k, n_out)
    assert np.isfinite(to_host(y)).all()
    assert rel_l2(to_host(y), to_host(y3)) <= END_TO_END_TOL
    # a 64-row slice against the CPU checker (the whole matrix would take the scalar checker minutes)
    g, u = q8.debug_ffn_gate_up(n_ff)
    aq = oracle.silu_mul_quantize_rows(to_host(g), to_host(u))[0]
    rows = 64
    wd_rows = oracle.fill_weights(3, rows, n_ff)
    assert rel_l2(to_host(y)[:rows], oracle.gemv(wd_rows, aq, rows, n_ff)) <= REL_L2_TOL


def test_ffn_back_to_back_launches_with_changing_inputs(q8):
    n_ff, k, n_out = 14336, 4096, 4096
    rng, _, (wg_t, wu_t, wd_t) = make(7, n_ff, k, n_out, q8)
    xs = [to_dev(rng.standard_normal(k).astype(np.float32) * (1 + i % 3)) for i in range(6)]
    import torch

    want = []
    for x in xs:  # each input's answer from a launch of its own, with a synchronisation after it
        want.append(to_host(q8.ffn(wg_t, wu_t, wd_t, x, n_ff, k, n_out)))
        torch.cuda.synchronize()
        assert rel_l2(want[-1], to_host(gpu_three_launches(q8, wg_t, wu_t, wd_t, x, n_ff, k, n_out)[0])) <= END_TO_END_TOL

    outs = []
    for rep in range(5):  # 30 launches queued back to back, no synchronisation in between
        for x in xs:
            outs.append(q8.ffn(wg_t, wu_t, wd_t, x, n_ff, k, n_out))
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert np.array_equal(to_host(o), want[i % len(xs)]), i


def test_ffn_unit_scales_give_exact_integers(q8, oracle):
    # power-of-two scales and integer activations: every fp32 sum of the gate/up stage is exact, whatever the order
    n_ff, k, n_out = 256, 256, 64
    rng = np.random.default_rng(11)

    def unit_blocks(rows, cols, d_hi=0x24):  # fp16 0x2400 = 2^-6: keeps silu(g) * u far inside the fp16 range of its scale
        b = np.empty((rows * (cols // 32), 34), dtype=np.uint8)
        b[:, 0], b[:, 1] = 0x00, d_hi
        b[:, 2:] = rng.integers(-3, 4, size=(b.shape[0], 32), dtype=np.int8).view(np.uint8)
        return b.reshape(-1)

    wg, wu, wd = unit_blocks(n_ff, k), unit_blocks(n_ff, k), unit_blocks(n_out, n_ff, 0x3C)
    x = rng.integers(-127, 128, size=k).astype(np.float32)
    x[::32] = 127.0  # every block's amax is 127: d = 1, the quants are the values themselves
    y = q8.ffn(q8.tile(to_dev(wg), n_ff, k), q8.tile(to_dev(wu), n_ff, k), q8.tile(to_dev(wd), n_out, n_ff), to_dev(x), n_ff, k, n_out)
    g, u = q8.debug_ffn_gate_up(n_ff)
    want, g_cpu, u_cpu = cpu_ffn(oracle, wg, wu, wd, x, n_ff, k, n_out)
    assert np.array_equal(to_host(g), g_cpu) and np.array_equal(to_host(u), u_cpu)
    assert np.array_equal(g_cpu * 64, np.rint(g_cpu * 64)) and np.isfinite(want).all()
    assert rel_l2(to_host(y), want) <= 2e-6


def test_ffn_empty_and_errors(q8):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    w = torch.zeros(4 * 4352, dtype=torch.uint8, device="cuda")  # [128 x 128] tiled, also large enough as [32 x 128]
    x = torch.ones(128, dtype=torch.float32, device="cuda")
    r = torch.arange(32, dtype=torch.float32, device="cuda")
    y = torch.full((32,), 7.0, dtype=torch.float32, device="cuda")
    p = lambda t: t.data_ptr()
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, None, p(y), 128, 128, 0, None) == 0
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, p(r), p(y), 0, 128, 32, None) == 0  # empty hidden dim: y = residual
    assert torch.equal(y, r)
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, None, p(y), 128, 0, 32, None) == 0
    assert torch.equal(y, torch.zeros_like(y))
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, None, p(y), 96, 128, 32, None) == -3
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, None, p(y), 128, 96, 32, None) == -3
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, None, p(y), 65536 + 128, 128, 32, None) == -5
    assert lib.nh_q8_0_ffn_f32(None, p(w), p(w), p(x), None, 0.0, None, p(y), 128, 128, 32, None) == -1
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, None, None, 128, 128, 32, None) == -1
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x) + 4, None, 0.0, None, p(y), 128, 128, 32, None) == -2
    # zero weights: g = u = 0, activation 0, y = residual exactly
    assert lib.nh_q8_0_ffn_f32(p(w), p(w), p(w), p(x), None, 0.0, p(r), p(y), 128, 128, 32, None) == 0
    assert torch.equal(y, r)

"""GPU: nh_q8_0_set_in_kernel_waits(0) -- no workgroup of any launch waits for another workgroup of the same launch.

The one-launch FFN, the chained block and the shared norm row of a large mat-vec rest on workgroups being dispatched in index
order.  With the switch off the same calls run as the launches they stand for (the forms a capturing stream gets).  Checked here:
the number of launches each call makes (through the library's per-launch timer, which counts them), and that the results are the
one-launch forms' (bit-identical where the arithmetic is the same, to 2e-6 where a sum is cut differently) and the CPU checker's.
The switch is process-wide: every test puts it back.
"""
import ctypes as C

import numpy as np
import pytest
import torch

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

KIND_QUANTIZE, KIND_GEMV = 0, 1
EPS = 1e-5


def _launches(lib, kind, fn):
    """How many launches of one kernel kind fn() makes."""
    assert lib.nh_profile_begin(kind, 64) == 0
    try:
        out = fn()
        torch.cuda.synchronize()
    finally:
        tot, cnt, mn, mx = C.c_double(), C.c_int64(), C.c_double(), C.c_double()
        assert lib.nh_profile_end(C.byref(tot), C.byref(cnt), C.byref(mn), C.byref(mx)) == 0
    return out, cnt.value


@pytest.fixture
def lib(q8):
    lb = q8._lib.lib()
    assert lb.nh_q8_0_set_in_kernel_waits(1) == 1  # the default
    yield lb
    lb.nh_q8_0_set_in_kernel_waits(1)


def test_ffn_as_three_launches(q8, oracle, lib):
    n_ff, k, n_out = 2048, 1024, 512
    rng = np.random.default_rng(21)
    wg, wu, wd = (random_blocks(rng, n, kk, 0.02) for n, kk in ((n_ff, k), (n_ff, k), (n_out, n_ff)))
    t = [q8.tile(to_dev(b), r, c) for b, r, c in ((wg, n_ff, k), (wu, n_ff, k), (wd, n_out, n_ff))]
    x = (rng.standard_normal(k) * 2).astype(np.float32)
    w = (1 + 0.1 * rng.standard_normal(k)).astype(np.float32)
    res = rng.standard_normal(n_out).astype(np.float32)
    call = lambda: q8.ffn(t[0], t[1], t[2], to_dev(x), n_ff, k, n_out, residual=to_dev(res), norm_weight=to_dev(w), eps=EPS)
    y_on, n_on = _launches(lib, KIND_GEMV, call)
    assert n_on == 1
    assert lib.nh_q8_0_set_in_kernel_waits(0) == 1
    y_off, n_off = _launches(lib, KIND_GEMV, call)
    assert n_off == 2  # gate/up, then down (the SiLU * up quantizer between them is a launch of another kind)
    _, n_q = _launches(lib, KIND_QUANTIZE, call)
    assert n_q == 1
    assert rel_l2(to_host(y_off), to_host(y_on)) <= 2e-6
    g, u = q8.debug_ffn_gate_up(n_ff)
    xq = oracle.rms_norm_quantize_rows(x[None, :], w, EPS)[0]
    assert rel_l2(to_host(g), oracle.gemv(wg, xq, n_ff, k)) <= REL_L2_TOL and rel_l2(to_host(u), oracle.gemv(wu, xq, n_ff, k)) <= REL_L2_TOL
    aq = oracle.silu_mul_quantize_rows(to_host(g)[None, :], to_host(u)[None, :])[0]
    assert rel_l2(to_host(y_off), oracle.gemv(wd, aq, n_out, n_ff) + res) <= 2e-6
    assert lib.nh_q8_0_set_in_kernel_waits(1) == 0
    _, n_again = _launches(lib, KIND_GEMV, call)
    assert n_again == 1


def test_decode_layer_as_its_three_steps(q8, oracle, lib):
    hidden, n_kv, n_ff = 512, 128, 1536
    rng = np.random.default_rng(22)

    def sigma(k_in):
        return 1.0 / (58.0 * np.sqrt(k_in))

    wo, wq, wk = (random_blocks(rng, n, hidden, sigma(hidden)) for n in (hidden, hidden, n_kv))
    wg, wu, wd = random_blocks(rng, n_ff, hidden, sigma(hidden)), random_blocks(rng, n_ff, hidden, sigma(hidden)), random_blocks(rng, hidden, n_ff, sigma(n_ff))
    t = {name: q8.tile(to_dev(b), n, k) for name, (b, n, k) in {"o": (wo, hidden, hidden), "q": (wq, hidden, hidden), "k": (wk, n_kv, hidden), "g": (wg, n_ff, hidden),
                                                               "u": (wu, n_ff, hidden), "d": (wd, hidden, n_ff)}.items()}
    attn = rng.standard_normal(hidden).astype(np.float32)
    layer_in = rng.standard_normal(hidden).astype(np.float32)
    fw = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    nw = (1 + 0.1 * rng.standard_normal(hidden)).astype(np.float32)
    call = lambda: q8.decode_layer(t["o"], to_dev(attn), to_dev(layer_in), t["g"], t["u"], t["d"], to_dev(fw), [t["q"], t["k"]], [hidden, n_kv], to_dev(nw), EPS, hidden, n_ff)
    (inp_on, out_on, ys_on), n_on = _launches(lib, KIND_GEMV, call)
    assert n_on == 1
    lib.nh_q8_0_set_in_kernel_waits(0)
    (inp_off, out_off, ys_off), n_off = _launches(lib, KIND_GEMV, call)
    assert n_off == 4  # attn_out; gate/up; down; the next block's q/k
    assert rel_l2(to_host(inp_off), to_host(inp_on)) <= 2e-6  # one mat-vec + residual either way, K cut over the waves differently
    assert rel_l2(to_host(out_off), to_host(out_on)) <= 2e-6
    for a, b in zip(ys_off, ys_on):
        assert rel_l2(to_host(a), to_host(b)) <= 2e-3  # behind one more quantizer: a last-bit difference of l_out may move a quant (6e-4 each)
    want_inp = oracle.gemv(wo, oracle.quantize_rows(attn[None, :])[0], hidden, hidden) + layer_in
    assert rel_l2(to_host(inp_off), want_inp) <= REL_L2_TOL


def test_norm_row_worked_out_by_every_workgroup(q8, oracle, lib):
    n, k = 32768 + 64, 512  # more than 1024 strips: with waits on, the first strip's workgroup publishes the row for the rest
    rng = np.random.default_rng(23)
    wt = q8.tile(q8.fill_weight_blocks(3, n, k), n, k)
    x = (rng.standard_normal(k) * 3).astype(np.float32)
    w = (1 + 0.2 * rng.standard_normal(k)).astype(np.float32)
    call = lambda: q8.gemv_f32(wt, to_dev(x), n, k, norm_weight=to_dev(w), eps=EPS)
    y_on = to_host(call())
    lib.nh_q8_0_set_in_kernel_waits(0)
    y_off = to_host(call())
    assert np.array_equal(y_off, y_on)  # the same quantized row either way, the same mat-vec
    xq = q8.rms_norm_quantize(to_dev(x[None, :]), to_dev(w), EPS)
    assert np.array_equal(y_off, to_host(q8.gemv(wt, xq.reshape(-1), n, k, True)))

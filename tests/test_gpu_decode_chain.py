"""GPU: a block's decode mat-vecs from one attention to the next as ONE launch (nh_q8_0_decode_layer_f32).

Checked three ways: (1) stage by stage against the CPU checker fed with the launch's own output of the stage before (the
contract's 1e-4, quantized activations implied bit for bit: a wrong quant in a staged row would show at the 1e-2 level);
(2) against the three launches it stands for (nh_q8_0_gemv_tiled_residual_f32, nh_q8_0_ffn_f32, nh_q8_0_gemv_tiled_multi_norm_f32),
bit for bit where both cut the work the same way (a small attn_out matrix is cut by rows as a launch of its own and by whole strips
here: same products, another order of the fp32 sums); (3) repeated launches with changing inputs, back to back without a wait in
between: the hand-offs go through per-GPU scratch tagged with a launch epoch, so a stale word of the previous launch must never be
taken for a fresh one.
"""
import numpy as np
import pytest
import torch

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

EPS = 1e-5


def _weights(q8, rng, n_embd, n_ff, next_rows):
    def sigma(k_in):  # about unit gain per projection: values stay O(1) through the chain
        return 1.0 / (58.0 * np.sqrt(k_in))

    host = {"o": (random_blocks(rng, n_embd, n_embd, sigma(n_embd)), n_embd, n_embd), "g": (random_blocks(rng, n_ff, n_embd, sigma(n_embd)), n_ff, n_embd),
            "u": (random_blocks(rng, n_ff, n_embd, sigma(n_embd)), n_ff, n_embd), "d": (random_blocks(rng, n_embd, n_ff, sigma(n_ff)), n_embd, n_ff)}
    for i, n in enumerate(next_rows):
        host[f"n{i}"] = (random_blocks(rng, n, n_embd, sigma(n_embd)), n, n_embd)
    dev = {name: q8.tile(to_dev(w), n, k) for name, (w, n, k) in host.items()}
    norms = [(1.0 + 0.1 * rng.standard_normal(n_embd)).astype(np.float32) for _ in range(2)]
    return host, dev, norms


def _three_launches(q8, dev, norms, attn, layer_in, n_embd, n_ff, next_rows):
    h = q8.gemv_residual_f32(dev["o"], attn, layer_in, n_embd, n_embd)
    y = q8.ffn(dev["g"], dev["u"], dev["d"], h, n_ff, n_embd, n_embd, residual=h, norm_weight=to_dev(norms[0]), eps=EPS)
    nxt = q8.gemv_f32([dev[f"n{i}"] for i in range(len(next_rows))], y, list(next_rows), n_embd, norm_weight=to_dev(norms[1]), eps=EPS) if next_rows else []
    return h, y, list(nxt)


SHAPES = [
    (4096, 14336, (4096, 1024, 1024), False),  # LLaMA-3-8B block -> next block's q / k / v
    (512, 1536, (512, 128, 128), False),  # a small block: few strips everywhere
    (1024, 3584, (4000,), False),  # last block -> logits, a ragged vocabulary
    (2048, 5632, (), False),  # nothing behind the block
    (8192, 28672, (8192, 1024, 1024), False),  # LLaMA-3-70B block: a wave's three or four groups walked two at a time (another order of the sums than the separate launches')
    (8192, 3584, (1024, 256), False),  # the longest hidden state the one launch takes: four groups per wave, gate/up in two chunks of two groups of both matrices
    (4096, 9216, (8000,), False),  # a row-cut down stage with a long, ragged stage behind it
    (4096, 14336, (1024,), False),  # ... and with a short one
]


@pytest.mark.parametrize("n_embd,n_ff,next_rows,same_cut", SHAPES, ids=[f"{s[0]}x{s[1]}" for s in SHAPES])
def test_decode_layer_one_launch(q8, oracle, n_embd, n_ff, next_rows, same_cut):
    rng = np.random.default_rng(n_embd + n_ff)
    host, dev, norms = _weights(q8, rng, n_embd, n_ff, next_rows)
    attn = rng.standard_normal(n_embd).astype(np.float32)
    layer_in = rng.standard_normal(n_embd).astype(np.float32)
    d_attn, d_in = to_dev(attn), to_dev(layer_in)
    h, y, nxt = q8.decode_layer(dev["o"], d_attn, d_in, dev["g"], dev["u"], dev["d"], to_dev(norms[0]), [dev[f"n{i}"] for i in range(len(next_rows))], list(next_rows),
                                to_dev(norms[1]) if next_rows else None, EPS, n_embd, n_ff)
    g_gpu, u_gpu = (to_host(a) for a in q8.debug_ffn_gate_up(n_ff))
    h_gpu, y_gpu = to_host(h), to_host(y)
    assert np.isfinite(h_gpu).all() and np.isfinite(y_gpu).all()

    # (1) stage by stage: the checker on the launch's own previous stage
    assert rel_l2(h_gpu, oracle.gemv(host["o"][0], oracle.quantize_rows(attn[None, :])[0], n_embd, n_embd) + layer_in) <= REL_L2_TOL
    hq = oracle.rms_norm_quantize_rows(h_gpu[None, :], norms[0], EPS)[0]
    assert rel_l2(g_gpu, oracle.gemv(host["g"][0], hq, n_ff, n_embd)) <= REL_L2_TOL
    assert rel_l2(u_gpu, oracle.gemv(host["u"][0], hq, n_ff, n_embd)) <= REL_L2_TOL
    aq = oracle.silu_mul_quantize_rows(g_gpu[None, :], u_gpu[None, :])[0]
    assert rel_l2(y_gpu, oracle.gemv(host["d"][0], aq, n_embd, n_ff) + h_gpu) <= REL_L2_TOL
    if next_rows:
        yq = oracle.rms_norm_quantize_rows(y_gpu[None, :], norms[1], EPS)[0]
        for i, n in enumerate(next_rows):
            assert rel_l2(to_host(nxt[i]), oracle.gemv(host[f"n{i}"][0], yq, n, n_embd)) <= REL_L2_TOL, i

    # (2) the three launches it stands for
    h3, y3, nxt3 = _three_launches(q8, dev, norms, d_attn, d_in, n_embd, n_ff, next_rows)
    if same_cut:
        assert np.array_equal(h_gpu.view(np.uint32), to_host(h3).view(np.uint32))
        assert np.array_equal(y_gpu.view(np.uint32), to_host(y3).view(np.uint32))
        for a, b in zip(nxt, nxt3):
            assert np.array_equal(to_host(a).view(np.uint32), to_host(b).view(np.uint32))
    else:
        assert rel_l2(h_gpu, to_host(h3)) <= REL_L2_TOL
        assert rel_l2(y_gpu, to_host(y3)) <= 2e-3  # a quantizer sits between the stages: last-bit differences in h move single quants
        for a, b in zip(nxt, nxt3):
            assert rel_l2(to_host(a), to_host(b)) <= 2e-3


def test_decode_layer_launches_back_to_back_do_not_mix(q8, oracle):
    # a token's worth of launches on one stream without a wait in between, each block fed by the one before, then the same again
    # with one launch at a time: every word handed over inside a launch must be that launch's own
    n_embd, n_ff, next_rows, blocks = 1024, 3584, (1024, 256, 256), 6
    rng = np.random.default_rng(5)
    layers = [_weights(q8, rng, n_embd, n_ff, next_rows) for _ in range(blocks)]
    x0 = to_dev(rng.standard_normal(n_embd).astype(np.float32))

    def run(wait: bool):
        layer_in, attn, outs = x0, x0, []
        for host, dev, norms in layers:
            h, y, nxt = q8.decode_layer(dev["o"], attn, layer_in, dev["g"], dev["u"], dev["d"], to_dev(norms[0]), [dev[f"n{i}"] for i in range(3)], list(next_rows), to_dev(norms[1]), EPS,
                                        n_embd, n_ff)
            if wait:
                torch.cuda.synchronize()
            layer_in, attn = y, nxt[0]  # the next block's query stands in for its attention output
            outs.append((h, y, nxt))
        torch.cuda.synchronize()
        return [(to_host(h), to_host(y), [to_host(t) for t in nxt]) for h, y, nxt in outs]

    one_by_one = run(True)
    for _ in range(3):
        streamed = run(False)
        for (h0, y0, n0), (h1, y1, n1) in zip(one_by_one, streamed):
            assert np.array_equal(h0.view(np.uint32), h1.view(np.uint32)) and np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
            assert all(np.array_equal(a.view(np.uint32), b.view(np.uint32)) for a, b in zip(n0, n1))


def test_decode_layer_arguments(q8):
    lib = q8._lib.lib()
    n_embd, n_ff = 256, 512
    w = torch.zeros(q8.tiled_bytes(max(n_embd, n_ff), max(n_embd, n_ff)), dtype=torch.uint8, device="cuda")
    x = torch.zeros(n_embd, dtype=torch.float32, device="cuda")
    a, b = torch.zeros_like(x), torch.zeros_like(x)
    args = lambda ffn_inp, l_out, ne=n_embd, nf=n_ff: (w.data_ptr(), x.data_ptr(), x.data_ptr(), ffn_inp, w.data_ptr(), w.data_ptr(), w.data_ptr(), x.data_ptr(), l_out, None, None, None, 0,  # noqa: E731
                                                        None, 1e-5, ne, nf, None)
    import ctypes

    def call(t):
        t = list(t)
        t[14] = ctypes.c_float(t[14])
        return lib.nh_q8_0_decode_layer_f32(*t)

    assert call(args(a.data_ptr(), b.data_ptr())) == 0
    assert call(args(a.data_ptr(), a.data_ptr())) == -6  # ffn_inp and l_out must be distinct buffers
    assert call(args(None, b.data_ptr())) == -1
    assert call(args(a.data_ptr(), b.data_ptr(), ne=200)) == -3
    assert call(args(a.data_ptr() + 4, b.data_ptr())) == -2
    torch.cuda.synchronize()

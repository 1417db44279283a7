"""GPU: launches captured into a HIP graph and replayed.

A replay runs every kernel with the arguments it was recorded with.  The K-split hand-off of the mat-vec and the published
blocks of the one-launch FFN are tagged with a per-launch epoch that the host hands to the kernel, which a replay cannot
renew: the launchers therefore pick forms without per-launch state for a capturing stream (no K split in the mat-vec and its
2- and 3-row form, three launches for the FFN; the MFMA streaming kernel's arrival counters reset themselves).  The test
captures one of each on long-K shapes, where the eager forms do split, replays the graph several times with new inputs and
with eager launches of the same entry points in between, and checks every replay against the eager results.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def test_captured_launches_replay_with_new_inputs(q8, oracle):
    import torch

    from nihilus_amd import _lib

    _lib.check("nh_q8_0_prepare", _lib.lib().nh_q8_0_prepare())  # every internal buffer exists before the capture starts
    rng = np.random.default_rng(11)
    n, k = 1024, 14336  # a down-projection-like shape: split over workgroups when launched eagerly
    n_ff, kf, n_out = 4096, 1024, 512
    w = q8.tile(to_dev(random_blocks(rng, n, k, 1e-3)), n, k)
    wg, wu = (q8.tile(to_dev(random_blocks(rng, n_ff, kf, 1e-3)), n_ff, kf) for _ in range(2))
    wd = q8.tile(to_dev(random_blocks(rng, n_out, n_ff, 1e-3)), n_out, n_ff)
    x1 = torch.zeros(k, dtype=torch.float32, device="cuda")
    x8 = torch.zeros((8, k), dtype=torch.float32, device="cuda")
    xf = torch.zeros(kf, dtype=torch.float32, device="cuda")
    res = to_dev(rng.standard_normal(n_out).astype(np.float32))

    def launches():
        return (q8.gemv_f32(w, x1, n, k), q8.mul_mat(w, x8[:3], n, k), q8.mul_mat(w, x8, n, k), q8.ffn(wg, wu, wd, xf, n_ff, kf, n_out, residual=res),
                q8.mul_mat_f32_activations(w, x1, n, k))  # one row of a long K: split over workgroups eagerly, unsplit under capture

    def new_inputs(seed):
        x8.copy_(to_dev(oracle.fill_activations(seed, 8 * k).reshape(8, k)))
        x1.copy_(x8[5])
        xf.copy_(to_dev(oracle.fill_activations(seed + 1000, kf)))

    new_inputs(1)
    launches()  # warm-up outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = launches()
    for seed in (2, 3, 4, 5):
        new_inputs(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [to_host(t).copy() for t in captured]
        want = [to_host(t) for t in launches()]  # eager: the split forms, with fresh epochs, between the replays
        torch.cuda.synchronize()
        for i, (g, e) in enumerate(zip(got[:3], want[:3])):
            assert rel_l2(g, e) < 2e-6, (seed, i)  # same arithmetic, different cut of K
        assert rel_l2(got[3], want[3]) <= 1e-3, seed  # a quantizer sits between the FFN's stages
        assert np.isfinite(got[3]).all()
        assert rel_l2(got[4], want[4]) < 2e-6, seed
    # and against the checker once, so that "equal to eager" cannot hide a common mistake
    aq = oracle.quantize_rows(to_host(x1))[0]
    assert rel_l2(got[0], oracle.gemv(to_host(q8.untile(w, n, k)), aq, n, k)) <= REL_L2_TOL


def test_captured_decode_layer_replays_with_new_inputs(q8, oracle):
    # the chained decode layer hands data between its stages under a per-launch epoch: a capturing stream gets the three launches it
    # stands for (themselves in their replay-safe forms); replays must follow new inputs and agree with the eager one-launch form
    import torch

    from nihilus_amd import _lib

    _lib.check("nh_q8_0_prepare", _lib.lib().nh_q8_0_prepare())
    rng = np.random.default_rng(23)
    n_embd, n_ff, nxt = 1024, 3584, [1024, 256]
    sig = lambda k_in: 1.0 / (58.0 * np.sqrt(k_in))  # noqa: E731
    ws = {name: q8.tile(to_dev(random_blocks(rng, n, k, sig(k))), n, k) for name, n, k in
          [("o", n_embd, n_embd), ("g", n_ff, n_embd), ("u", n_ff, n_embd), ("d", n_embd, n_ff), ("q", 1024, n_embd), ("k", 256, n_embd)]}
    norm1 = to_dev((1.0 + 0.1 * rng.standard_normal(n_embd)).astype(np.float32))
    norm2 = to_dev((1.0 + 0.1 * rng.standard_normal(n_embd)).astype(np.float32))
    attn = torch.zeros(n_embd, dtype=torch.float32, device="cuda")
    x = torch.zeros(n_embd, dtype=torch.float32, device="cuda")

    def launch():
        h, y, outs = q8.decode_layer(ws["o"], attn, x, ws["g"], ws["u"], ws["d"], norm1, [ws["q"], ws["k"]], nxt, norm2, 1e-5, n_embd, n_ff)
        return [h, y, *outs]

    def new_inputs(seed):
        attn.copy_(to_dev(oracle.fill_activations(seed, n_embd)))
        x.copy_(to_dev(oracle.fill_activations(seed + 500, n_embd)))

    new_inputs(1)
    launch()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = launch()
    for seed in (2, 3, 4):
        new_inputs(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [to_host(t).copy() for t in captured]
        want = [to_host(t) for t in launch()]  # eager: one launch, fresh epoch, between the replays
        torch.cuda.synchronize()
        assert rel_l2(got[0], want[0]) < 2e-6, seed  # attn_out + residual: same arithmetic, another cut
        for g, e in zip(got[1:], want[1:]):
            assert np.isfinite(g).all() and rel_l2(g, e) <= 2e-3, seed  # quantizers sit between the stages


def test_captured_batch_of_independent_mat_vecs(q8, oracle):
    # a batch call whose entries the runner may group: under capture the short-K ones still share a launch (no per-launch
    # state when K is not split), the long-K one falls back to its own unsplit launch; replays must follow new inputs
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    _lib.check("nh_q8_0_prepare", lib.nh_q8_0_prepare())
    shapes = [(2048, 1024), (1024, 1024), (512, 14336)]
    ws = [q8.tile(q8.fill_weight_blocks(90 + i, n, k), n, k) for i, (n, k) in enumerate(shapes)]
    xs = [torch.zeros(k, dtype=torch.float32, device="cuda") for _, k in shapes]
    ys = [torch.zeros(n, dtype=torch.float32, device="cuda") for n, _ in shapes]
    ops = (_lib.MulMatOp * 3)()
    for i, (n, k) in enumerate(shapes):
        ops[i] = _lib.MulMatOp(ws[i].data_ptr(), xs[i].data_ptr(), ys[i].data_ptr(), 1, n, k, 0, 0)
    dummy = torch.empty(256, dtype=torch.uint8, device="cuda")

    def call():
        _lib.check("nh_q8_0_mul_mat_batch", lib.nh_q8_0_mul_mat_batch(ops, 3, dummy.data_ptr(), dummy.numel(), torch.cuda.current_stream().cuda_stream))

    def new_inputs(seed):
        for i, (_, k) in enumerate(shapes):
            xs[i].copy_(to_dev(oracle.fill_activations(seed + i, k)))

    new_inputs(1)
    call()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for seed in (10, 20, 30):
        new_inputs(seed)
        graph.replay()
        torch.cuda.synchronize()
        got = [to_host(y).copy() for y in ys]
        call()  # eager, with the K split and fresh epochs, between the replays
        torch.cuda.synchronize()
        for i in range(3):
            assert rel_l2(got[i], to_host(ys[i])) < 2e-6, (seed, i)
    aq = oracle.quantize_rows(to_host(xs[2]).reshape(1, -1))[0]
    assert rel_l2(got[2], oracle.gemv(to_host(q8.untile(ws[2], *shapes[2])), aq, *shapes[2])) <= REL_L2_TOL


def test_eager_split_launch_on_another_stream_while_a_stream_captures(q8, oracle):
    # Global-mode capture (torch's default) refuses stream queries from the capturing thread and a refused call invalidates the
    # capture.  The scratch's one-stream guard queries the stream of the previous K-split launch: it has to do so without
    # disturbing a capture that is going on elsewhere in the thread.
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    _lib.check("nh_q8_0_prepare", lib.nh_q8_0_prepare())
    n, k = 1024, 14336  # K split over workgroups when launched eagerly
    w = oracle.fill_weights(21, n, k)
    x = oracle.fill_activations(21, k)
    wt, xd = q8.tile(to_dev(w), n, k), to_dev(x)
    y_c = torch.empty(n, dtype=torch.float32, device="cuda")
    y_b = torch.empty(n, dtype=torch.float32, device="cuda")
    y_g = torch.empty(n, dtype=torch.float32, device="cuda")
    b, c = torch.cuda.Stream(), torch.cuda.Stream()
    assert lib.nh_q8_0_gemv_tiled_f32(wt.data_ptr(), xd.data_ptr(), y_c.data_ptr(), n, k, c.cuda_stream) == 0  # the scratch's user is now stream c
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        cap = torch.cuda.current_stream().cuda_stream
        assert lib.nh_q8_0_gemv_tiled_f32(wt.data_ptr(), xd.data_ptr(), y_g.data_ptr(), n, k, cap) == 0  # captured: the unsplit form
        # eager, on stream b, in the middle of the capture: the guard looks at stream c
        assert lib.nh_q8_0_gemv_tiled_f32(wt.data_ptr(), xd.data_ptr(), y_b.data_ptr(), n, k, b.cuda_stream) == 0
    b.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    want = oracle.gemv(w, oracle.quantize_rows(x)[0], n, k)
    assert rel_l2(to_host(y_b), want) <= REL_L2_TOL and np.array_equal(to_host(y_b), to_host(y_c))
    assert rel_l2(to_host(y_g), want) <= REL_L2_TOL

"""GPU: independent mat-vecs sharing one launch (nh_q8_0_gemv_tiled_group_f32) and the batch runner's use of it.

A grouped matrix is cut exactly as its own launch would cut it, so against separate launches the results are bit-identical
whenever the separate launch does not split the strip by rows (a form only small unsplit matrices take), and equal to fp32
summation order otherwise; against the CPU checker they meet the fp32 contract.  The batch runner may only group entries
whose x and y ranges show them independent: a batch with read-after-write, write-after-write and write-after-read
neighbours, and one with the `ordered` mark, must give what running the entries one after another gives.
"""
import ctypes as C

import numpy as np
import pytest

from helpers import REL_L2_TOL, random_blocks, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

FFN_TRIO = [(14336, 4096), (14336, 4096), (4096, 14336)]
LAYER = [(4096, 4096), (1024, 4096), (1024, 4096), (4096, 4096), (14336, 4096), (14336, 4096), (4096, 14336)]
RAGGED = [(1000, 1024), (33, 128), (4096, 14336), (1, 256), (777, 3584), (64, 28672), (2048, 8192), (31, 128), (500, 512), (96, 2048)]  # more than one group's worth


def _launch_count(lib, fn):
    import torch

    from nihilus_amd import _lib

    torch.cuda.synchronize()
    _lib.check("nh_profile_begin", lib.nh_profile_begin(1, 64))
    fn()
    tot, cnt, mn, mx = C.c_double(), C.c_int64(), C.c_double(), C.c_double()
    _lib.check("nh_profile_end", lib.nh_profile_end(C.byref(tot), C.byref(cnt), C.byref(mn), C.byref(mx)))
    return cnt.value


@pytest.mark.parametrize("shapes", [FFN_TRIO, LAYER, RAGGED], ids=["ffn_trio", "layer", "ragged"])
def test_group_equals_separate_launches(q8, oracle, shapes):
    from nihilus_amd import _lib

    ws = [q8.tile(q8.fill_weight_blocks(60 + i, n, k), n, k) for i, (n, k) in enumerate(shapes)]
    xs = [q8.fill_activations(80 + i, k) for i, (_, k) in enumerate(shapes)]
    ns, ks = [n for n, _ in shapes], [k for _, k in shapes]
    res = [to_dev(np.random.default_rng(i).standard_normal(n).astype(np.float32)) if i % 3 == 2 else None for i, (n, _) in enumerate(shapes)]
    ys = None

    def grouped():
        nonlocal ys
        ys = q8.gemv_group_f32(ws, xs, ns, ks, residuals=res)

    launches = _launch_count(_lib.lib(), grouped)
    assert launches == (len(shapes) + 7) // 8
    for i, (n, k) in enumerate(shapes):
        single = q8.gemv_f32(ws[i], xs[i], n, k) if res[i] is None else q8.gemv_residual_f32(ws[i], xs[i], res[i], n, k)
        strips, tiles = (n + 31) // 32, (k // 128 + 15) // 16
        if tiles > 4 or strips * 2 > 256:  # the separate launch splits K (as the group does) or runs whole strips: same arithmetic, same order
            assert (ys[i] == single).all(), (i, n, k)
        else:
            assert rel_l2(to_host(ys[i]), to_host(single)) < 2e-6, (i, n, k)
    # and against the checker, for the matrices it finishes quickly
    for i, (n, k) in enumerate(shapes):
        if n * k <= 4096 * 4096:
            w = to_host(q8.untile(ws[i], n, k))
            want = oracle.gemv(w, oracle.quantize_rows(to_host(xs[i]).reshape(1, k))[0], n, k) + (0 if res[i] is None else to_host(res[i]))
            assert rel_l2(to_host(ys[i]), want) <= REL_L2_TOL, (i, n, k)


def test_group_in_place_residual_and_empty_entries(q8):
    # a residual that is the op's own output (in-place accumulate) beside K == 0 and N == 0 entries
    import torch

    n, k = 4096, 14336  # split over workgroups: several of them store the row
    w = q8.tile(q8.fill_weight_blocks(7, n, k), n, k)
    x = q8.fill_activations(8, k)
    acc = q8.fill_activations(9, n)
    want = q8.gemv_f32(w, x, n, k) + acc
    y0 = torch.full((64,), float("nan"), dtype=torch.float32, device="cuda")
    empty = torch.empty(0, dtype=torch.float32, device="cuda")
    ew = torch.empty(0, dtype=torch.uint8, device="cuda")
    q8.gemv_group_f32([w, ew, ew], [x, empty, x[:128].contiguous()], [n, 64, 0], [k, 0, 128], residuals=[acc, None, None], outs=[acc, y0, empty])
    assert (acc == want).all()
    assert (y0 == 0).all()  # an empty dot product


def test_batch_runner_groups_independent_entries_only(q8, oracle):
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(5)
    k = n = 512  # square, so that outputs can feed inputs
    ws_host = [random_blocks(rng, n, k, 1.0 / (58.0 * np.sqrt(k))) for _ in range(4)]
    ws = [q8.tile(to_dev(w), n, k) for w in ws_host]
    x0 = q8.fill_activations(3, k)
    dummy = torch.empty(256, dtype=torch.uint8, device="cuda")

    def batch(entries):
        ops = (_lib.MulMatOp * len(entries))()
        for i, (w, x, y, ordered) in enumerate(entries):
            ops[i] = _lib.MulMatOp(w.data_ptr(), x.data_ptr(), y.data_ptr(), 1, n, k, 0, ordered)
        return _launch_count(lib, lambda: _lib.check("nh_q8_0_mul_mat_batch", lib.nh_q8_0_mul_mat_batch(ops, len(entries), dummy.data_ptr(), dummy.numel(), stream)))

    def fresh():
        return torch.full((n,), float("nan"), dtype=torch.float32, device="cuda")

    # four independent entries with different inputs: one launch
    xs = [q8.fill_activations(20 + i, k) for i in range(4)]
    ys = [fresh() for _ in range(4)]
    assert batch([(ws[i], xs[i], ys[i], 0) for i in range(4)]) == 1
    for i in range(4):
        assert rel_l2(to_host(ys[i]), to_host(q8.gemv_f32(ws[i], xs[i], n, k))) < 2e-6

    # the same with the second pair marked ordered: three launches (the first two still share one)
    ys2 = [fresh() for _ in range(4)]
    assert batch([(ws[i], xs[i], ys2[i], 1 if i >= 2 else 0) for i in range(4)]) == 3
    for i in range(4):
        assert rel_l2(to_host(ys2[i]), to_host(ys[i])) < 2e-6

    # read after write: a chain y1 = W1 . Q(W0 . Q(x0)), then an entry that overwrites the chain's input (write after read),
    # then two entries writing the same output (write after write: the later one stays)
    y_a, y_b, y_c = fresh(), fresh(), fresh()
    x_in = x0.clone()
    launches = batch([(ws[0], x_in, y_a, 0), (ws[1], y_a, y_b, 0), (ws[2], xs[0], x_in, 0), (ws[3], xs[1], y_c, 0), (ws[0], xs[2], y_c, 0)])
    assert launches == 3  # [first] [second, third, fourth: independent of each other] [fifth]
    want_a = q8.gemv_f32(ws[0], x0, n, k)
    assert rel_l2(to_host(y_a), to_host(want_a)) < 2e-6
    assert rel_l2(to_host(y_b), to_host(q8.gemv_f32(ws[1], want_a, n, k))) < 1e-3  # a quantizer between the stages
    assert rel_l2(to_host(x_in), to_host(q8.gemv_f32(ws[2], xs[0], n, k))) < 2e-6
    assert rel_l2(to_host(y_c), to_host(q8.gemv_f32(ws[0], xs[2], n, k))) < 2e-6
    # and the chain's first stage against the checker
    assert rel_l2(to_host(y_a), oracle.gemv(ws_host[0], oracle.quantize_rows(to_host(x0).reshape(1, k))[0], n, k)) <= REL_L2_TOL


@pytest.mark.parametrize("seed", range(6))
def test_batch_runner_random_dependency_patterns(q8, seed):
    # random lists of M = 1 entries over a small pool of buffers, so that reads-after-writes, writes-after-reads and
    # writes-after-writes occur in every position; the batch call must leave the pool exactly as one-by-one execution in
    # list order does.  The shape is one whose single launch and grouped form do the same arithmetic in the same order
    # (132 strips: no row split), so "exactly" means bit for bit however deep the chains get.
    import torch

    from nihilus_amd import _lib

    lib = _lib.lib()
    rng = np.random.default_rng(300 + seed)
    d = 4224
    hw = [random_blocks(rng, d, d, 1.0 / (58.0 * np.sqrt(d))) for _ in range(4)]  # about unit gain, so chains stay finite
    ws = [q8.tile(to_dev(w), d, d) for w in hw]
    pool0 = [q8.fill_activations(600 + i, d) for i in range(5)]
    entries = []
    for _ in range(14):
        src, dst = rng.choice(5, size=2, replace=False)
        entries.append((int(rng.integers(0, 4)), int(src), int(dst), int(rng.integers(0, 4) == 0)))
    pool = [p.clone() for p in pool0]
    ops = (_lib.MulMatOp * len(entries))()
    for i, (wi, src, dst, ordered) in enumerate(entries):
        ops[i] = _lib.MulMatOp(ws[wi].data_ptr(), pool[src].data_ptr(), pool[dst].data_ptr(), 1, d, d, 0, ordered)
    dummy = torch.empty(256, dtype=torch.uint8, device="cuda")
    _lib.check("nh_q8_0_mul_mat_batch", lib.nh_q8_0_mul_mat_batch(ops, len(entries), dummy.data_ptr(), dummy.numel(), torch.cuda.current_stream().cuda_stream))
    ref2 = [p.clone() for p in pool0]  # one by one, in list order
    for wi, src, dst, _ in entries:
        ref2[dst].copy_(q8.gemv_f32(ws[wi], ref2[src], d, d))
    for i in range(5):
        a, b = to_host(pool[i]), to_host(ref2[i])
        assert np.isfinite(b).all() and np.array_equal(a, b), (seed, i, entries)

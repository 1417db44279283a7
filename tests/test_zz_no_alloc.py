"""GPU: the mat-vec entry point that allocates nothing (nh_q8_0_gemv_tiled_f32_noalloc) against nh_q8_0_gemv_tiled_f32.

Same kernels and the same cut of the matrix, so y must be the same bits.  Two calls in a row share the built-in array, the
second with a smaller input; shapes with and without a K split; a shape whose cut does not fit the array is rejected before
anything is launched.  Runs through the C ABI; collected last so that a failure here cannot hide another test.
"""
import numpy as np
import pytest
import torch

from helpers import REL_L2_TOL, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def _both(lib, wt, x, n, k, stream):
    y_ref = torch.full((n,), float("nan"), dtype=torch.float32, device="cuda")
    y_new = torch.full((n,), float("nan"), dtype=torch.float32, device="cuda")
    assert lib.nh_q8_0_gemv_tiled_f32(wt.data_ptr(), x.data_ptr(), y_ref.data_ptr(), n, k, stream) == 0
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(wt.data_ptr(), x.data_ptr(), y_new.data_ptr(), n, k, stream) == 0
    return to_host(y_ref), to_host(y_new)


def test_no_alloc_mat_vec_allocates_nothing(q8):
    # Free device memory must not move across a call whose K split needs the hand-off array.  A first call on a shape without
    # a split gets the runtime's own first-launch set-up out of the way (code object, kernel-argument pool); run alone in a
    # fresh process, no allocating entry point has been called before this point, so a hidden hipMalloc would show.
    lib = q8._lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    n0, k0, n, k = 14336, 4096, 4096, 14336
    w0 = torch.zeros(q8.tiled_bytes(n0, k0), dtype=torch.uint8, device="cuda")
    w = torch.zeros(q8.tiled_bytes(n, k), dtype=torch.uint8, device="cuda")
    x = torch.ones(max(k0, k), dtype=torch.float32, device="cuda")
    y = torch.empty(max(n0, n), dtype=torch.float32, device="cuda")
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(w0.data_ptr(), x.data_ptr(), y.data_ptr(), n0, k0, stream) == 0
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(2):
        assert lib.nh_q8_0_gemv_tiled_f32_noalloc(w.data_ptr(), x.data_ptr(), y.data_ptr(), n, k, stream) == 0
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before, (free_before, free_after)
    assert bool((y[:n] == 0).all())


def test_no_alloc_mat_vec_refuses_a_second_stream_while_the_first_is_busy(q8):
    # the built-in array serves one stream at a time, like the allocated scratch
    lib = q8._lib.lib()
    n, k = 4096, 14336
    w = torch.zeros(q8.tiled_bytes(n, k), dtype=torch.uint8, device="cuda")
    x = torch.ones(k, dtype=torch.float32, device="cuda")
    y_a = torch.empty(n, dtype=torch.float32, device="cuda")
    y_b = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    a, b = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    rc, still_running, batch = None, False, 300
    while not still_running and batch <= 30000:
        a.synchronize()
        for _ in range(batch):
            assert lib.nh_q8_0_gemv_tiled_f32_noalloc(w.data_ptr(), x.data_ptr(), y_a.data_ptr(), n, k, a.cuda_stream) == 0
        rc = lib.nh_q8_0_gemv_tiled_f32_noalloc(w.data_ptr(), x.data_ptr(), y_b.data_ptr(), n, k, b.cuda_stream)
        still_running = not a.query()
        if rc == 0:
            b.synchronize()
            y_b.fill_(7.0)
            torch.cuda.synchronize()
        batch *= 10
    if not still_running:
        pytest.skip("stream a drains faster than this host enqueues: the overlap could not be set up")
    assert rc == -10, rc  # NH_ERR_BUSY
    torch.cuda.synchronize()
    assert bool((y_b == 7.0).all())  # nothing was launched
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(w.data_ptr(), x.data_ptr(), y_b.data_ptr(), n, k, b.cuda_stream) == 0
    torch.cuda.synchronize()
    assert bool((y_b == 0).all())


def test_no_alloc_mat_vec_matches_the_allocating_one(q8, oracle):
    lib = q8._lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    # first call: LLaMA-3-8B down projection (K split over 4 workgroups per strip: 512 slots of the array);
    # second call, smaller: [1024 x 8192] (K split, 256 slots), then shapes with no split and a ragged N
    for n, k in [(4096, 14336), (1024, 8192), (4096, 4096), (14336, 4096), (100, 14336), (33, 128)]:
        w = oracle.fill_weights(n + k, n, k)
        x = oracle.fill_activations(n, k)
        wt = q8.tile(to_dev(w), n, k)
        y_ref, y_new = _both(lib, wt, to_dev(x), n, k, stream)
        assert np.array_equal(y_new.view(np.uint32), y_ref.view(np.uint32)), (n, k)
        assert rel_l2(y_new, oracle.gemv(w, oracle.quantize_rows(x)[0], n, k)) <= REL_L2_TOL, (n, k)
    # the same pair again, back to back on one stream, results checked after both: the second must not see the first's tags
    shapes = [(4096, 14336), (1024, 8192)]
    keep = []
    for n, k in shapes:
        w = oracle.fill_weights(n * 3 + k, n, k)
        x = oracle.fill_activations(n + 1, k)
        wt, xd = q8.tile(to_dev(w), n, k), to_dev(x)
        y = torch.full((n,), float("nan"), dtype=torch.float32, device="cuda")
        assert lib.nh_q8_0_gemv_tiled_f32_noalloc(wt.data_ptr(), xd.data_ptr(), y.data_ptr(), n, k, stream) == 0
        keep.append((w, x, wt, xd, y, n, k))
    for w, x, wt, xd, y, n, k in keep:
        y_ref = torch.empty(n, dtype=torch.float32, device="cuda")
        assert lib.nh_q8_0_gemv_tiled_f32(wt.data_ptr(), xd.data_ptr(), y_ref.data_ptr(), n, k, stream) == 0
        assert np.array_equal(to_host(y).view(np.uint32), to_host(y_ref).view(np.uint32)), (n, k)


def test_no_alloc_mat_vec_rejects_what_does_not_fit(q8):
    lib = q8._lib.lib()
    stream = torch.cuda.current_stream().cuda_stream
    n, k = 16384, 28672  # 512 strips x 8 K parts = 4096 slots > 2048
    wt = torch.empty(q8.tiled_bytes(n, k), dtype=torch.uint8, device="cuda")
    x = torch.zeros(k, dtype=torch.float32, device="cuda")
    y = torch.full((n,), 7.0, dtype=torch.float32, device="cuda")
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(wt.data_ptr(), x.data_ptr(), y.data_ptr(), n, k, stream) == -5  # NH_ERR_TOO_LARGE
    torch.cuda.synchronize()
    assert bool((y == 7.0).all())  # nothing was launched
    # argument checks as in the allocating entry point
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(wt.data_ptr(), x.data_ptr(), y.data_ptr(), 32, 100, stream) == -3
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(None, x.data_ptr(), y.data_ptr(), 32, 128, stream) == -1
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(wt.data_ptr(), x.data_ptr(), y.data_ptr() + 4, 32, 128, stream) == -2
    assert lib.nh_q8_0_gemv_tiled_f32_noalloc(wt.data_ptr(), x.data_ptr(), y.data_ptr(), 0, 128, stream) == 0

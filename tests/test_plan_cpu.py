"""CPU: the kernel each mul_mat shape runs is decided by one host-side plan function, exposed through the C ABI
(nh_q8_0_debug_plan_mul_mat).  The launchers execute that plan, so pinning it here pins the route of every benchmark shape:
a change of a threshold that moves one of them shows up as a failure of this file, not as a silent change of what a parity
test covers.  No GPU needed."""
import pytest

from nihilus_amd import q8_0

L8B = {"q_o": (4096, 4096), "k_v": (1024, 4096), "gate_up": (14336, 4096), "down": (4096, 14336), "lm_head": (128256, 4096)}
L70B = {"q_o": (8192, 8192), "k_v": (1024, 8192), "gate_up": (28672, 8192), "down": (8192, 28672), "lm_head": (128256, 8192)}


def kernel(m, n, k):
    return q8_0.plan_mul_mat(m, n, k)["kernel"]


def test_decode_rows_never_leave_the_mat_vec_kernel():
    for n, k in list(L8B.values()) + list(L70B.values()):
        p = q8_0.plan_mul_mat(1, n, k)
        assert p["kernel"] == "gemv" and not p["quantize_launch"], (n, k)
        for m in (2, 3):
            p = q8_0.plan_mul_mat(m, n, k)
            assert p["kernel"] == "gemv_rows" and not p["quantize_launch"], (m, n, k)


def test_mat_vec_cut_of_the_decode_shapes():
    # (K splits, groups per wave, row parts): long K goes over several workgroups, few strips are cut by rows, never both
    want = {(4096, 4096): (1, 2, 2), (1024, 4096): (1, 2, 4), (14336, 4096): (1, 2, 1), (4096, 14336): (4, 2, 1), (128256, 4096): (1, 2, 1),
            (8192, 8192): (1, 4, 1), (1024, 8192): (1, 4, 4), (28672, 8192): (1, 4, 1), (8192, 28672): (8, 2, 1), (128256, 8192): (1, 4, 1),
            (6144, 4096): (1, 2, 1)}
    for (n, k), (splits, tiles, parts) in want.items():
        p = q8_0.plan_mul_mat(1, n, k)
        assert (p["k_splits"], p["groups_per_wave"], p["row_parts"]) == (splits, tiles, parts), (n, k, p)


def test_four_to_sixteen_rows_on_small_matrices_take_the_mfma_mat_vec():
    # no quantize launch, no workspace: up to 16 rows on matrices of at most 40 MB, 4 rows up to 80 MB; beyond that the quantize launch
    # and the MFMA kernels (every strip's workgroup quantizing the rows again would cost more than the launch)
    for n, k in (L8B["q_o"], L8B["k_v"], L70B["k_v"]):
        for m in (4, 5, 8, 9, 16):
            p = q8_0.plan_mul_mat(m, n, k)
            assert p["kernel"] == "gemv_rows_mfma" and not p["quantize_launch"], (m, n, k)
        assert kernel(17, n, k) == "gemm_skinny"
    for n, k in (L8B["gate_up"], L8B["down"], L70B["q_o"]):
        assert kernel(4, n, k) == "gemv_rows_mfma" and kernel(5, n, k) != "gemv_rows_mfma" and kernel(8, n, k) != "gemv_rows_mfma"
    for n, k in (L70B["gate_up"], L70B["down"], L70B["lm_head"], L8B["lm_head"]):
        assert kernel(4, n, k) not in ("gemv_rows", "gemv_rows_mfma")
    # its cut: a workgroup per CU where K allows it, a wave at most two groups
    assert q8_0.plan_mul_mat(8, 4096, 4096)["k_splits"] == 2 and q8_0.plan_mul_mat(8, 4096, 4096)["groups_per_wave"] == 1
    assert q8_0.plan_mul_mat(4, 1024, 8192)["k_splits"] == 4
    assert q8_0.plan_mul_mat(4, 14336, 4096)["k_splits"] == 1 and q8_0.plan_mul_mat(4, 14336, 4096)["groups_per_wave"] == 2
    # nine to sixteen rows: one group per wave at a time (the rows' fp32 slices share the registers with the weight tiles)
    assert q8_0.plan_mul_mat(16, 4096, 4096)["k_splits"] == 2 and q8_0.plan_mul_mat(16, 4096, 4096)["groups_per_wave"] == 1
    assert q8_0.plan_mul_mat(16, 1024, 8192)["k_splits"] == 4


def test_crossover_shapes():
    # BASELINE configs[2]: M in {1, 8, 32, 128, 512} on [4096 x 4096] and [14336 x 4096]
    assert [kernel(m, 4096, 4096) for m in (1, 8, 32, 128, 512)] == ["gemv", "gemv_rows_mfma", "gemm_skinny", "gemm_skinny", "gemm_tile"]
    assert [kernel(m, 14336, 4096) for m in (1, 8, 32, 128, 512)] == ["gemv", "gemm_skinny", "gemm_skinny", "gemm_tile", "gemm_tile"]
    p = q8_0.plan_mul_mat(512, 4096, 4096)  # a grid short of four waves per SIMD: four K sets per workgroup
    assert (p["activation_strips"], p["k_sets"], p["k_splits"], p["grid"]) == (2, 4, 1, (32, 8))
    p = q8_0.plan_mul_mat(512, 14336, 4096)
    assert (p["activation_strips"], p["k_sets"], p["k_splits"], p["grid"]) == (2, 1, 1, (112, 8))


def test_batched_decode_at_the_70b_shapes():
    # BASELINE configs[4]: M in {4, 16, 64}
    want = {
        "q_o": ["gemv_rows_mfma", "gemm_tile_stream", "gemm_tile_stream"],
        "k_v": ["gemv_rows_mfma", "gemv_rows_mfma", "gemm_skinny"],
        "gate_up": ["gemm_tile_stream"] * 3,
        "down": ["gemm_skinny", "gemm_tile_stream", "gemm_tile_stream"],
        "lm_head": ["gemm_tile_stream"] * 3,
    }
    for name, (n, k) in L70B.items():
        assert [kernel(m, n, k) for m in (4, 16, 64)] == want[name], name
    # matrices with few column blocks reach every CU through a K split over workgroups
    for name in ("q_o", "down"):
        p = q8_0.plan_mul_mat(64, *L70B[name])
        assert p["k_sets"] == 4 and p["k_splits"] == 4 and p["grid"] == (64, 1), p
    assert q8_0.plan_mul_mat(64, *L70B["gate_up"])["k_splits"] == 1


def test_tile_kernel_is_not_chosen_where_its_k_split_cannot_be_made():
    # 33..64 rows, 32..191 column blocks, >= 48 Mi weights: the tile kernel only with K over several workgroups; a shape whose
    # K does not divide that way keeps the weight-streaming kernel (an unsplit tile grid of 160 workgroups on 256 CUs is the
    # form measured slower)
    assert kernel(64, 20480, 4096) == "gemm_skinny"
    assert kernel(64, 14336, 4096) == "gemm_tile_stream" and q8_0.plan_mul_mat(64, 14336, 4096)["k_splits"] == 2
    # K = 4096 + 128: 33 groups, no K set divides them
    assert kernel(64, 14336, 4224) == "gemm_skinny"


def test_empty_and_rejected_shapes():
    assert kernel(0, 4096, 4096) == "nothing" and kernel(4, 0, 4096) == "nothing" and kernel(4, 4096, 0) == "nothing"
    with pytest.raises(q8_0._lib.Q8Error):
        q8_0.plan_mul_mat(4, 4096, 100)
    with pytest.raises(q8_0._lib.Q8Error):
        q8_0.plan_mul_mat(-1, 4096, 4096)

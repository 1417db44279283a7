"""GPU: the prefill FFN's first half as one call (nh_q8_0_gemm_tiled_gate_up_silu): gate and up mat-mats, SiLU * up and the
quantizer of the down projection's activation.

Where the fused MFMA kernel takes the shape (workspace bytes == 0) the quantized activation is compared, byte for byte, with the
CPU quantizer applied to the fp32 gate / up sums that the launch itself computed (dumped through the debug entry), those sums with
the CPU mat-mat (1e-4), and the bytes with the three-call sequence the call stands for (where that sequence sums K in the same order).  Shapes the fused kernel does not take go
through that sequence inside the call.
"""
import numpy as np
import pytest

from helpers import REL_L2_TOL, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu

# (M, n_ff, K, fused)
SHAPES = [
    (200, 16384, 1024, True),  # two activation strips per wave, a ragged last strip (200 = 6 * 32 + 8)
    (512, 14336, 512, True),  # the benchmark's M and n_ff at a short K
    (65, 16384, 384, True),  # three groups: no K sets possible; 65 rows = two full strips + one row
    (130, 2816, 1024, False),  # too few tiles for the prefill kernel: the three-call sequence inside
    (37, 3584, 1024, False),
]


@pytest.mark.parametrize("m,n_ff,k,fused", SHAPES, ids=[f"{s[0]}x{s[1]}x{s[2]}" for s in SHAPES])
def test_gate_up_silu(q8, oracle, m, n_ff, k, fused):
    lib = q8._lib.lib()
    assert (lib.nh_q8_0_gate_up_silu_workspace_bytes(m, n_ff, k) == 0) == fused
    wg, wu = oracle.fill_weights(11 + m, n_ff, k), oracle.fill_weights(12 + m, n_ff, k)
    x = oracle.fill_activations(m + k, m * k).reshape(m, k)
    aq_cpu = oracle.quantize_rows(x)
    tg, tu = q8.tile(to_dev(wg), n_ff, k), q8.tile(to_dev(wu), n_ff, k)
    aq = q8.quantize_row_q8_0(to_dev(x), tiled=True)

    def cpu_mm(w):  # the threaded checker takes block counts that are multiples of 16
        return oracle.gemm(w, aq_cpu, m, n_ff, k, threads=8) if (k // 32) % 16 == 0 else oracle.gemm(w, aq_cpu, m, n_ff, k)

    act, gate, up = q8.gate_up_silu(tg, tu, aq, m, n_ff, k, debug=True)
    gate, up = to_host(gate), to_host(up)
    # the two mat-mats against the checker
    assert rel_l2(gate, cpu_mm(wg)) <= REL_L2_TOL
    assert rel_l2(up, cpu_mm(wu)) <= REL_L2_TOL
    # the quantized activation: the checker's SiLU * up quantizer on the launch's own sums, byte for byte
    act_blocks = to_host(q8.untile(act, m, n_ff)).reshape(m, -1)
    assert np.array_equal(act_blocks, oracle.silu_mul_quantize_rows(gate, up))
    # rows past M of the last strip are zero blocks, as the stand-alone quantizer leaves them
    padded = (m + 31) // 32 * 32
    if padded > m:
        whole = to_host(q8.untile(act, padded, n_ff)).reshape(padded, -1)
        assert not whole[m:].any()
    # the production entry (no fp32 copies) writes the same bytes, and so does the three-call sequence it stands for
    act2 = q8.gate_up_silu(tg, tu, aq, m, n_ff, k)
    assert np.array_equal(to_host(act2), to_host(act))
    g3, u3 = q8.gemm(tg, aq, m, n_ff, k, tiled=True), q8.gemm(tu, aq, m, n_ff, k, tiled=True)
    plan = q8.plan_mul_mat(m, n_ff, k)
    if not fused or plan.get("k_sets") == 1:
        # the single mat-mat cuts K the same way (one K set per workgroup): same fp32 sums, hence the same bytes
        assert np.array_equal(to_host(g3).view(np.uint32), gate.view(np.uint32)) and np.array_equal(to_host(u3).view(np.uint32), up.view(np.uint32))
        assert np.array_equal(to_host(q8.silu_mul_quantize(g3, u3, tiled=True)), to_host(act))
    else:
        # the single mat-mat adds K sets in another order: last-bit differences in the sums (and with them single quants)
        assert rel_l2(to_host(g3), gate) <= 1e-6 and rel_l2(to_host(u3), up) <= 1e-6


def test_gate_up_silu_arguments(q8):
    import torch

    lib = q8._lib.lib()
    assert lib.nh_q8_0_gate_up_silu_workspace_bytes(512, 14336, 4096) == 0  # the benchmark shape takes the fused kernel
    assert lib.nh_q8_0_gate_up_silu_workspace_bytes(37, 3584, 1024) == 2 * 37 * 3584 * 4
    assert lib.nh_q8_0_gate_up_silu_workspace_bytes(37, 100, 1024) == -3
    w = torch.zeros(q8.tiled_bytes(3584, 1024), dtype=torch.uint8, device="cuda")
    a = torch.zeros(q8.tiled_bytes(37, 1024), dtype=torch.uint8, device="cuda")
    out = torch.zeros(q8.tiled_bytes(37, 3584), dtype=torch.uint8, device="cuda")
    # a shape that needs the workspace and does not get it
    assert lib.nh_q8_0_gemm_tiled_gate_up_silu(w.data_ptr(), w.data_ptr(), a.data_ptr(), out.data_ptr(), None, 0, 37, 3584, 1024, None) == -6
    assert lib.nh_q8_0_gemm_tiled_gate_up_silu(w.data_ptr(), w.data_ptr(), a.data_ptr(), None, None, 0, 37, 3584, 1024, None) == -1
    assert lib.nh_q8_0_gemm_tiled_gate_up_silu(None, None, None, None, None, 0, 0, 3584, 1024, None) == 0
    # an empty inner dimension: gate = up = 0, silu(0) * 0 = 0, every block of the output is a zero block (scale 0, quants 0)
    ws = torch.empty(lib.nh_q8_0_gate_up_silu_workspace_bytes(37, 3584, 0), dtype=torch.uint8, device="cuda")
    out.fill_(0xFF)
    assert lib.nh_q8_0_gemm_tiled_gate_up_silu(None, None, None, out.data_ptr(), ws.data_ptr(), ws.numel(), 37, 3584, 0, None) == 0
    torch.cuda.synchronize()
    assert not out.cpu().numpy().any()

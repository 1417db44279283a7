"""GPU: tensors of a GGUF file land on the device byte for byte (as stored, or in the tiled layout) and feed the kernels."""
import numpy as np
import pytest

import gguf_writer as W
from helpers import REL_L2_TOL, rel_l2, to_dev, to_host

pytestmark = pytest.mark.gpu


def test_upload_q8_0_and_f32_tensors(q8, oracle, tmp_path):
    from nihilus_amd import gguf as G

    k, rows = 4096, 320
    w = oracle.fill_weights(5, rows, k)
    norm = np.linspace(-1, 1, k).astype(np.float32)
    path = str(tmp_path / "m.gguf")
    W.write_gguf(path, [("general.alignment", W.U32, 64)], [("blk.0.attn_norm.weight", [k], 0, norm.tobytes()), ("blk.0.ffn_gate.weight", [k, rows], 8, w.tobytes())], alignment=64)
    with G.GGUFFile(path) as f:
        t = f.find("blk.0.ffn_gate.weight")
        blocks = f.upload(t, tiled=False)
        assert np.array_equal(to_host(blocks), w)
        tiled = f.upload(t, tiled=True)
        assert np.array_equal(to_host(q8.untile(tiled, rows, k)), w)
        n = f.upload(f.find("blk.0.attn_norm.weight"), tiled=False)
        assert np.array_equal(to_host(n).view(np.float32), norm)
        # the uploaded weight drives the mat-vec and the embedding lookup exactly like one tiled from host bytes
        x = q8.fill_activations(3, k)
        assert np.array_equal(to_host(q8.gemv_f32(tiled, x, rows, k)), to_host(q8.gemv_f32(q8.tile(to_dev(w), rows, k), x, rows, k)))
        xq = oracle.quantize_rows(to_host(x))[0]
        assert rel_l2(to_host(q8.gemv_f32(tiled, x, rows, k)), oracle.gemv(w, xq, rows, k)) <= REL_L2_TOL
        ids = np.array([0, 319, 7], dtype=np.int32)
        assert np.array_equal(to_host(q8.get_rows(blocks, to_dev(ids), rows, k, False)), oracle.get_rows(w, ids, rows, k)[0])


def test_upload_errors(q8, oracle, tmp_path):
    import ctypes as C

    import torch

    from nihilus_amd import _lib
    from nihilus_amd import gguf as G

    path = str(tmp_path / "e.gguf")
    W.write_gguf(path, [], [("a", [96, 4], 8, oracle.fill_weights(1, 4, 96).tobytes()), ("b", [128], 0, W.f32_bytes(np.zeros(128))),
                               ("c", [128, 4], 8, oracle.fill_weights(2, 4, 128).tobytes())])
    lib = _lib.lib()
    with G.GGUFFile(path) as f:
        a, b, c = f.find("a"), f.find("b"), f.find("c")
        dst = torch.zeros(8192, dtype=torch.uint8, device="cuda")
        st = torch.zeros(8192, dtype=torch.uint8, device="cuda")
        up = lambda info, tiled, staging, n: lib.nh_gguf_upload_tensor(f._h, C.byref(info), dst.data_ptr(), tiled, staging, n, None)
        assert up(a, 1, st.data_ptr(), 8192) == -3  # K = 96 is not a multiple of 128
        assert up(b, 1, st.data_ptr(), 8192) == -6  # not Q8_0
        assert up(a, 0, None, 0) == 0
        assert up(c, 1, None, 0) == -1
        assert up(c, 1, st.data_ptr(), 10) == -6
        assert up(c, 1, st.data_ptr(), 8192) == 0
        a.dims[0] = 128  # a record edited by the caller no longer matches its byte size
        assert up(a, 1, st.data_ptr(), 8192) == -6

"""ctypes binding of the GGUF reader / tensor upload declared in include/nihilus_amd/gguf_q8_0.h.

Parsing is host-only (no GPU needed); `upload` needs the GPU and, like everything else here, has no fallback.
"""
from __future__ import annotations

import ctypes as C

from . import _lib

_vp, _i64, _u64, _u32, _int = C.c_void_p, C.c_int64, C.c_uint64, C.c_uint32, C.c_int

GGML_F32, GGML_F16, GGML_Q8_0, GGML_I32 = 0, 1, 8, 26


class TensorInfo(C.Structure):
    """nh_gguf_tensor_info"""

    _fields_ = [("name", C.c_char_p), ("n_dims", _u32), ("ggml_type", _u32), ("dims", _u64 * 4), ("offset", _u64), ("file_offset", _u64), ("byte_size", _u64),
                ("layer", C.c_int32), ("reserved", C.c_int32)]


# name -> (restype, argtypes); mirrors gguf_q8_0.h one to one
SIGNATURES = {
    "nh_ggml_tensor_bytes": (_i64, [_u32, C.POINTER(_u64), _u32]),
    "nh_gguf_open": (_int, [C.c_char_p, C.POINTER(_vp)]),
    "nh_gguf_close": (None, [_vp]),
    "nh_gguf_tensor_count": (_i64, [_vp]),
    "nh_gguf_metadata_count": (_i64, [_vp]),
    "nh_gguf_alignment": (_u64, [_vp]),
    "nh_gguf_data_offset": (_u64, [_vp]),
    "nh_gguf_version": (_u32, [_vp]),
    "nh_gguf_tensor_at": (_int, [_vp, _i64, C.POINTER(TensorInfo)]),
    "nh_gguf_find_tensor": (_int, [_vp, C.c_char_p, C.POINTER(TensorInfo)]),
    "nh_gguf_tensor_data": (_vp, [_vp, C.POINTER(TensorInfo)]),
    "nh_gguf_metadata_u64": (_int, [_vp, C.c_char_p, C.POINTER(_u64)]),
    "nh_gguf_metadata_i64": (_int, [_vp, C.c_char_p, C.POINTER(_i64)]),
    "nh_gguf_metadata_f64": (_int, [_vp, C.c_char_p, C.POINTER(C.c_double)]),
    "nh_gguf_metadata_string": (_int, [_vp, C.c_char_p, C.POINTER(_vp), C.POINTER(_u64)]),  # the value is not NUL-terminated: raw pointer
    "nh_gguf_metadata_array": (_int, [_vp, C.c_char_p, C.POINTER(_u32), C.POINTER(_u64), C.POINTER(_vp)]),
    "nh_gguf_upload_tensor": (_int, [_vp, C.POINTER(TensorInfo), _vp, _int, _vp, _i64, _vp]),
}

_bound = False


def _l() -> C.CDLL:
    global _bound
    lib = _lib.lib()
    if not _bound:
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _bound = True
    return lib


def tensor_bytes(ggml_type: int, dims: list[int]) -> int:
    arr = (_u64 * len(dims))(*dims)
    return int(_l().nh_ggml_tensor_bytes(ggml_type, arr, len(dims)))


class GGUFFile:
    """An open GGUF file: tensor directory, metadata lookups, tensor upload."""

    def __init__(self, path: str):
        self._h = _vp()
        _lib.check("nh_gguf_open", _l().nh_gguf_open(path.encode(), C.byref(self._h)))

    def close(self) -> None:
        if self._h:
            _l().nh_gguf_close(self._h)
            self._h = _vp()

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    @property
    def version(self) -> int:
        return int(_l().nh_gguf_version(self._h))

    @property
    def alignment(self) -> int:
        return int(_l().nh_gguf_alignment(self._h))

    @property
    def data_offset(self) -> int:
        return int(_l().nh_gguf_data_offset(self._h))

    @property
    def tensor_count(self) -> int:
        return int(_l().nh_gguf_tensor_count(self._h))

    @property
    def metadata_count(self) -> int:
        return int(_l().nh_gguf_metadata_count(self._h))

    def tensor_at(self, index: int) -> TensorInfo:
        info = TensorInfo()
        _lib.check("nh_gguf_tensor_at", _l().nh_gguf_tensor_at(self._h, index, C.byref(info)))
        return info

    def find(self, name: str) -> TensorInfo:
        info = TensorInfo()
        _lib.check("nh_gguf_find_tensor", _l().nh_gguf_find_tensor(self._h, name.encode(), C.byref(info)))
        return info

    def data(self, info: TensorInfo) -> bytes:
        p = _l().nh_gguf_tensor_data(self._h, C.byref(info))
        if not p:
            raise ValueError("not a tensor of this file")
        return C.string_at(p, info.byte_size)

    def u64(self, key: str) -> int:
        v = _u64()
        _lib.check("nh_gguf_metadata_u64", _l().nh_gguf_metadata_u64(self._h, key.encode(), C.byref(v)))
        return int(v.value)

    def i64(self, key: str) -> int:
        v = _i64()
        _lib.check("nh_gguf_metadata_i64", _l().nh_gguf_metadata_i64(self._h, key.encode(), C.byref(v)))
        return int(v.value)

    def f64(self, key: str) -> float:
        v = C.c_double()
        _lib.check("nh_gguf_metadata_f64", _l().nh_gguf_metadata_f64(self._h, key.encode(), C.byref(v)))
        return float(v.value)

    def string(self, key: str) -> str:
        raw, n = _vp(), _u64()
        _lib.check("nh_gguf_metadata_string", _l().nh_gguf_metadata_string(self._h, key.encode(), C.byref(raw), C.byref(n)))
        return C.string_at(raw.value, n.value).decode()

    def array(self, key: str):
        """(element type, count, address of the first element as stored in the file)"""
        t, n, p = _u32(), _u64(), _vp()
        _lib.check("nh_gguf_metadata_array", _l().nh_gguf_metadata_array(self._h, key.encode(), C.byref(t), C.byref(n), C.byref(p)))
        return int(t.value), int(n.value), p.value

    def upload(self, info: TensorInfo, tiled: bool):
        """The tensor on the current GPU as a uint8 torch tensor: its bytes as stored, or (Q8_0 matrices) the tiled layout."""
        import torch

        from . import q8_0

        stream = torch.cuda.current_stream().cuda_stream
        if not tiled:
            dst = torch.empty(info.byte_size, dtype=torch.uint8, device="cuda")
            _lib.check("nh_gguf_upload_tensor", _l().nh_gguf_upload_tensor(self._h, C.byref(info), dst.data_ptr(), 0, None, 0, stream))
            return dst
        rows, k = int(info.dims[1]), int(info.dims[0])
        dst = torch.empty(q8_0.tiled_bytes(rows, k), dtype=torch.uint8, device="cuda")
        staging = torch.empty(info.byte_size, dtype=torch.uint8, device="cuda")
        _lib.check("nh_gguf_upload_tensor", _l().nh_gguf_upload_tensor(self._h, C.byref(info), dst.data_ptr(), 1, staging.data_ptr(), staging.numel(), stream))
        torch.cuda.current_stream().synchronize()  # the staging buffer goes away with this frame
        return dst

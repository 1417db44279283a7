"""ctypes binding of libnihilus_q8_hip.so, the C ABI declared in include/nihilus_amd/q8_0_abi.h.

There is no fallback: if the library is missing, loading raises, and every wrapper turns a non-zero
status into ``Q8Error``.
"""
from __future__ import annotations

import ctypes as C
import os

from .build import LIB_PATH

_vp, _i64, _u64, _int = C.c_void_p, C.c_int64, C.c_uint64, C.c_int

# name -> (restype, argtypes); mirrors q8_0_abi.h one to one
SIGNATURES = {
    "nh_status_string": (C.c_char_p, [_int]),
    "nh_abi_version": (_int, []),
    "nh_device_info": (_int, [C.c_char_p, _i64, C.POINTER(_i64), C.POINTER(_i64)]),
    "nh_malloc": (_int, [C.POINTER(_vp), _i64]),
    "nh_free": (_int, [_vp]),
    "nh_memcpy_h2d": (_int, [_vp, _vp, _i64, _vp]),
    "nh_memcpy_d2h": (_int, [_vp, _vp, _i64, _vp]),
    "nh_memset": (_int, [_vp, _int, _i64, _vp]),
    "nh_stream_sync": (_int, [_vp]),
    "nh_q8_0_quantize": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_quantize_tiled": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_silu_mul_quantize": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_silu_mul_quantize_tiled": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_blocks_bytes": (_i64, [_i64, _i64]),
    "nh_q8_0_tiled_bytes": (_i64, [_i64, _i64]),
    "nh_q8_0_tile": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_untile": (_int, [_vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_get_rows": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_get_rows_tiled": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_ffn_f32": (_int, [_vp, _vp, _vp, _vp, _vp, C.c_float, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_gate_up_silu_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "nh_q8_0_gemm_tiled_gate_up_silu": (_int, [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _vp]),
    "nh_q8_0_debug_gemm_tiled_gate_up_silu": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_decode_layer_f32": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _vp, C.c_float, _i64, _i64, _vp]),
    "nh_q8_0_rms_norm_quantize": (_int, [_vp, _vp, C.c_float, _vp, _i64, _i64, _vp]),
    "nh_q8_0_rms_norm_quantize_tiled": (_int, [_vp, _vp, C.c_float, _vp, _i64, _i64, _vp]),
    "nh_q8_0_mul_mat_f32_activations": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_gemv_tiled_group_f32": (_int, [C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64), C.POINTER(_i64), _i64, _vp]),
    "nh_q8_0_gemv_tiled_multi_norm_f32": (_int, [C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64), _i64, _vp, _vp, C.c_float, _i64, _vp]),
    "nh_q8_0_debug_fused_norm_quantize": (_int, [_vp, _vp, C.c_float, _vp, _i64, _vp]),
    "nh_q8_0_debug_ffn_gate_up": (_int, [_vp, _vp, _i64, _vp]),
    "nh_q8_0_gemv": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_gemv_tiled": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_gemv_tiled_f32": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_gemv_tiled_f32_noalloc": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_prepare": (_int, []),
    "nh_q8_0_last_error": (_int, []),
    "nh_q8_0_clear_error": (_int, []),
    "nh_q8_0_debug_set_spin_limit": (_int, [_i64]),
    "nh_q8_0_set_in_kernel_waits": (_int, [_int]),
    "nh_q8_0_debug_plan_mul_mat": (_int, [_i64, _i64, _i64, _vp]),
    "nh_q8_0_gemv_tiled_residual_f32": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _vp]),
    "nh_q8_0_gemv_tiled_multi_f32": (_int, [C.POINTER(_vp), C.POINTER(_vp), C.POINTER(_i64), _i64, _vp, _i64, _vp]),
    "nh_q8_0_debug_fused_quantize": (_int, [_vp, _vp, _i64, _vp]),
    "nh_q8_0_gemm": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_gemm_tiled": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_gemm_tiled_residual": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp]),
    "nh_q8_0_mul_mat_workspace_bytes": (_i64, [_i64, _i64]),
    "nh_q8_0_mul_mat": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "nh_q8_0_mul_mat_residual": (_int, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp, _i64, _vp]),
    "nh_q8_0_mul_mat_batch": (_int, [_vp, _i64, _vp, _i64, _vp]),
    "nh_profile_begin": (_int, [_int, _i64]),
    "nh_profile_shader_clock": (_int, [C.POINTER(C.c_double), _i64]),
    "nh_profile_end": (_int, [C.POINTER(C.c_double), C.POINTER(_i64), C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "nh_q8_0_debug_block_sums": (_int, [_vp, _vp, _vp, _i64, _i64, _i64, _int, _vp]),
    "nh_q8_0_fill_weight_blocks": (_int, [_vp, _u64, _i64, _i64, _vp]),
    "nh_q8_0_fill_activations": (_int, [_vp, _u64, _i64, _vp]),
}


class MulMatOp(C.Structure):
    """nh_q8_0_mul_mat_op"""

    _fields_ = [("W_tiled", _vp), ("x", _vp), ("y", _vp), ("M", _i64), ("N", _i64), ("K", _i64), ("reuse_quantized_x", C.c_int32), ("ordered", C.c_int32)]


class Q8Error(RuntimeError):
    """A call into the HIP library returned a non-zero status."""

    def __init__(self, fn: str, status: int, text: str):
        super().__init__(f"{fn} failed: status {status} ({text})")
        self.status = status


_lib = None


def lib() -> C.CDLL:
    """The loaded library; raises if it has not been built (run ``python -m nihilus_amd.build``)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP extension must be built (python -m nihilus_amd.build); "
                "there is no CPU fallback for this path"
            )
        handle = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(handle, name)  # AttributeError if the library does not export a declared symbol
            fn.restype, fn.argtypes = res, args
        _lib = handle
    return _lib


def status_string(status: int) -> str:
    return lib().nh_status_string(int(status)).decode()


def check(fn: str, status: int) -> None:
    if status != 0:
        raise Q8Error(fn, int(status), status_string(status))

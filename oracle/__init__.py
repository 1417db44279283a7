"""ctypes bindings of the CPU checker (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the benchmark's cpu_baseline leg may import this package; the
product (``nihilus_amd``) never does.  All functions take and return numpy arrays; Q8_0 data is a
``uint8`` array of packed 34-byte blocks (2-byte little-endian fp16 scale, then 32 int8 quants).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
QK = 32
BLOCK_BYTES = 34


def build(force: bool = False) -> None:
    """Compile both checker libraries with the Makefile beside this file."""
    args = ["make", "-C", _HERE]
    if force:
        args.append("-B")
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


def _load(name: str) -> C.CDLL:
    path = os.path.join(_HERE, name)
    if not os.path.exists(path):
        build()
    return C.CDLL(path)


_o = _load("libq8_0_oracle.so")
_a = _load("libq8_0_avx2.so")

_vp, _i64, _f32p = C.c_void_p, C.c_int64, C.POINTER(C.c_float)


def _sig(lib, name, res, *args):
    fn = getattr(lib, name)
    fn.restype = res
    fn.argtypes = list(args)
    return fn


_fp16_to_fp32 = _sig(_o, "nho_fp16_to_fp32", C.c_float, C.c_uint16)
_fp32_to_fp16 = _sig(_o, "nho_fp32_to_fp16", C.c_uint16, C.c_float)
_a_fp16_to_fp32 = _sig(_a, "nha_fp16_to_fp32", C.c_float, C.c_uint16)
_a_fp32_to_fp16 = _sig(_a, "nha_fp32_to_fp16", C.c_uint16, C.c_float)
_q8_bytes = _sig(_o, "nho_q8_0_bytes", _i64, _i64, _i64)
_dequant = _sig(_o, "nho_dequantize_row_q8_0", None, _vp, _vp, _i64)
_get_rows = _sig(_o, "nho_get_rows_q8_0", _i64, _vp, _vp, _vp, _i64, _i64, _i64)
_rms_scale = _sig(_o, "nho_rms_norm_scale", C.c_float, _vp, _i64, C.c_float)
_rms_mul_row = _sig(_o, "nho_rms_norm_mul_row", None, _vp, _vp, C.c_float, _vp, _i64)
_rms_quant_rows = _sig(_o, "nho_rms_norm_quantize_rows_q8_0", None, _vp, _vp, C.c_float, _vp, _i64, _i64, _vp)
_expf = _sig(_o, "nho_expf", C.c_float, C.c_float)
_silu_mul = _sig(_o, "nho_silu_mul", C.c_float, C.c_float, C.c_float)
_silu_mul_quant_rows = _sig(_o, "nho_silu_mul_quantize_rows_q8_0", None, _vp, _vp, _vp, _i64, _i64)
_quant_rows = _sig(_o, "nho_quantize_rows_q8_0", None, _vp, _vp, _i64, _i64)
_a_quant_rows = _sig(_a, "nha_quantize_rows_q8_0", None, _vp, _vp, _i64, _i64)
_sums_gemv = _sig(_o, "nho_block_sums_gemv", None, _vp, _vp, _vp, _i64, _i64)
_vec_dot = _sig(_o, "nho_vec_dot_q8_0_q8_0", C.c_float, _i64, _vp, _vp)
_vec_dot_rt = _sig(_o, "nho_vec_dot_q8_0_q8_0_rt", C.c_float, _i64, _vp, _vp)
_vec_dot_f64 = _sig(_o, "nho_vec_dot_f64", C.c_double, _i64, _vp, _vp)
_a_vec_dot = _sig(_a, "nha_vec_dot_q8_0_q8_0_x16", C.c_float, _i64, _vp, _vp)
_gemv = _sig(_o, "nho_gemv_q8_0", None, _vp, _vp, _vp, _i64, _i64)
_gemv_f64 = _sig(_o, "nho_gemv_q8_0_f64", None, _vp, _vp, _vp, _i64, _i64)
_gemm = _sig(_o, "nho_gemm_q8_0", None, _vp, _vp, _vp, _i64, _i64, _i64)
_a_gemm = _sig(_a, "nha_gemm_q8_0_mt", C.c_int, _vp, _vp, _vp, _i64, _i64, _i64, C.c_int, C.c_int)
_a_time_gemv = _sig(_a, "nha_time_gemv", C.c_double, _vp, _i64, _vp, _vp, _i64, _i64, C.c_int, C.c_int, C.c_int)
_mul_mat_f32 = _sig(_o, "nho_mul_mat_q8_f32", None, _vp, _vp, _vp, _i64, _i64, _i64, C.c_int)
_mul_mat_f32_f64 = _sig(_o, "nho_mul_mat_q8_f32_f64", None, _vp, _vp, _vp, _i64, _i64, _i64)
_fill_act = _sig(_o, "nho_fill_activations", None, C.c_uint64, _vp, _i64)
_fill_w = _sig(_o, "nho_fill_weight_blocks", None, C.c_uint64, _vp, _i64, _i64)


def _ptr(a: np.ndarray) -> int:
    assert a.flags["C_CONTIGUOUS"]
    return a.ctypes.data


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _u8(a) -> np.ndarray:
    a = np.ascontiguousarray(a)
    assert a.dtype == np.uint8
    return a


# ---------------------------------------------------------------- fp16


def fp16_to_fp32(h: int) -> float:
    return float(_fp16_to_fp32(int(h) & 0xFFFF))


def fp32_to_fp16(f) -> int:
    return int(_fp32_to_fp16(C.c_float(f)))


def fp16_to_fp32_f16c(h: int) -> float:
    return float(_a_fp16_to_fp32(int(h) & 0xFFFF))


def fp32_to_fp16_f16c(f) -> int:
    return int(_a_fp32_to_fp16(C.c_float(f)))


# ---------------------------------------------------------------- layout


def q8_0_bytes(rows: int, k: int) -> int:
    return int(_q8_bytes(rows, k))


def split_blocks(blocks: np.ndarray):
    """Packed blocks -> (d as uint16 [..., nb], qs as int8 [..., nb, 32]) by plain byte slicing."""
    b = _u8(blocks).reshape(-1, BLOCK_BYTES)
    d = b[:, 0].astype(np.uint16) | (b[:, 1].astype(np.uint16) << 8)
    qs = b[:, 2:].view(np.int8)
    return d, qs


def pack_blocks(d_u16: np.ndarray, qs_i8: np.ndarray) -> np.ndarray:
    d = np.ascontiguousarray(d_u16, dtype=np.uint16).reshape(-1)
    q = np.ascontiguousarray(qs_i8, dtype=np.int8).reshape(-1, QK)
    out = np.empty((d.size, BLOCK_BYTES), dtype=np.uint8)
    out[:, 0] = d & 0xFF
    out[:, 1] = d >> 8
    out[:, 2:] = q.view(np.uint8)
    return out.reshape(-1)


def dequantize_row(blocks: np.ndarray, k: int) -> np.ndarray:
    y = np.empty(k // QK * QK, dtype=np.float32)
    b = _u8(blocks)
    _dequant(_ptr(b), _ptr(y), k)
    return y


def get_rows(blocks: np.ndarray, ids: np.ndarray, n_rows: int, k: int):
    """Token-embedding lookup on a [n_rows, k] block matrix; returns (fp32 [n_tokens, k], number of out-of-range ids)."""
    b = _u8(blocks)
    ids = np.ascontiguousarray(ids, dtype=np.int32)
    out = np.empty((ids.size, k), dtype=np.float32)
    bad = _get_rows(_ptr(b), _ptr(ids), _ptr(out), ids.size, n_rows, k)
    return out, int(bad)


def rms_norm_scale(x: np.ndarray, eps: float) -> float:
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    return float(_rms_scale(_ptr(x), x.size, eps))


def rms_norm_mul(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """(x * 1/rms(x)) * w for one fp32 row, in the checker's fixed order."""
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    w = np.ascontiguousarray(w, dtype=np.float32).ravel()
    y = np.empty_like(x)
    _rms_mul_row(_ptr(x), _ptr(w), eps, _ptr(y), x.size)
    return y


def rms_norm_quantize_rows(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x: fp32 [m, k], w: fp32 [k]; returns uint8 [m, (k//32)*34] = quantize_rows(rms_norm(x) * w)."""
    x = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32).ravel()
    m, k = x.shape
    out = np.empty((m, k // QK * BLOCK_BYTES), dtype=np.uint8)
    tmp = np.empty(k, dtype=np.float32)
    _rms_quant_rows(_ptr(x), _ptr(w), eps, _ptr(out), m, k, _ptr(tmp))
    return out


def expf(x: np.ndarray) -> np.ndarray:
    """The checker's fixed-sequence fp32 exp, element-wise."""
    x = np.ascontiguousarray(x, dtype=np.float32).ravel()
    return np.array([_expf(float(v)) for v in x], dtype=np.float32)


def silu_mul(g: np.ndarray, u: np.ndarray) -> np.ndarray:
    g = np.ascontiguousarray(g, dtype=np.float32).ravel()
    u = np.ascontiguousarray(u, dtype=np.float32).ravel()
    return np.array([_silu_mul(float(a), float(b)) for a, b in zip(g, u)], dtype=np.float32)


def silu_mul_quantize_rows(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    """gate, up: fp32 [m, k]; returns uint8 [m, (k//32)*34] = quantize_rows(silu(gate) * up)."""
    g = np.ascontiguousarray(np.atleast_2d(gate), dtype=np.float32)
    u = np.ascontiguousarray(np.atleast_2d(up), dtype=np.float32)
    m, k = g.shape
    out = np.empty((m, k // QK * BLOCK_BYTES), dtype=np.uint8)
    _silu_mul_quant_rows(_ptr(g), _ptr(u), _ptr(out), m, k)
    return out


# ---------------------------------------------------------------- quantize


def quantize_rows(x: np.ndarray, k: int | None = None, avx2: bool = False) -> np.ndarray:
    """x: [m, k_alloc] fp32 (or [k]); returns uint8 [m, (k//32)*34]."""
    x = _f32(x)
    if x.ndim == 1:
        x = x[None, :]
    m, kk = x.shape
    k = kk if k is None else k
    assert k <= kk
    if k != kk:
        x = np.ascontiguousarray(x[:, :k])
    out = np.zeros((m, (k // QK) * BLOCK_BYTES), dtype=np.uint8)
    if out.size:
        (_a_quant_rows if avx2 else _quant_rows)(_ptr(x), _ptr(out), m, k)
    return out


# ---------------------------------------------------------------- dots


def block_sums_gemv(w: np.ndarray, xq: np.ndarray, n: int, k: int) -> np.ndarray:
    w, xq = _u8(w), _u8(xq)
    sums = np.empty((n, k // QK), dtype=np.int32)
    _sums_gemv(_ptr(w), _ptr(xq), _ptr(sums), n, k)
    return sums


def vec_dot(nb: int, x: np.ndarray, y: np.ndarray) -> np.float32:
    x, y = _u8(x), _u8(y)
    return np.float32(_vec_dot(nb, _ptr(x), _ptr(y)))


def vec_dot_rt(k: int, x: np.ndarray, y: np.ndarray) -> np.float32:
    x, y = _u8(x), _u8(y)
    return np.float32(_vec_dot_rt(k, _ptr(x), _ptr(y)))


def vec_dot_f64(nb: int, x: np.ndarray, y: np.ndarray) -> float:
    x, y = _u8(x), _u8(y)
    return float(_vec_dot_f64(nb, _ptr(x), _ptr(y)))


def vec_dot_avx2(nb: int, x: np.ndarray, y: np.ndarray) -> np.float32:
    assert nb % 16 == 0
    x, y = _u8(x), _u8(y)
    return np.float32(_a_vec_dot(nb, _ptr(x), _ptr(y)))


def gemv(w: np.ndarray, xq: np.ndarray, n: int, k: int) -> np.ndarray:
    w, xq = _u8(w), _u8(xq)
    y = np.empty(n, dtype=np.float32)
    _gemv(_ptr(w), _ptr(xq), _ptr(y), n, k)
    return y


def gemv_f64(w: np.ndarray, xq: np.ndarray, n: int, k: int) -> np.ndarray:
    w, xq = _u8(w), _u8(xq)
    y = np.empty(n, dtype=np.float64)
    _gemv_f64(_ptr(w), _ptr(xq), _ptr(y), n, k)
    return y


def mul_mat_f32_activations(w: np.ndarray, x: np.ndarray, n: int, k: int, prompt_order: bool = False) -> np.ndarray:
    """fp32 activations [m, k] against Q8_0 weights, no activation quantize: y [m, n] in the eval_time leaf's summation
    order, or the prompt_eval_time leaf's."""
    w, x = _u8(w), _f32(x).reshape(-1, k)
    y = np.empty((x.shape[0], n), dtype=np.float32)
    _mul_mat_f32(_ptr(w), _ptr(x), _ptr(y), x.shape[0], n, k, 1 if prompt_order else 0)
    return y


def mul_mat_f32_activations_f64(w: np.ndarray, x: np.ndarray, n: int, k: int) -> np.ndarray:
    w, x = _u8(w), _f32(x).reshape(-1, k)
    y = np.empty((x.shape[0], n), dtype=np.float64)
    _mul_mat_f32_f64(_ptr(w), _ptr(x), _ptr(y), x.shape[0], n, k)
    return y


def gemm(w: np.ndarray, aq: np.ndarray, m: int, n: int, k: int, threads: int = 0) -> np.ndarray:
    """C [m, n] fp32.  threads > 0 uses the AVX2 restatement (needs (k/32) % 16 == 0)."""
    w, aq = _u8(w), _u8(aq)
    c = np.empty((m, n), dtype=np.float32)
    if threads > 0:
        rc = _a_gemm(_ptr(w), _ptr(aq), _ptr(c), m, n, k, threads, 0)
        if rc != 0:
            raise ValueError("AVX2 restatement handles only block counts that are multiples of 16")
    else:
        _gemm(_ptr(w), _ptr(aq), _ptr(c), m, n, k)
    return c


def time_gemv_avx2(w_all: np.ndarray, n_mats: int, x: np.ndarray, n: int, k: int, threads: int, iters: int, pin: bool = True) -> float:
    """Seconds per (quantize + GEMV) over rotating weight copies; see nha_time_gemv."""
    w_all, x = _u8(w_all), _f32(x)
    y = np.empty(n, dtype=np.float32)
    t = float(_a_time_gemv(_ptr(w_all), n_mats, _ptr(x), _ptr(y), n, k, threads, 1 if pin else 0, iters))
    if t < 0:
        raise ValueError("unsupported shape for the AVX2 baseline")
    return t


# ---------------------------------------------------------------- synthetic inputs


def fill_activations(seed: int, count: int) -> np.ndarray:
    x = np.empty(count, dtype=np.float32)
    _fill_act(C.c_uint64(seed), _ptr(x), count)
    return x


def fill_weights(seed: int, n: int, k: int, first_block: int = 0) -> np.ndarray:
    nblk = n * (k // QK)
    w = np.empty(nblk * BLOCK_BYTES, dtype=np.uint8)
    _fill_w(C.c_uint64(seed), _ptr(w), first_block, nblk)
    return w

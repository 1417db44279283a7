"""Host-side wrappers of the Q8_0 path for callers that hold torch tensors.

torch is used for device memory and streams only; every operation below is one call through the C ABI
(``include/nihilus_amd/q8_0_abi.h``).  Names follow the reference: ``quantize_row_q8_0``
(cpu/avx_2.hpp:4439-4489), ``mul_mat`` (kernel_types::mul_mat, cpu/avx_2.hpp:1296-1444).  Q8_0 data is a
``torch.uint8`` tensor: "blocks" = rows of packed 34-byte block_q8_0, "tiled" = the device layout
described in the ABI header.
"""
from __future__ import annotations

import torch

from . import _lib

QK = 32
BLOCK_BYTES = 34


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _dev(t: torch.Tensor, dtype: torch.dtype, name: str) -> torch.Tensor:
    if not (t.is_cuda and t.dtype == dtype and t.is_contiguous()):
        raise TypeError(f"{name} must be a contiguous {dtype} tensor on the GPU")
    return t


def blocks_bytes(rows: int, k: int) -> int:
    n = _lib.lib().nh_q8_0_blocks_bytes(rows, k)
    _lib.check("nh_q8_0_blocks_bytes", n if n < 0 else 0)
    return n


def tiled_bytes(rows: int, k: int) -> int:
    n = _lib.lib().nh_q8_0_tiled_bytes(rows, k)
    _lib.check("nh_q8_0_tiled_bytes", n if n < 0 else 0)
    return n


KERNEL_NAMES = {0: "nothing", 1: "gemv", 2: "gemv_rows", 3: "gemm_skinny", 4: "gemm_tile_stream", 5: "gemm_tile", 6: "gemv_rows_mfma"}


def plan_mul_mat(m: int, n: int, k: int) -> dict:
    """Which kernel mul_mat runs for fp32 activations [m, k] against a tiled weight [n, k], and its cut (no GPU needed)."""
    import ctypes

    raw = (ctypes.c_int32 * 8)()
    _lib.check("nh_q8_0_debug_plan_mul_mat", _lib.lib().nh_q8_0_debug_plan_mul_mat(m, n, k, raw))
    plan = {"kernel": KERNEL_NAMES[raw[0]], "quantize_launch": bool(raw[1])}
    if raw[0] in (1, 6):
        plan.update(k_splits=raw[2], groups_per_wave=raw[3], row_parts=raw[4])
    elif raw[0] == 3:
        plan.update(activation_strips=raw[2], k_splits=raw[3])
    elif raw[0] in (4, 5):
        plan.update(activation_strips=raw[2], k_sets=raw[3], k_splits=raw[4], grid=(raw[5], raw[6]))
    return plan


def quantize_row_q8_0(x: torch.Tensor, tiled: bool = False) -> torch.Tensor:
    """x fp32 [M, K] (or [K]) -> uint8 blocks [M, K/32*34] (or the tiled byte stream)."""
    x = _dev(x, torch.float32, "x")
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    m, k = x2.shape
    if tiled:
        out = torch.empty(tiled_bytes(m, k), dtype=torch.uint8, device=x.device)
        _lib.check("nh_q8_0_quantize_tiled", _lib.lib().nh_q8_0_quantize_tiled(x2.data_ptr(), out.data_ptr(), m, k, _stream()))
        return out
    out = torch.empty((m, blocks_bytes(1, k)), dtype=torch.uint8, device=x.device)
    _lib.check("nh_q8_0_quantize", _lib.lib().nh_q8_0_quantize(x2.data_ptr(), out.data_ptr(), m, k, _stream()))
    return out


def silu_mul_quantize(gate: torch.Tensor, up: torch.Tensor, tiled: bool = False) -> torch.Tensor:
    """quantize_row_q8_0(silu(gate) * up) for fp32 [M, K] (or [K]) operands, one kernel; output as quantize_row_q8_0."""
    gate, up = _dev(gate, torch.float32, "gate"), _dev(up, torch.float32, "up")
    if gate.shape != up.shape:
        raise ValueError("gate and up must have the same shape")
    g2 = gate.reshape(1, -1) if gate.dim() == 1 else gate
    m, k = g2.shape
    if tiled:
        out = torch.empty(tiled_bytes(m, k), dtype=torch.uint8, device=gate.device)
        _lib.check("nh_q8_0_silu_mul_quantize_tiled", _lib.lib().nh_q8_0_silu_mul_quantize_tiled(gate.data_ptr(), up.data_ptr(), out.data_ptr(), m, k, _stream()))
        return out
    out = torch.empty((m, blocks_bytes(1, k)), dtype=torch.uint8, device=gate.device)
    _lib.check("nh_q8_0_silu_mul_quantize", _lib.lib().nh_q8_0_silu_mul_quantize(gate.data_ptr(), up.data_ptr(), out.data_ptr(), m, k, _stream()))
    return out


def tile(blocks: torch.Tensor, rows: int, k: int) -> torch.Tensor:
    blocks = _dev(blocks, torch.uint8, "blocks")
    if blocks.numel() != blocks_bytes(rows, k):
        raise ValueError("blocks tensor does not hold rows*(k/32) blocks")
    out = torch.empty(tiled_bytes(rows, k), dtype=torch.uint8, device=blocks.device)
    _lib.check("nh_q8_0_tile", _lib.lib().nh_q8_0_tile(blocks.data_ptr(), out.data_ptr(), rows, k, _stream()))
    return out


def untile(tiled: torch.Tensor, rows: int, k: int) -> torch.Tensor:
    tiled = _dev(tiled, torch.uint8, "tiled")
    if tiled.numel() != tiled_bytes(rows, k):
        raise ValueError("tiled tensor has the wrong size for rows x k")
    out = torch.empty(blocks_bytes(rows, k), dtype=torch.uint8, device=tiled.device)
    _lib.check("nh_q8_0_untile", _lib.lib().nh_q8_0_untile(tiled.data_ptr(), out.data_ptr(), rows, k, _stream()))
    return out


def get_rows(w: torch.Tensor, ids: torch.Tensor, n_rows: int, k: int, tiled: bool, count_invalid: bool = False):
    """Token-embedding lookup: fp32 [n_tokens, k] = dequantized rows `ids` of the Q8_0 matrix w (blocks or tiled).

    With count_invalid the number of ids outside [0, n_rows) comes back as a second value (their rows are zero)."""
    w, ids = _dev(w, torch.uint8, "w"), _dev(ids, torch.int32, "ids")
    if w.numel() != (tiled_bytes(n_rows, k) if tiled else blocks_bytes(n_rows, k)):
        raise ValueError("w has the wrong size for n_rows x k")
    n_tokens = ids.numel()
    out = torch.empty((n_tokens, k), dtype=torch.float32, device=w.device)
    bad = torch.zeros(1, dtype=torch.int32, device=w.device) if count_invalid else None
    fn = "nh_q8_0_get_rows_tiled" if tiled else "nh_q8_0_get_rows"
    _lib.check(fn, getattr(_lib.lib(), fn)(w.data_ptr(), ids.data_ptr(), out.data_ptr(), bad.data_ptr() if count_invalid else None, n_tokens, n_rows, k, _stream()))
    return (out, int(bad.item())) if count_invalid else out


def ffn(w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, x: torch.Tensor, n_ff: int, k: int, n_out: int, residual: torch.Tensor | None = None,
        norm_weight: torch.Tensor | None = None, eps: float = 0.0) -> torch.Tensor:
    """Decode-time FFN in one launch: W_down . Q(silu(W_gate . Q(n)) * (W_up . Q(n))) (+ residual), n = x or its RMS norm
    times norm_weight; weights tiled, x fp32 [k]."""
    w_gate, w_up, w_down = _dev(w_gate, torch.uint8, "w_gate"), _dev(w_up, torch.uint8, "w_up"), _dev(w_down, torch.uint8, "w_down")
    x = _dev(x, torch.float32, "x")
    if w_gate.numel() != tiled_bytes(n_ff, k) or w_up.numel() != tiled_bytes(n_ff, k) or w_down.numel() != tiled_bytes(n_out, n_ff) or x.numel() != k:
        raise ValueError("operand sizes do not match n_ff x k / n_out x n_ff")
    if residual is not None:
        residual = _dev(residual, torch.float32, "residual")
        if residual.numel() != n_out:
            raise ValueError("residual must hold n_out values")
    if norm_weight is not None and _dev(norm_weight, torch.float32, "norm_weight").numel() != k:
        raise ValueError("norm_weight must hold k floats")
    y = torch.empty(n_out, dtype=torch.float32, device=x.device)
    _lib.check("nh_q8_0_ffn_f32", _lib.lib().nh_q8_0_ffn_f32(w_gate.data_ptr(), w_up.data_ptr(), w_down.data_ptr(), x.data_ptr(),
                                                           norm_weight.data_ptr() if norm_weight is not None else None, eps,
                                                           residual.data_ptr() if residual is not None else None, y.data_ptr(), n_ff, k, n_out, _stream()))
    return y


def decode_layer(w_o: torch.Tensor, attn: torch.Tensor, layer_in: torch.Tensor, w_gate: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, ffn_norm: torch.Tensor,
                 w_next: list[torch.Tensor], n_next: list[int], next_norm: torch.Tensor | None, eps: float, n_embd: int, n_ff: int):
    """One block's decode mat-vecs from one attention to the next (nh_q8_0_decode_layer_f32): returns (ffn_inp, l_out, [y_next...])."""
    import ctypes

    attn, layer_in, ffn_norm = _dev(attn, torch.float32, "attn"), _dev(layer_in, torch.float32, "layer_in"), _dev(ffn_norm, torch.float32, "ffn_norm")
    ffn_inp = torch.empty(n_embd, dtype=torch.float32, device=attn.device)
    l_out = torch.empty(n_embd, dtype=torch.float32, device=attn.device)
    ys = [torch.empty(n, dtype=torch.float32, device=attn.device) for n in n_next]
    cnt = len(w_next)
    wp = (ctypes.c_void_p * max(cnt, 1))(*[w.data_ptr() for w in w_next])
    yp = (ctypes.c_void_p * max(cnt, 1))(*[y.data_ptr() for y in ys])
    np_ = (ctypes.c_int64 * max(cnt, 1))(*n_next)
    _lib.check("nh_q8_0_decode_layer_f32", _lib.lib().nh_q8_0_decode_layer_f32(
        w_o.data_ptr(), attn.data_ptr(), layer_in.data_ptr(), ffn_inp.data_ptr(), w_gate.data_ptr(), w_up.data_ptr(), w_down.data_ptr(), ffn_norm.data_ptr(), l_out.data_ptr(),
        wp, yp, np_, cnt, next_norm.data_ptr() if next_norm is not None else None, ctypes.c_float(eps), n_embd, n_ff, _stream()))
    return ffn_inp, l_out, ys


def debug_ffn_gate_up(n_ff: int):
    """The gate and up outputs (fp32 [n_ff] each) of the last ffn() on this device."""
    g = torch.empty(n_ff, dtype=torch.float32, device="cuda")
    u = torch.empty(n_ff, dtype=torch.float32, device="cuda")
    _lib.check("nh_q8_0_debug_ffn_gate_up", _lib.lib().nh_q8_0_debug_ffn_gate_up(g.data_ptr(), u.data_ptr(), n_ff, _stream()))
    return g, u


def gemv(w: torch.Tensor, xq_blocks: torch.Tensor, n: int, k: int, tiled: bool) -> torch.Tensor:
    w, xq_blocks = _dev(w, torch.uint8, "w"), _dev(xq_blocks, torch.uint8, "xq_blocks")
    if w.numel() != (tiled_bytes(n, k) if tiled else blocks_bytes(n, k)) or xq_blocks.numel() != blocks_bytes(1, k):
        raise ValueError("operand sizes do not match n x k")
    y = torch.empty(n, dtype=torch.float32, device=w.device)
    fn = "nh_q8_0_gemv_tiled" if tiled else "nh_q8_0_gemv"
    _lib.check(fn, getattr(_lib.lib(), fn)(w.data_ptr(), xq_blocks.data_ptr(), y.data_ptr(), n, k, _stream()))
    return y


def gemv_f32(w_tiled: list[torch.Tensor] | torch.Tensor, x: torch.Tensor, n: list[int] | int, k: int, norm_weight: torch.Tensor | None = None,
             eps: float = 0.0) -> list[torch.Tensor] | torch.Tensor:
    """Fused quantize + mat-vec on tiled weights; a list of up to 3 weights sharing x and k runs as one launch.
    With norm_weight the activation is RMS-normalised and multiplied by it first, inside the same launch."""
    import ctypes as C

    single = not isinstance(w_tiled, (list, tuple))
    ws = [w_tiled] if single else list(w_tiled)
    ns = [n] if single else list(n)
    x = _dev(x, torch.float32, "x")
    if x.numel() != k or len(ws) != len(ns):
        raise ValueError("x must hold k floats and every weight needs its row count")
    for w, nn in zip(ws, ns):
        if _dev(w, torch.uint8, "w_tiled").numel() != tiled_bytes(nn, k):
            raise ValueError("weight size does not match n x k")
    ys = [torch.empty(nn, dtype=torch.float32, device=x.device) for nn in ns]
    cnt = len(ws)
    wp = (C.c_void_p * cnt)(*[w.data_ptr() for w in ws])
    yp = (C.c_void_p * cnt)(*[y.data_ptr() for y in ys])
    np_ = (C.c_int64 * cnt)(*ns)
    if norm_weight is not None:
        nw = _dev(norm_weight, torch.float32, "norm_weight")
        if nw.numel() != k:
            raise ValueError("norm_weight must hold k floats")
        _lib.check("nh_q8_0_gemv_tiled_multi_norm_f32", _lib.lib().nh_q8_0_gemv_tiled_multi_norm_f32(wp, yp, np_, cnt, x.data_ptr(), nw.data_ptr(), eps, k, _stream()))
    else:
        _lib.check("nh_q8_0_gemv_tiled_multi_f32", _lib.lib().nh_q8_0_gemv_tiled_multi_f32(wp, yp, np_, cnt, x.data_ptr(), k, _stream()))
    return ys[0] if single else ys


def gemv_group_f32(w_tiled: list[torch.Tensor], xs: list[torch.Tensor], ns: list[int], ks: list[int], residuals: list[torch.Tensor | None] | None = None,
                   outs: list[torch.Tensor] | None = None) -> list[torch.Tensor]:
    """Independent mat-vecs, each with its own activation row, k and n, in as few launches as their shapes allow (one per up
    to eight matrices).  The caller vouches that no output is another op's input, residual or output."""
    import ctypes as C

    cnt = len(w_tiled)
    if not (len(xs) == len(ns) == len(ks) == cnt) or (residuals is not None and len(residuals) != cnt) or (outs is not None and len(outs) != cnt):
        raise ValueError("one x, n and k (and residual, out) per weight")
    xs = [_dev(x, torch.float32, "x") for x in xs]
    for w, x, n, k in zip(w_tiled, xs, ns, ks):
        if x.numel() != k or _dev(w, torch.uint8, "w_tiled").numel() != tiled_bytes(n, k):
            raise ValueError("operand sizes do not match n x k")
    ys = [torch.empty(n, dtype=torch.float32, device=xs[0].device) for n in ns] if outs is None else [_dev(o, torch.float32, "out") for o in outs]
    if any(y.numel() != n for y, n in zip(ys, ns)):
        raise ValueError("every out must hold n floats")
    rs = [None] * cnt if residuals is None else [None if r is None else _dev(r, torch.float32, "residual") for r in residuals]
    if any(r is not None and r.numel() != n for r, n in zip(rs, ns)):
        raise ValueError("every residual must hold n floats")
    wp = (C.c_void_p * cnt)(*[w.data_ptr() for w in w_tiled])
    xp = (C.c_void_p * cnt)(*[x.data_ptr() for x in xs])
    yp = (C.c_void_p * cnt)(*[y.data_ptr() for y in ys])
    rp = (C.c_void_p * cnt)(*[None if r is None else r.data_ptr() for r in rs])
    _lib.check("nh_q8_0_gemv_tiled_group_f32",
               _lib.lib().nh_q8_0_gemv_tiled_group_f32(wp, xp, yp, rp, (C.c_int64 * cnt)(*ns), (C.c_int64 * cnt)(*ks), cnt, _stream()))
    return ys


def gemv_residual_f32(w_tiled: torch.Tensor, x: torch.Tensor, residual: torch.Tensor, n: int, k: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """y = W . Q(x) + residual in one launch (out may be the residual tensor itself: in-place accumulate)."""
    w_tiled, x, residual = _dev(w_tiled, torch.uint8, "w_tiled"), _dev(x, torch.float32, "x"), _dev(residual, torch.float32, "residual")
    if x.numel() != k or residual.numel() != n or w_tiled.numel() != tiled_bytes(n, k):
        raise ValueError("operand sizes do not match n x k")
    y = torch.empty(n, dtype=torch.float32, device=x.device) if out is None else _dev(out, torch.float32, "out")
    if y.numel() != n:
        raise ValueError("out must hold n floats")
    _lib.check("nh_q8_0_gemv_tiled_residual_f32", _lib.lib().nh_q8_0_gemv_tiled_residual_f32(w_tiled.data_ptr(), x.data_ptr(), residual.data_ptr(), y.data_ptr(), n, k, _stream()))
    return y


def debug_fused_quantize(x: torch.Tensor, norm_weight: torch.Tensor | None = None, eps: float = 0.0) -> torch.Tensor:
    """The activation row exactly as the fused mat-vec stages it (after the RMS norm, if a norm weight is given), as packed blocks."""
    x = _dev(x, torch.float32, "x")
    k = x.numel()
    out = torch.zeros(blocks_bytes(1, k), dtype=torch.uint8, device=x.device)
    if norm_weight is not None:
        nw = _dev(norm_weight, torch.float32, "norm_weight")
        _lib.check("nh_q8_0_debug_fused_norm_quantize", _lib.lib().nh_q8_0_debug_fused_norm_quantize(x.data_ptr(), nw.data_ptr(), eps, out.data_ptr(), k, _stream()))
    else:
        _lib.check("nh_q8_0_debug_fused_quantize", _lib.lib().nh_q8_0_debug_fused_quantize(x.data_ptr(), out.data_ptr(), k, _stream()))
    return out


def rms_norm_quantize(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, tiled: bool = False) -> torch.Tensor:
    """quantize_row_q8_0((x * 1/rms(x)) * norm_weight) for fp32 [M, K] (or [K]) rows, one kernel; output as quantize_row_q8_0."""
    x, nw = _dev(x, torch.float32, "x"), _dev(norm_weight, torch.float32, "norm_weight")
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    m, k = x2.shape
    if nw.numel() != k:
        raise ValueError("norm_weight must hold k floats")
    if tiled:
        out = torch.empty(tiled_bytes(m, k), dtype=torch.uint8, device=x.device)
        _lib.check("nh_q8_0_rms_norm_quantize_tiled", _lib.lib().nh_q8_0_rms_norm_quantize_tiled(x2.data_ptr(), nw.data_ptr(), eps, out.data_ptr(), m, k, _stream()))
        return out
    out = torch.empty((m, blocks_bytes(1, k)), dtype=torch.uint8, device=x.device)
    _lib.check("nh_q8_0_rms_norm_quantize", _lib.lib().nh_q8_0_rms_norm_quantize(x2.data_ptr(), nw.data_ptr(), eps, out.data_ptr(), m, k, _stream()))
    return out


def gemm(w: torch.Tensor, aq: torch.Tensor, m: int, n: int, k: int, tiled: bool) -> torch.Tensor:
    w, aq = _dev(w, torch.uint8, "w"), _dev(aq, torch.uint8, "aq")
    size = tiled_bytes if tiled else blocks_bytes
    if w.numel() != size(n, k) or aq.numel() != size(m, k):
        raise ValueError("operand sizes do not match m x n x k")
    c = torch.empty((m, n), dtype=torch.float32, device=w.device)
    fn = "nh_q8_0_gemm_tiled" if tiled else "nh_q8_0_gemm"
    _lib.check(fn, getattr(_lib.lib(), fn)(w.data_ptr(), aq.data_ptr(), c.data_ptr(), m, n, k, _stream()))
    return c


def gemm_residual(w_tiled: torch.Tensor, aq_tiled: torch.Tensor, residual: torch.Tensor, m: int, n: int, k: int, out: torch.Tensor | None = None) -> torch.Tensor:
    """C = W . Aq + residual on tiled operands in one launch (out may be the residual tensor itself: in-place accumulate)."""
    w, aq, residual = _dev(w_tiled, torch.uint8, "w_tiled"), _dev(aq_tiled, torch.uint8, "aq_tiled"), _dev(residual, torch.float32, "residual")
    if w.numel() != tiled_bytes(n, k) or aq.numel() != tiled_bytes(m, k) or residual.numel() != m * n:
        raise ValueError("operand sizes do not match m x n x k")
    c = torch.empty((m, n), dtype=torch.float32, device=w.device) if out is None else _dev(out, torch.float32, "out")
    if c.numel() != m * n:
        raise ValueError("out must hold m x n floats")
    _lib.check("nh_q8_0_gemm_tiled_residual", _lib.lib().nh_q8_0_gemm_tiled_residual(w.data_ptr(), aq.data_ptr(), residual.data_ptr(), c.data_ptr(), m, n, k, _stream()))
    return c


def gate_up_silu(w_gate: torch.Tensor, w_up: torch.Tensor, aq_tiled: torch.Tensor, m: int, n_ff: int, k: int, debug: bool = False):
    """Tiled Q8_0 activation of the down projection: quantize(silu(W_gate . Aq) * (W_up . Aq)) (nh_q8_0_gemm_tiled_gate_up_silu).
    debug=True also returns the fp32 gate and up outputs the call computed."""
    lib = _lib.lib()
    out = torch.empty(tiled_bytes(m, n_ff), dtype=torch.uint8, device=aq_tiled.device)
    if debug:
        gate = torch.empty((m, n_ff), dtype=torch.float32, device=aq_tiled.device)
        up = torch.empty((m, n_ff), dtype=torch.float32, device=aq_tiled.device)
        _lib.check("nh_q8_0_debug_gemm_tiled_gate_up_silu", lib.nh_q8_0_debug_gemm_tiled_gate_up_silu(w_gate.data_ptr(), w_up.data_ptr(), aq_tiled.data_ptr(), out.data_ptr(), gate.data_ptr(),
                                                                                                          up.data_ptr(), m, n_ff, k, _stream()))
        return out, gate, up
    need = lib.nh_q8_0_gate_up_silu_workspace_bytes(m, n_ff, k)
    _lib.check("nh_q8_0_gate_up_silu_workspace_bytes", need if need < 0 else 0)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=aq_tiled.device)
    _lib.check("nh_q8_0_gemm_tiled_gate_up_silu", lib.nh_q8_0_gemm_tiled_gate_up_silu(w_gate.data_ptr(), w_up.data_ptr(), aq_tiled.data_ptr(), out.data_ptr(), ws.data_ptr(), ws.numel(), m, n_ff, k, _stream()))
    return out


def mul_mat(w_tiled: torch.Tensor, x: torch.Tensor, n: int, k: int, workspace: torch.Tensor | None = None, residual: torch.Tensor | None = None) -> torch.Tensor:
    """fp32 activations [M, K] x tiled Q8_0 weight [N, K] -> fp32 [M, N]: quantize + GEMV/GEMM (+ residual [M, N] if given)."""
    w_tiled, x = _dev(w_tiled, torch.uint8, "w_tiled"), _dev(x, torch.float32, "x")
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    m = x2.shape[0]
    if x2.shape[1] != k or w_tiled.numel() != tiled_bytes(n, k):
        raise ValueError("operand sizes do not match m x n x k")
    need = _lib.lib().nh_q8_0_mul_mat_workspace_bytes(m, k)
    _lib.check("nh_q8_0_mul_mat_workspace_bytes", need if need < 0 else 0)
    if workspace is None:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device=x.device)
    y = torch.empty((m, n), dtype=torch.float32, device=x.device)
    if residual is not None:
        residual = _dev(residual, torch.float32, "residual")
        if residual.numel() != m * n:
            raise ValueError("residual must hold m x n floats")
        _lib.check("nh_q8_0_mul_mat_residual", _lib.lib().nh_q8_0_mul_mat_residual(w_tiled.data_ptr(), x2.data_ptr(), residual.data_ptr(), y.data_ptr(), m, n, k, workspace.data_ptr(),
                                                                             workspace.numel(), _stream()))
        return y
    _lib.check("nh_q8_0_mul_mat", _lib.lib().nh_q8_0_mul_mat(w_tiled.data_ptr(), x2.data_ptr(), y.data_ptr(), m, n, k, workspace.data_ptr(), workspace.numel(), _stream()))
    return y


def mul_mat_f32_activations(w_tiled: torch.Tensor, x: torch.Tensor, n: int, k: int) -> torch.Tensor:
    """fp32 activations [M, K] (or [K]) x tiled Q8_0 weight [N, K] -> fp32 [M, N] without quantizing the activations."""
    w_tiled, x = _dev(w_tiled, torch.uint8, "w_tiled"), _dev(x, torch.float32, "x")
    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    if x2.shape[1] != k or w_tiled.numel() != tiled_bytes(n, k):
        raise ValueError("operand sizes do not match m x n x k")
    y = torch.empty((x2.shape[0], n), dtype=torch.float32, device=x.device)
    _lib.check("nh_q8_0_mul_mat_f32_activations", _lib.lib().nh_q8_0_mul_mat_f32_activations(w_tiled.data_ptr(), x2.data_ptr(), y.data_ptr(), x2.shape[0], n, k, _stream()))
    return y


def debug_block_sums(w: torch.Tensor, aq: torch.Tensor, m: int, n: int, k: int, path: int) -> torch.Tensor:
    """int32 [m, n, k/32] block sums: path 0/1 = mat-vec / MFMA kernel on blocks, 2/3 = the same on the tiled layout."""
    sums = torch.full((m, n, k // QK), -(2**31), dtype=torch.int32, device=w.device)
    _lib.check("nh_q8_0_debug_block_sums", _lib.lib().nh_q8_0_debug_block_sums(w.data_ptr(), aq.data_ptr(), sums.data_ptr(), m, n, k, path, _stream()))
    return sums


def fill_weight_blocks(seed: int, n: int, k: int, first_block: int = 0, device="cuda") -> torch.Tensor:
    nblk = n * (k // QK)
    w = torch.empty(nblk * BLOCK_BYTES, dtype=torch.uint8, device=device)
    _lib.check("nh_q8_0_fill_weight_blocks", _lib.lib().nh_q8_0_fill_weight_blocks(w.data_ptr(), seed, first_block, nblk, _stream()))
    return w


def fill_activations(seed: int, count: int, device="cuda") -> torch.Tensor:
    x = torch.empty(count, dtype=torch.float32, device=device)
    _lib.check("nh_q8_0_fill_activations", _lib.lib().nh_q8_0_fill_activations(x.data_ptr(), seed, count, _stream()))
    return x

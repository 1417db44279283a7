"""Shared helpers for the parity tests: seeded inputs, host<->device moves, error measures."""
from __future__ import annotations

import numpy as np

REL_L2_TOL = 1e-4  # fp32 outputs: relative L2 error over the whole output against the CPU restatement


def rel_l2(a: np.ndarray, ref: np.ndarray) -> float:
    a = np.asarray(a, dtype=np.float64).ravel()
    ref = np.asarray(ref, dtype=np.float64).ravel()
    den = np.linalg.norm(ref)
    return float(np.linalg.norm(a - ref) / den) if den > 0 else float(np.linalg.norm(a))


def to_dev(a: np.ndarray):
    import torch

    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def to_host(t) -> np.ndarray:
    return t.detach().cpu().numpy()


def random_blocks(rng: np.random.Generator, rows: int, k: int, scale_sigma: float = 0.01) -> np.ndarray:
    """Rows of packed Q8_0 blocks: quants uniform in [-127,127], d = fp16(|N(0,1)| * scale_sigma)."""
    nb = rows * (k // 32)
    out = np.empty((nb, 34), dtype=np.uint8)
    d = np.abs(rng.standard_normal(nb).astype(np.float32) * np.float32(scale_sigma)).astype(np.float16).view(np.uint16)
    out[:, 0] = d & 0xFF
    out[:, 1] = d >> 8
    out[:, 2:] = rng.integers(-127, 128, size=(nb, 32), dtype=np.int8).view(np.uint8)
    return out.reshape(-1)

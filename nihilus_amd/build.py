"""Builds libnihilus_q8_hip.so (the gfx950 Q8_0 kernels + their C ABI) in-tree with hipcc."""
from __future__ import annotations

import os
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
OBJ_DIR = os.path.join(CSRC, "build")
LIB_NAME = "libnihilus_q8_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

SOURCES = ["q8_0_abi.hip", "q8_0_quantize.hip", "q8_0_layout.hip", "q8_0_get_rows.hip", "q8_0_gemv.hip", "q8_0_gemv_rows.hip", "q8_0_gemv_rows_mfma.hip", "q8_0_gemv_group.hip", "q8_0_mul_mat_f32act.hip", "q8_0_ffn.hip", "q8_0_decode_layer.hip", "q8_0_gemm.hip", "q8_0_gemm_skinny.hip", "q8_0_profile.hip", "gguf_q8_0.cpp"]

# -packed-fp32-ops off: v_pk_{add,mul,fma}_f32 are kept out of the generated code on purpose.
# No -ffast-math: the quantizer needs IEEE divide, unfused multiply and round-half-even.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-fno-fast-math",
    "-ffp-contract=off",
    "-Wall",
    "-Wextra",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results stay in ordinary VGPRs: the mat-mat converts every int32 block sum on the VALU right away, and a
    # result parked in an accumulation register would cost one extra copy instruction per value (doubling the VALU work)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]
# the host pass does not know the packed-fp32 feature name and says so once per source: not an error
NOISE = "is not a recognized feature for this target"


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the Q8_0 library can only be built with ROCm's hipcc")
    return exe


def _run(cmd: list[str]) -> str:
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if NOISE not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{' '.join(cmd)}\n{err}")
    return err


def _newest_header_mtime(include: str) -> float:
    newest = 0.0
    for folder in (CSRC, os.path.join(include, "nihilus_amd")):
        for name in os.listdir(folder):
            if name.endswith(".h"):
                newest = max(newest, os.path.getmtime(os.path.join(folder, name)))
    return newest


def build_library(verbose: bool = False, extra_flags: list[str] | None = None, incremental: bool = False, jobs: int = 8) -> str:
    """Compile every HIP source to an object (in parallel) and link them into one shared library next to this file.

    Recompiles everything unless incremental=True, which keeps objects newer than their source and every header.
    """
    include = os.path.join(os.path.dirname(PKG_DIR), "include")
    os.makedirs(OBJ_DIR, exist_ok=True)
    flags = [*HIPCC_FLAGS, "-I", include, *(extra_flags or [])]
    headers = _newest_header_mtime(include)

    def compile_one(src: str) -> str:
        path = os.path.join(CSRC, src)
        obj = os.path.join(OBJ_DIR, os.path.splitext(src)[0] + ".o")
        if incremental and not extra_flags and os.path.exists(obj) and os.path.getmtime(obj) > max(os.path.getmtime(path), headers):
            return ""
        return _run([hipcc(), *flags, "-c", path, "-o", obj])

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        notes = list(pool.map(compile_one, SOURCES))
    objs = [os.path.join(OBJ_DIR, os.path.splitext(s)[0] + ".o") for s in SOURCES]
    notes.append(_run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH, *objs]))
    if verbose:
        text = "\n".join(n for n in notes if n.strip())
        if text:
            print(text)
    return LIB_PATH


if __name__ == "__main__":
    import sys

    print(build_library(verbose=True, incremental="--incremental" in sys.argv))

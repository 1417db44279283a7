"""Builds libnihilus_q8_hip.so (the gfx950 Q8_0 kernels + their C ABI) in-tree with hipcc."""
from __future__ import annotations

import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libnihilus_q8_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

SOURCES = ["q8_0_abi.hip", "q8_0_quantize.hip", "q8_0_layout.hip", "q8_0_get_rows.hip", "q8_0_gemv.hip", "q8_0_gemv_rows.hip", "q8_0_gemv_group.hip", "q8_0_mul_mat_f32act.hip", "q8_0_ffn.hip", "q8_0_gemm.hip", "q8_0_gemm_skinny.hip", "q8_0_profile.hip", "gguf_q8_0.cpp"]

# -packed-fp32-ops off: v_pk_{add,mul,fma}_f32 are kept out of the generated code on purpose.
# No -ffast-math: the quantizer needs IEEE divide, unfused multiply and round-half-even.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++20",
    "-fPIC",
    "-shared",
    "-fno-fast-math",
    "-ffp-contract=off",
    "-Wall",
    "-Wextra",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # MFMA results stay in ordinary VGPRs: the mat-mat converts every int32 block sum on the VALU right away, and a
    # result parked in an accumulation register would cost one extra copy instruction per value (doubling the VALU work)
    "-mllvm", "-amdgpu-mfma-vgpr-form",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; the Q8_0 library can only be built with ROCm's hipcc")
    return exe


def build_library(verbose: bool = False, extra_flags: list[str] | None = None) -> str:
    """Compile every HIP source into one shared library next to this file. Always recompiles."""
    include = os.path.join(os.path.dirname(PKG_DIR), "include")
    cmd = [hipcc(), *HIPCC_FLAGS, "-I", include, *(extra_flags or []), "-o", LIB_PATH, *[os.path.join(CSRC, s) for s in SOURCES]]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass does not know the packed-fp32 feature name and says so once per source: not an error
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed ({res.returncode}):\n{' '.join(cmd)}\n{err}")
    if verbose and err.strip():
        print(err)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))

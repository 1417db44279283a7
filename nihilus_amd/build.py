"""Builds libnihilus_q8_hip.so (the gfx950 Q8_0 kernels + their C ABI) in-tree with hipcc."""
from __future__ import annotations

import os
import shutil
import subprocess

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_NAME = "libnihilus_q8_hip.so"
LIB_PATH = os.path.join(PKG_DIR, LIB_NAME)

SOURCES = ["q8_0_abi.hip", "q8_0_quantize.hip", "q8_0_layout.hip", "q8_0_get_rows.hip", "q8_0_gemv.hip", "q8_0_gemv_rows.hip", "q8_0_ffn.hip", "q8_0_gemm.hip", "q8_0_gemm_skinny.hip", "q8_0_profile.hip", "gguf_q8_0.cpp"]

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


HOST_TEST_SRC = os.path.join(os.path.dirname(PKG_DIR), "tests", "cpp", "test_mul_mat_dispatch.cpp")
HOST_TEST_BIN = os.path.join(os.path.dirname(PKG_DIR), "tests", "cpp", "test_mul_mat_dispatch")


def build_host_tests() -> str:
    """Compile the C++23 dispatch-surface test: a host-only translation unit (no HIP header) linked against the C ABI
    library and the CPU checker.  Needs build_library() and oracle/ built first."""
    root = os.path.dirname(PKG_DIR)
    cxx = os.path.join(os.path.dirname(hipcc()), "amdclang++")
    if not os.path.exists(cxx):
        cxx = "/opt/rocm/bin/amdclang++"
    oracle_dir = os.path.join(root, "oracle")
    cmd = [
        cxx, "-std=c++23", "-O2", "-Wall", "-Wextra", "-I", os.path.join(root, "include"), HOST_TEST_SRC, "-o", HOST_TEST_BIN,
        "-L", PKG_DIR, "-lnihilus_q8_hip", "-L", oracle_dir, "-lq8_0_oracle",
        f"-Wl,-rpath,$ORIGIN/../../nihilus_amd", f"-Wl,-rpath,$ORIGIN/../../oracle", "-Wl,-rpath,/opt/rocm/lib",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host test build failed:\n{' '.join(cmd)}\n{res.stderr}")
    return HOST_TEST_BIN


if __name__ == "__main__":
    print(build_library(verbose=True))

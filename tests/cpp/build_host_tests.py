"""Builds the C++23 dispatch-surface test: a host-only translation unit (no HIP header) linked against the C-ABI
library and the CPU checker.  Needs the library (nihilus_amd.build.build_library) and oracle/ built first."""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HOST_TEST_SRC = os.path.join(HERE, "test_mul_mat_dispatch.cpp")
HOST_TEST_BIN = os.path.join(HERE, "test_mul_mat_dispatch")


def build_host_tests() -> str:
    from nihilus_amd.build import PKG_DIR, hipcc

    cxx = os.path.join(os.path.dirname(hipcc()), "amdclang++")
    if not os.path.exists(cxx):
        cxx = "/opt/rocm/bin/amdclang++"
    oracle_dir = os.path.join(ROOT, "oracle")
    cmd = [
        cxx, "-std=c++23", "-O2", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "include"), HOST_TEST_SRC, "-o", HOST_TEST_BIN,
        "-L", PKG_DIR, "-lnihilus_q8_hip", "-L", oracle_dir, "-lq8_0_oracle",
        "-Wl,-rpath,$ORIGIN/../../nihilus_amd", "-Wl,-rpath,$ORIGIN/../../oracle", "-Wl,-rpath,/opt/rocm/lib",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host test build failed:\n{' '.join(cmd)}\n{res.stderr}")
    return HOST_TEST_BIN


if __name__ == "__main__":
    print(build_host_tests())

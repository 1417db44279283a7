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
MEGA_TEST_BIN = os.path.join(HERE, "test_mega_dispatch")  # the live dispatch point (core_types key), run on the GPU
REFERENCE_MODE_BIN = os.path.join(HERE, "test_reference_mode_compiles")  # the headers against the reference's own primary template
LAUNCH_FLOOR_BIN = os.path.join(HERE, "launch_floor_probe")  # cost of a dispatch that does nothing (a HIP program of its own, no library)
READ_PROBE_BIN = os.path.join(HERE, "read_probe")  # what a bare read of a matrix's bytes costs (a HIP program of its own, no library)
COISSUE_PROBE_BIN = os.path.join(HERE, "coissue_probe")  # whether the matrix pipe and the VALU of a SIMD overlap (a HIP program of its own, no library)
TIME_MEGA_BIN = os.path.join(HERE, "time_mega_dispatch")  # decode token timed through the dispatch point (links the library only, not the checker)


def _build_one(src: str, out: str, with_checker: bool = True) -> str:
    from nihilus_amd.build import PKG_DIR, hipcc

    cxx = os.path.join(os.path.dirname(hipcc()), "amdclang++")
    if not os.path.exists(cxx):
        cxx = "/opt/rocm/bin/amdclang++"
    oracle_dir = os.path.join(ROOT, "oracle")
    cmd = [
        cxx, "-std=c++23", "-O2", "-Wall", "-Wextra", "-I", os.path.join(ROOT, "include"), os.path.join(HERE, src), "-o", out,
        "-L", PKG_DIR, "-lnihilus_q8_hip", "-Wl,-rpath,$ORIGIN/../../nihilus_amd", "-Wl,-rpath,/opt/rocm/lib",
    ]
    if with_checker:
        cmd += ["-L", oracle_dir, "-lq8_0_oracle", "-Wl,-rpath,$ORIGIN/../../oracle"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"host test build failed:\n{' '.join(cmd)}\n{res.stderr}")
    return out


def _build_probe(src: str, out: str, extra: tuple[str, ...] = ()) -> str:
    """A stand-alone HIP measurement program (no library): the library's own device flags."""
    from nihilus_amd.build import hipcc

    cmd = [hipcc(), "--offload-arch=gfx950", "-O3", "-std=c++20", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", *extra,
           os.path.join(HERE, src), "-o", out]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"probe build failed:\n{' '.join(cmd)}\n{res.stderr}")
    return out


def build_host_tests() -> str:
    _build_probe("launch_floor_probe.hip", LAUNCH_FLOOR_BIN)
    _build_probe("read_probe.hip", READ_PROBE_BIN)
    _build_probe("coissue_probe.hip", COISSUE_PROBE_BIN, ("-mllvm", "-amdgpu-mfma-vgpr-form"))
    _build_one("test_mega_dispatch.cpp", MEGA_TEST_BIN)
    _build_one("time_mega_dispatch.cpp", TIME_MEGA_BIN, with_checker=False)
    _build_one("test_reference_mode_compiles.cpp", REFERENCE_MODE_BIN)
    return _build_one("test_mul_mat_dispatch.cpp", HOST_TEST_BIN)


FUZZ_SRC = os.path.join(HERE, "fuzz_gguf.cpp")
FUZZ_BIN = os.path.join(HERE, "fuzz_gguf")


def build_gguf_fuzz() -> str:
    """The GGUF reader's source compiled with AddressSanitizer + UBSan into a mutation driver (host code only; the upload path's
    HIP and tile symbols resolve against the built library and are never called)."""
    from nihilus_amd.build import CSRC, PKG_DIR

    cmd = [
        "g++", "-std=c++20", "-g", "-O1", "-fsanitize=address,undefined", "-fno-sanitize-recover=undefined", "-D__HIP_PLATFORM_AMD__",
        "-I", os.path.join(ROOT, "include"), "-I", "/opt/rocm/include", FUZZ_SRC, os.path.join(CSRC, "gguf_q8_0.cpp"), "-o", FUZZ_BIN,
        "-L", PKG_DIR, "-lnihilus_q8_hip", "-L", "/opt/rocm/lib", "-lamdhip64", "-Wl,-rpath,$ORIGIN/../../nihilus_amd", "-Wl,-rpath,/opt/rocm/lib",
    ]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"fuzz driver build failed:\n{' '.join(cmd)}\n{res.stderr}")
    return FUZZ_BIN


if __name__ == "__main__":
    print(build_host_tests())
    print(build_gguf_fuzz())

"""CPU: the C-ABI library loads, exports every function the header declares, and rejects bad arguments before it
touches a device.  No compute call is made here."""
import ctypes as C
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "nihilus_amd", "q8_0_abi.h")


def _declared_functions() -> list[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(nh_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from nihilus_amd import _lib

    lib = _lib.lib()
    names = _declared_functions()
    assert len(names) >= 25
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in q8_0_abi.h but not exported"
    # and the Python binding table names exactly the declared functions
    assert sorted(_lib.SIGNATURES) == names
    assert lib.nh_abi_version() == 1


def test_size_helpers_and_status_strings():
    from nihilus_amd import _lib

    lib = _lib.lib()
    assert lib.nh_q8_0_blocks_bytes(4096, 4096) == 17825792  # blk.0.attn_q.weight in the reference's dump
    assert lib.nh_q8_0_blocks_bytes(128256, 4096) == 558170112
    assert lib.nh_q8_0_tiled_bytes(4096, 4096) == 17825792  # same bytes per block, rows already a multiple of 32
    assert lib.nh_q8_0_tiled_bytes(33, 128) == 2 * 4352  # rows padded to the next strip
    assert lib.nh_q8_0_blocks_bytes(1, 33) == -3 and lib.nh_q8_0_tiled_bytes(1, 96) == -3 and lib.nh_q8_0_blocks_bytes(-1, 32) == -3
    assert lib.nh_q8_0_mul_mat_workspace_bytes(1, 4096) % 256 == 0
    assert lib.nh_q8_0_mul_mat_workspace_bytes(512, 4096) >= 512 * 128 * 34
    for code in range(-6, 1):
        assert _lib.status_string(code)
    assert "null" in _lib.status_string(-1) and "aligned" in _lib.status_string(-2)


def test_arguments_are_rejected_before_any_device_work():
    from nihilus_amd import _lib

    lib = _lib.lib()
    bogus = 0x1000  # never dereferenced: every call below must fail in validation
    assert lib.nh_q8_0_quantize(bogus, bogus, 1, 33, None) == -3
    assert lib.nh_q8_0_quantize(bogus, bogus, -1, 32, None) == -3
    assert lib.nh_q8_0_quantize(None, bogus, 1, 32, None) == -1
    assert lib.nh_q8_0_quantize(bogus + 4, bogus, 1, 32, None) == -2
    assert lib.nh_q8_0_quantize_tiled(bogus, bogus, 1, 96, None) == -3
    assert lib.nh_q8_0_gemv(bogus, bogus, bogus, 32, 100, None) == -3
    assert lib.nh_q8_0_gemv(bogus, bogus, bogus, 32, 1 << 20, None) == -5
    assert lib.nh_q8_0_gemv(None, bogus, bogus, 32, 128, None) == -1
    assert lib.nh_q8_0_gemv_tiled(bogus, bogus, bogus, 32, 96, None) == -3
    assert lib.nh_q8_0_gemv_tiled_f32(bogus, None, bogus, 32, 128, None) == -1
    assert lib.nh_q8_0_gemm(bogus, bogus, bogus + 8, 4, 32, 128, None) == -2
    assert lib.nh_q8_0_gemm_tiled(bogus, bogus, bogus, 4, 32, 32, None) == -3
    assert lib.nh_q8_0_mul_mat(bogus, bogus, bogus, 4, 32, 128, bogus, 0, None) == -6  # workspace too small
    assert lib.nh_q8_0_debug_block_sums(bogus, bogus, bogus, 2, 32, 128, 0, None) == -6  # mat-vec path needs M == 1
    assert lib.nh_q8_0_debug_block_sums(bogus, bogus, bogus, 1, 32, 128, 9, None) == -6
    assert lib.nh_profile_begin(7, 10) == -6 and lib.nh_profile_end(None, None, None, None) == -6
    assert lib.nh_q8_0_mul_mat_batch(None, 3, None, 0, None) == -1
    ops = (_lib.MulMatOp * 1)(_lib.MulMatOp(bogus, bogus, bogus, 1, 32, 100, 0, 0))
    assert lib.nh_q8_0_mul_mat_batch(ops, 1, None, 0, None) == -3
    ops = (_lib.MulMatOp * 1)(_lib.MulMatOp(bogus, bogus + 4, bogus, 1, 32, 128, 0, 0))
    assert lib.nh_q8_0_mul_mat_batch(ops, 1, None, 0, None) == -2  # misaligned x: caught before the first launch
    vp, i64 = C.c_void_p * 2, C.c_int64 * 2
    w, x, y = vp(bogus, bogus), vp(bogus, bogus), vp(bogus, bogus)
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, x, y, None, i64(32, 32), i64(128, 100), 2, None) == -3
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, x, y, None, i64(32, 32), i64(128, 128), -1, None) == -6
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, None, y, None, i64(32, 32), i64(128, 128), 2, None) == -1
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, vp(bogus, None), y, None, i64(32, 32), i64(128, 128), 2, None) == -1
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, x, vp(bogus, bogus + 8), None, i64(32, 32), i64(128, 128), 2, None) == -2
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, x, y, vp(bogus, bogus + 4), i64(32, 32), i64(128, 128), 2, None) == -2
    assert lib.nh_q8_0_gemv_tiled_group_f32(w, x, y, None, i64(0, 0), i64(128, 128), 2, None) == 0  # nothing to do
    # empty work is success without a device
    assert lib.nh_q8_0_quantize(None, None, 0, 32, None) == 0
    assert lib.nh_q8_0_gemm(None, None, None, 0, 0, 128, None) == 0
    assert lib.nh_q8_0_mul_mat_batch(None, 0, None, 0, None) == 0


def test_fails_loudly_without_a_gpu():
    import torch

    from nihilus_amd import _lib

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = _lib.lib()
    p = C.c_void_p()
    assert lib.nh_malloc(C.byref(p), 1024) == -4  # no device: an error, never a silent CPU path
    assert lib.nh_q8_0_prepare() == -4
    # the row limit of the mat-mat follows the launch grid of the kernel that would run (checked before any device call):
    # 32 rows per workgroup row on tiled operands, 128 on packed blocks
    assert lib.nh_q8_0_gemm_tiled(None, None, None, 65535 * 32 + 1, 32, 128, None) == -5
    assert lib.nh_q8_0_gemm_tiled(None, None, None, 65535 * 32, 32, 128, None) == -1
    assert lib.nh_q8_0_gemm(None, None, None, 65535 * 128 + 1, 32, 128, None) == -5
    assert lib.nh_q8_0_gemm(None, None, None, 65535 * 128, 32, 128, None) == -1
    assert lib.nh_q8_0_last_error() == -4
    # the status plumbing of the device-side reports needs no device
    assert "another stream" in _lib.status_string(-10) and "bounded wait" in _lib.status_string(-11)
    # the spin-limit test hook works only for a process that opted in through its environment
    os.environ.pop("NH_Q8_0_DEBUG_HOOKS", None)
    assert lib.nh_q8_0_debug_set_spin_limit(1 << 20) == -6
    os.environ["NH_Q8_0_DEBUG_HOOKS"] = "1"
    try:
        assert lib.nh_q8_0_debug_set_spin_limit(0) == -6 and lib.nh_q8_0_debug_set_spin_limit(1 << 20) == 0
    finally:
        os.environ.pop("NH_Q8_0_DEBUG_HOOKS", None)
    assert lib.nh_q8_0_clear_error() == -4
    assert lib.nh_q8_0_quantize(0x1000, 0x2000, 1, 32, None) == -4
    with pytest.raises(_lib.Q8Error):
        _lib.check("nh_q8_0_quantize", lib.nh_q8_0_quantize(0x1000, 0x2000, 1, 32, None))


def test_product_never_imports_the_checker():
    # nothing under nihilus_amd/ or include/ may reference oracle/
    for base in ("nihilus_amd", "include"):
        for dirpath, _, files in os.walk(os.path.join(ROOT, base)):
            for f in files:
                if f.endswith((".py", ".h", ".hpp", ".hip", ".cpp")):
                    text = open(os.path.join(dirpath, f), errors="ignore").read()
                    assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
                    assert "q8_0_oracle" not in text, f


def test_bench_refuses_more_than_one_gpu():
    res = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert res.returncode != 0 and "ONE GPU" in res.stderr


def _host_tests():
    sys.path.insert(0, os.path.join(ROOT, "tests", "cpp"))
    import build_host_tests as b

    return b


def test_cpp_dispatch_surface_compiles_and_static_checks_hold():
    b = _host_tests()

    exe = b.HOST_TEST_BIN
    if not os.path.exists(exe):
        import oracle  # noqa: F401  (builds the checker the C++ test links against)

        b.build_host_tests()
    res = subprocess.run([exe, "--compile-only-check"], capture_output=True, text=True)
    assert res.returncode == 0 and "static checks ok" in res.stdout


def test_cpp_live_dispatch_point_compiles_against_the_reference_declaration():
    # mega_dispatch.hpp / mul_mat_dispatch.hpp with NIHILUS_AMD_WITH_REFERENCE_HEADERS: every reference name comes from a
    # test-local header whose primary template is the reference's own declaration of the live specialisation point; all eight
    # specialisations are instantiated through the reference's caller-side template.  Also the stand-alone build's static checks.
    b = _host_tests()
    if not (os.path.exists(b.REFERENCE_MODE_BIN) and os.path.exists(b.MEGA_TEST_BIN) and os.path.exists(b.TIME_MEGA_BIN) and os.path.exists(b.LAUNCH_FLOOR_BIN)):
        import oracle  # noqa: F401

        b.build_host_tests()
    res = subprocess.run([b.REFERENCE_MODE_BIN], capture_output=True, text=True)
    assert res.returncode == 0 and "reference-mode build ok" in res.stdout
    res = subprocess.run([b.MEGA_TEST_BIN, "--compile-only-check"], capture_output=True, text=True)
    assert res.returncode == 0 and "static checks ok" in res.stdout
    # the mode switch is real: the headers must not pull the mirror in when the reference's names are already there
    text = open(os.path.join(ROOT, "include", "nihilus_amd", "mul_mat_dispatch.hpp")).read()
    assert re.search(r"#ifndef NIHILUS_AMD_WITH_REFERENCE_HEADERS\s+#include \"reference_mirror.hpp\"", text)


def test_customisation_points_must_be_specialised_by_a_real_config():
    # a config without rope / attention / sampling hooks that does not declare amd_matmul_only must be stopped by the compiler
    from nihilus_amd.build import hipcc

    cxx = os.path.join(os.path.dirname(hipcc()), "amdclang++")
    src = os.path.join(ROOT, "tests", "cpp", "customisation_points_are_mandatory.cpp")
    res = subprocess.run([cxx, "-std=c++23", "-fsyntax-only", "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "tests", "cpp"), src], capture_output=True, text=True)
    errors = [ln for ln in res.stderr.splitlines() if " error: " in ln]
    assert res.returncode != 0 and len(errors) == 1, res.stderr
    assert "specialise nihilus::amd_attention<config>" in errors[0] and "amd_matmul_only" in errors[0]


@pytest.mark.gpu
def test_cpp_live_dispatch_point_on_gpu():
    # the four mega cores, both phases, through kernel_dispatcher<config, phase, core>::impl on a two-block graph
    b = _host_tests()
    res = subprocess.run([b.MEGA_TEST_BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "mega dispatch ok" in res.stdout


@pytest.mark.gpu
def test_launch_floor_probe_runs():
    import json

    b = _host_tests()
    res = subprocess.run([b.LAUNCH_FLOOR_BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    out = json.loads(res.stdout.strip().splitlines()[-1])
    assert all(0.2 < v < 20.0 for v in out["empty_kernel_queued_us"] + out["one_load_kernel_queued_us"])


@pytest.mark.gpu
def test_read_probe_and_coissue_probe_run():
    import json

    b = _host_tests()
    res = subprocess.run([b.READ_PROBE_BIN, "17825792", "62390272"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    reads = json.loads(res.stdout.strip().splitlines()[-1])["reads"]
    assert [r["bytes"] for r in reads] == [17825792, 62390272] and all(1000 < r["GBs"] < 8000 for r in reads)
    res = subprocess.run([b.COISSUE_PROBE_BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    out = json.loads(res.stdout.strip().splitlines()[-1])
    assert 28 < out["clocks_per_mfma"] < 40 and 1.5 < out["clocks_per_valu_instruction"] < 6
    assert 0.5 < out["at_four_waves"]["fraction_of_sum"] <= 1.1


@pytest.mark.gpu
def test_shader_clock_can_be_read():
    from nihilus_amd import _lib

    lib = _lib.lib()
    mhz = C.c_double()
    assert lib.nh_profile_shader_clock(C.byref(mhz), 200) == 0
    assert 300.0 < mhz.value < 3000.0, mhz.value
    assert lib.nh_profile_shader_clock(None, 200) == -6 and lib.nh_profile_shader_clock(C.byref(mhz), 0) == -6


@pytest.mark.gpu
def test_decode_token_timed_through_the_dispatch_point():
    # the measurement's own entry through the C++ dispatch header: a whole LLaMA-3-8B-shaped token and the FFN core alone
    import json

    b = _host_tests()
    res = subprocess.run([b.TIME_MEGA_BIN, "3", "1"], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    out = json.loads(res.stdout.strip().splitlines()[-1])
    assert out["decode"]["weight_bytes_per_token"] == 7973699584 and out["decode"]["tok_s"] > 100
    assert out["mega_ffn"]["GBs"] > 1000


@pytest.mark.gpu
def test_cpp_dispatch_surface_on_gpu():
    b = _host_tests()

    res = subprocess.run([b.HOST_TEST_BIN], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, res.stdout + res.stderr
    assert "mul_mat dispatch ok" in res.stdout

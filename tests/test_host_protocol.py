"""Builds and runs the C++ host-logic test (timing protocol with a fake clock, driver
stdout formats, GemmResult layout) with the host compiler; no GPU involved."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_host_protocol(tmp_path):
    exe = tmp_path / "test_host_protocol"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__",
                    "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "cudaintro_amd", "csrc"),
                    "-I", "/opt/rocm/include", os.path.join(ROOT, "tests", "cpp", "test_host_protocol.cpp"),
                    "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "host protocol OK" in out.stdout


def test_skinny_plan(tmp_path):
    """The decode kernel's choice of K ranges (csrc/skinny_plan.h): the counts the rule was
    measured at, and its invariants over a sweep of sizes."""
    exe = tmp_path / "test_skinny_plan"
    subprocess.run(["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "cudaintro_amd", "csrc"),
                    os.path.join(ROOT, "tests", "cpp", "test_skinny_plan.cpp"), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "skinny plan OK" in out.stdout


def test_gemm_common_header_names():
    """The drop-in header keeps the record and the four entry-point names."""
    text = open(os.path.join(ROOT, "include", "gemm_common.h")).read()
    for name in ("struct GemmResult", "run_gemm_bf16", "run_gemm_fp16", "run_gemm_fp32", "run_gemm_int8",
                 "const char* name;", "uint64_t iters;", "double secs;", "double tflops;"):
        assert name in text


def test_bench_refuses_more_than_one_gpu():
    """`bench.py --gpus N` with N > 1 exits with a message before it touches the GPU."""
    import sys
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                         capture_output=True, text=True, timeout=60)
    assert out.returncode != 0
    assert "one GPU" in (out.stdout + out.stderr)


def test_fill_kernels_division_free_forms_are_exact(tmp_path):
    """The device fills replace the IEEE division by 2^24 - 1 and the integer modulo by
    multiply-based forms; this checks them against the plain expressions for every operand."""
    exe = tmp_path / "test_exact_arith"
    subprocess.run(["gcc", "-O2", "-std=c11", "-ffp-contract=off", "-Wall",
                    os.path.join(ROOT, "tests", "cpp", "test_exact_arith.c"), "-o", str(exe), "-lm"],
                   check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stdout + out.stderr
    assert "exact arithmetic OK" in out.stdout


def test_gemm_suite_exits_with_the_reference_message_without_a_device():
    """The driver keeps the reference's fail-fast behaviour (quantization/gemm_common.h:47-55):
    a failing library call prints "cigemm error: <status> at <file>:<line>" to stderr and exits
    with status 1.  Without a GPU the first such call is cigemmCreate."""
    import re

    import pytest
    import torch

    import cudaintro_amd
    if torch.cuda.is_available():
        pytest.skip("a GPU is present: cigemmCreate succeeds")
    exe = cudaintro_amd.suite_path()
    assert os.path.exists(exe), "gemm_suite is not built"
    out = subprocess.run([exe, "--seconds", "0.01", "--size", "256"], capture_output=True, text=True,
                         timeout=120)
    assert out.returncode == 1, (out.returncode, out.stderr)
    assert re.search(r"cigemm error: CIGEMM_STATUS_\w+ at \S*main\.cpp:\d+\s*$", out.stderr), out.stderr
    assert "Running" not in out.stdout

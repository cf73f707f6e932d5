"""The host-side C and C++ of this repository under AddressSanitizer and
UndefinedBehaviorSanitizer (host compiler, CPU only, no GPU code involved): the oracle, through a
driver that calls every one of its functions on exactly sized heap buffers, and the three host
test programs (timing protocol and output formats, the decode planner, the exact-arithmetic
forms of the fill kernels).  Any report aborts the program (-fno-sanitize-recover)."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CPP = os.path.join(ROOT, "tests", "cpp")
SAN = ["-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-fno-omit-frame-pointer", "-g",
       "-static-libasan"]
ENV = dict(os.environ, ASAN_OPTIONS="detect_leaks=1:abort_on_error=0", UBSAN_OPTIONS="print_stacktrace=1",
           OMP_NUM_THREADS="4")

PROGRAMS = {
    "test_oracle_sanitized": (["gcc", "-std=c11", "-O1", "-fopenmp", "-ffp-contract=off", "-Wall"],
                              "test_oracle_sanitized.c", ["-lm"], "oracle sanitized OK"),
    "test_host_protocol": (["g++", "-std=c++17", "-O1", "-Wall", "-D__HIP_PLATFORM_AMD__",
                            "-I", os.path.join(ROOT, "include"), "-I", os.path.join(ROOT, "cudaintro_amd", "csrc"),
                            "-I", "/opt/rocm/include"], "test_host_protocol.cpp", [], "host protocol OK"),
    "test_skinny_plan": (["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "cudaintro_amd", "csrc")],
                         "test_skinny_plan.cpp", [], "skinny plan OK"),
    "test_tile_plan": (["g++", "-std=c++17", "-O1", "-Wall", "-I", os.path.join(ROOT, "cudaintro_amd", "csrc")],
                       "test_tile_plan.cpp", [], "tile plan OK"),
    # (the sweep over all 2^24 numerators runs some ten times slower instrumented: still seconds)
    "test_exact_arith": (["gcc", "-O2", "-std=c11", "-ffp-contract=off", "-Wall"], "test_exact_arith.c", ["-lm"],
                         "exact arithmetic OK"),
}


@pytest.mark.parametrize("name", sorted(PROGRAMS))
def test_host_program_is_clean_under_asan_and_ubsan(tmp_path, name):
    cc, src, libs, ok = PROGRAMS[name]
    exe = tmp_path / name
    subprocess.run([*cc, *SAN, os.path.join(CPP, src), "-o", str(exe), *libs], check=True)
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=900, env=ENV)
    if "ASan runtime does not come first" in out.stderr:
        pytest.skip("a preloaded library keeps AddressSanitizer from starting in this environment")
    assert out.returncode == 0, out.stdout[-2000:] + out.stderr[-4000:]
    assert ok in out.stdout
    assert "runtime error" not in out.stderr and "AddressSanitizer" not in out.stderr

"""The suite driver and the reference workload (4096^3 filled by the reference generator,
quantization/GEMM_*.cu:20-25, 41-46) checked against the oracle."""
import os
import re
import subprocess

import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import bits, error_bound_16

pytestmark = pytest.mark.gpu


def test_gemm_suite_driver_output():
    exe = ci.suite_path()
    assert os.path.exists(exe), "gemm_suite is not built"
    out = subprocess.run([exe, "--seconds", "0.25", "--size", "1024"], capture_output=True, text=True,
                         timeout=240)
    assert out.returncode == 0, out.stdout + out.stderr
    lines = out.stdout.strip().splitlines()
    assert lines[:4] == ["Running BF16...", "Running FP16...", "Running FP32...", "Running INT8..."]
    names = []
    for line in lines[4:]:
        m = re.fullmatch(r"Ran (\d+) (\w+) GEMMs in ([\d.e+-]+) s \(([\d.e+-]+) TFLOP/s\)", line)
        assert m, line
        iters, name, secs, tflops = int(m[1]), m[2], float(m[3]), float(m[4])
        names.append(name)
        assert iters % 256 == 0 and iters > 0 and secs >= 0.25
        assert abs(tflops - 2.0 * 1024 ** 3 * iters / (secs * 1e12)) <= 1e-3 * tflops
    assert names == ["BF16", "FP16", "FP32", "INT8"]


def test_reference_workload_int8_4096(handle, torch_gpu, oracle):
    torch = torch_gpu
    n = 4096
    a = handle.fill_random(torch.empty((n, n), dtype=torch.int8, device="cuda"), 0x4234, -127, 127)
    b = handle.fill_random(torch.empty((n, n), dtype=torch.int8, device="cuda"), 0x6676, -127, 127)
    c = handle.gemm_i8_i32(a, b)
    A = oracle.fill_random_i8(n * n, 0x4234).reshape(n, n)
    B = oracle.fill_random_i8(n * n, 0x6676).reshape(n, n)
    np.testing.assert_array_equal(c.cpu().numpy(), oracle.gemm_i8_i32(A, B))


@pytest.mark.parametrize("kind,sa,sb", [("bf16", 0x1234, 0x9876), ("f16", 0x2234, 0x8876)])
def test_reference_workload_16bit_4096(handle, torch_gpu, oracle, kind, sa, sb):
    torch = torch_gpu
    n = 4096
    dt = torch.bfloat16 if kind == "bf16" else torch.float16
    a = handle.fill_random(torch.empty((n, n), dtype=dt, device="cuda"), sa)
    b = handle.fill_random(torch.empty((n, n), dtype=dt, device="cuda"), sb)
    c = (handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16)(a, b)
    fill = oracle.fill_random_bf16 if kind == "bf16" else oracle.fill_random_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    A = widen(fill(n * n, sa)).reshape(n, n)
    B = widen(fill(n * n, sb)).reshape(n, n)
    got = widen(bits(torch, c)).astype(np.float64)
    for r0 in (0, 1000, 4088):
        ref, S = oracle.gemm_f64(A, B, rows=(r0, r0 + 8), with_abs=True)
        assert (np.abs(got[r0:r0 + 8] - ref) <= error_bound_16(ref, S, n, kind)).all()


def test_reference_workload_fp32_4096(handle, torch_gpu, oracle):
    torch = torch_gpu
    n = 4096
    a = handle.fill_random(torch.empty((n, n), dtype=torch.float32, device="cuda"), 0x3234)
    b = handle.fill_random(torch.empty((n, n), dtype=torch.float32, device="cuda"), 0x7776)
    c = handle.gemm_f32(a, b).cpu().numpy()
    A = oracle.fill_random_f32(n * n, 0x3234).reshape(n, n)
    B = oracle.fill_random_f32(n * n, 0x7776).reshape(n, n)
    # rows of the reference CPU loop (i-j-k, float accumulator)
    cpu = oracle.gemm_f32_ijk(A, B, 0, 16)[:16]
    rms = float(np.sqrt(np.mean(cpu.astype(np.float64) ** 2)))
    lim = 1e-5 * np.maximum(np.abs(cpu), rms)
    assert (np.abs(c[:16].astype(np.float64) - cpu) <= lim).all()
    ref, S = oracle.gemm_f64(A, B, rows=(2048, 2064), with_abs=True)
    assert (np.abs(c[2048:2064] - ref) <= n * 2.0 ** -24 * S).all()

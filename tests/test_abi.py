"""The C-ABI library loads and exports exactly what include/cigemm.h declares, and the
measurement library beside it exactly what include/cigemm_probe.h declares.
No compute call is made here (no GPU)."""
import ctypes
import os
import re
import subprocess

import pytest

import cudaintro_amd
from cudaintro_amd import cigemm, probe

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "cigemm.h")
PROBE_HEADER = os.path.join(ROOT, "include", "cigemm_probe.h")


def declared_symbols(header=HEADER):
    text = open(header).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"CIGEMM_API\s+[\w\s\*]+?\b(cigemm\w+)\s*\(", text)))


def test_header_declares_expected_entry_points():
    names = declared_symbols()
    for must in ["cigemmCreate", "cigemmDestroy", "cigemmSetStream", "cigemm_gemm_f32",
                 "cigemm_gemm_f16", "cigemm_gemm_bf16", "cigemm_gemm_i8_i32",
                 "cigemm_gemm_i8_dequant", "cigemm_fill_random_i8", "cigemm_quantize_rows_i8"]:
        assert must in names
    assert len(names) >= 18


def test_library_exports_every_declared_symbol():
    lib = cudaintro_amd.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), f"{name} declared in cigemm.h but not exported"


def test_binding_covers_every_declared_symbol():
    assert sorted(cigemm.SIGNATURES) == declared_symbols()


def test_no_unexpected_exports():
    """Only the C ABI is visible: no C++ symbols leak from the shared object."""
    assert exported(cudaintro_amd.library_path()) == declared_symbols()


def exported(path):
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True,
                         check=True).stdout
    return sorted(l.split()[-1] for l in out.splitlines() if " T " in l)


def test_probe_library_is_separate_and_matches_its_header():
    """The drop-in library exports no measurement aid; libcigemm_probe.so exports exactly what
    cigemm_probe.h declares and the binding covers it."""
    names = declared_symbols(PROBE_HEADER)
    assert names and all(n.startswith("cigemm_probe_") for n in names)
    assert not [n for n in declared_symbols() if "probe" in n]
    assert not [n for n in exported(cudaintro_amd.library_path()) if "probe" in n]
    lib = probe.load_library()
    for name in names:
        assert hasattr(lib, name), f"{name} declared in cigemm_probe.h but not exported"
    assert exported(probe.library_path()) == names
    assert sorted(probe.SIGNATURES) == names
    # null handle: a status code, never a crash
    assert lib.cigemm_probe_mfma(None, 0, 0, 1, None) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemm_probe_issue_cost(None, 0, 0, 0, 0, 1, 8, 1, 1, None) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemm_probe_dirty_workspace(None, 0, 0, 0) == cigemm.Status.NOT_INITIALIZED


@pytest.mark.parametrize("header", ["cigemm.h", "cigemm_probe.h"])
def test_header_compiles_as_c(tmp_path, header):
    src = tmp_path / "t.c"
    src.write_text('#include "%s"\nint main(void){cigemmHandle_t h=0;(void)h;return CIGEMM_STATUS_SUCCESS;}\n' % header)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    "-c", str(src), "-o", str(tmp_path / "t.o")], check=True)


def test_status_strings_and_null_handle():
    lib = cudaintro_amd.load_library()
    assert lib.cigemmGetStatusString(0) == b"CIGEMM_STATUS_SUCCESS"
    assert lib.cigemmGetStatusString(7) == b"CIGEMM_STATUS_INVALID_VALUE"
    assert lib.cigemmGetStatusString(99) == b"CIGEMM_STATUS_UNKNOWN"
    # every name the reference's table prints (quantization/gemm_common.h:10-35) has a counterpart
    for code, name in {0: "SUCCESS", 1: "NOT_INITIALIZED", 3: "ALLOC_FAILED", 7: "INVALID_VALUE",
                       8: "ARCH_MISMATCH", 11: "MAPPING_ERROR", 13: "EXECUTION_FAILED",
                       14: "INTERNAL_ERROR", 15: "NOT_SUPPORTED", 16: "LICENSE_ERROR"}.items():
        assert lib.cigemmGetStatusString(code) == b"CIGEMM_STATUS_" + name.encode()
        assert cigemm.Status(code).name == name
    assert lib.cigemmGetVersion() >= 100
    # null handle: status code, never a crash
    assert lib.cigemmDestroy(None) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemmSetStream(None, None) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemmResetWorkspace(None) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemm_gemm_f32(None, 1, 1, 1, None, 1, None, 1, None, 1) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemm_gemm_i8_i32(None, 1, 1, 1, None, 1, None, 1, 0, None, 1) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemm_fill_random_f32(None, None, 0, 0, 0.0, 1.0) == cigemm.Status.NOT_INITIALIZED
    assert lib.cigemmCreate(None) == cigemm.Status.INVALID_VALUE
    assert lib.cigemmGetLastErrorString(None) == b""


def test_create_fails_loudly_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    lib = cudaintro_amd.load_library()
    h = ctypes.c_void_p()
    st = lib.cigemmCreate(ctypes.byref(h))
    assert st != 0 and not h.value
    with pytest.raises(cudaintro_amd.CigemmError):
        cudaintro_amd.Handle()

"""Argument validation through the C ABI with a live handle: every bad call returns a
status code and launches nothing."""
import ctypes

import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import Status

pytestmark = pytest.mark.gpu


def test_invalid_arguments(handle, torch_gpu):
    torch = torch_gpu
    lib, h = handle.lib, handle.raw
    a = torch.zeros((8, 8), dtype=torch.float32, device="cuda")
    p = a.data_ptr()
    assert lib.cigemm_gemm_f32(h, -1, 8, 8, p, 8, p, 8, p, 8) == Status.INVALID_VALUE
    assert b"negative" in lib.cigemmGetLastErrorString(h)
    assert lib.cigemm_gemm_f32(h, 8, 8, 8, None, 8, p, 8, p, 8) == Status.INVALID_VALUE
    assert lib.cigemm_gemm_f32(h, 8, 8, 8, p, 8, p, 8, None, 8) == Status.INVALID_VALUE
    assert lib.cigemm_gemm_f32(h, 8, 8, 8, p, 7, p, 8, p, 8) == Status.INVALID_VALUE   # lda < K
    assert lib.cigemm_gemm_f32(h, 8, 8, 8, p, 8, p, 7, p, 8) == Status.INVALID_VALUE   # ldb < N
    assert lib.cigemm_gemm_f32(h, 8, 8, 8, p, 8, p, 8, p, 7) == Status.INVALID_VALUE   # ldc < N
    assert lib.cigemm_gemm_i8_i32(h, 8, 8, 8, p, 8, p, 8, 5, p, 8) == Status.INVALID_VALUE  # layout
    assert lib.cigemm_gemm_i8_dequant(h, 8, 8, 8, p, 8, p, 8, 0, None, 0, p, 0, p, 0, 8, None, 0) \
        == Status.INVALID_VALUE
    assert lib.cigemm_gemm_i8_dequant(h, 8, 8, 8, p, 8, p, 8, 0, p, 2, p, 0, p, 0, 8, None, 0) \
        == Status.INVALID_VALUE
    assert lib.cigemm_gemm_i8_dequant(h, 8, 8, 8, p, 8, p, 8, 0, p, 0, p, 0, p, 3, 8, None, 0) \
        == Status.INVALID_VALUE
    assert lib.cigemm_fill_random_f32(h, None, 4, 0, 0.0, 1.0) == Status.INVALID_VALUE
    assert lib.cigemm_fill_random_i8(h, p, 4, 0, 5, -5) == Status.INVALID_VALUE
    assert lib.cigemm_quantize_rows_i8(h, 4, 4, p, 3, p, 4, p) == Status.INVALID_VALUE
    # the buffer was never written
    torch.cuda.synchronize()
    assert (a.cpu().numpy() == 0).all()
    # M == 0 or N == 0 is a valid no-op
    assert lib.cigemm_gemm_f32(h, 0, 8, 8, None, 8, None, 8, None, 8) == Status.SUCCESS
    a8 = torch.zeros((8, 8), dtype=torch.int8, device="cuda")
    with pytest.raises(ci.CigemmError, match="INVALID_VALUE.*b_layout"):
        handle.gemm_i8_i32(a8, a8, b_layout=5)


def test_destroyed_handle_is_rejected(torch_gpu):
    h = ci.Handle()
    raw = h.raw
    h.close()
    assert h.raw is None
    # a second handle works and uses the stream it was given
    s = torch_gpu.cuda.Stream()
    with torch_gpu.cuda.stream(s):
        h2 = ci.Handle()
        got = ctypes.c_void_p()
        assert h2.lib.cigemmGetStream(h2.raw, ctypes.byref(got)) == 0
        assert (got.value or 0) == s.cuda_stream
        a = torch_gpu.ones((64, 64), device="cuda")
        c = h2.gemm_f32(a, a)
    s.synchronize()
    assert (c.cpu().numpy() == 64).all()
    h2.close()


def test_kernel_family_selection(torch_gpu):
    """cigemmSetAlgo restricts the dispatch; a family that does not take the call refuses it
    with NOT_SUPPORTED, writes nothing, and the handle keeps working."""
    torch = torch_gpu
    h = ci.Handle()
    assert h.get_algo() == ci.ALGO_DEFAULT
    assert h.lib.cigemmSetAlgo(h.raw, 6) == Status.INVALID_VALUE
    assert h.lib.cigemmSetAlgo(h.raw, -2) == Status.INVALID_VALUE
    assert h.lib.cigemmGetAlgo(h.raw, None) == Status.INVALID_VALUE
    a = torch.ones((64, 64), dtype=torch.float32, device="cuda")
    out = torch.full((64, 64), 5.0, dtype=torch.float32, device="cuda")
    for algo in (ci.ALGO_SKINNY,):                       # no fp32 skinny kernel
        h.set_algo(algo)
        with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
            h.gemm_f32(a, a, out=out)
    odd = torch.ones((64, 63), dtype=torch.float32, device="cuda")    # K = 63
    for algo in (ci.ALGO_TILE, ci.ALGO_SMALL):
        h.set_algo(algo)
        with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
            h.gemm_f32(odd, torch.ones((63, 64), device="cuda"), out=out)
    a16 = torch.ones((64, 64), dtype=torch.bfloat16, device="cuda")
    a8 = torch.ones((64, 64), dtype=torch.int8, device="cuda")
    for algo in (ci.ALGO_SKINNY, ci.ALGO_SMALL):         # M = 64 is not a skinny shape
        h.set_algo(algo)
        with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
            h.gemm_bf16(a16, a16)
        with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
            h.gemm_i8_i32(a8, a8)
    torch.cuda.synchronize()
    assert (out.cpu().numpy() == 5.0).all()
    for algo, frag in ((ci.ALGO_GENERIC, "generic"), (ci.ALGO_TILE, "x256x"), (ci.ALGO_DEFAULT, "mfma")):
        h.set_algo(algo)
        c = h.gemm_bf16(a16, a16)
        assert frag in h.last_kernel
        assert (c.float().cpu().numpy() == 64.0).all()
        c = h.gemm_i8_i32(a8, a8)
        assert (c.cpu().numpy() == 64).all()
    h.close()

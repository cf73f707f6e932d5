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

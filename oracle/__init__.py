"""ctypes loader for the CPU oracle (``oracle/oracle.c``).  TEST INFRASTRUCTURE ONLY.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py``
may import this module; the shipped package never does and has no CPU fallback.
All wrappers take and return numpy arrays (C-contiguous unless a leading dimension is
passed explicitly).
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build() -> str:
    """Compile oracle.c with the Makefile beside it and return the library path."""
    subprocess.run(["make", "-C", _HERE, "-B", "liboracle.so"], check=True,
                   stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    lib = C.CDLL(_LIB_PATH)
    i64, u64, f32, vp, ci = C.c_int64, C.c_uint64, C.c_float, C.c_void_p, C.c_int
    sig = {
        "oracle_num_threads": (ci, []),
        "oracle_hash64": (u64, [i64, u64]),
        "oracle_fill_random_f32": (None, [vp, i64, u64, f32, f32]),
        "oracle_fill_random_bf16": (None, [vp, i64, u64, f32, f32]),
        "oracle_fill_random_f16": (None, [vp, i64, u64, f32, f32]),
        "oracle_fill_random_i8": (None, [vp, i64, u64, ci, ci]),
        "oracle_f32_to_bf16": (C.c_uint16, [f32]),
        "oracle_f32_to_f16": (C.c_uint16, [f32]),
        "oracle_bf16_to_f32": (f32, [C.c_uint16]),
        "oracle_f16_to_f32": (f32, [C.c_uint16]),
        "oracle_f32_to_bf16_n": (None, [vp, vp, i64]),
        "oracle_f32_to_f16_n": (None, [vp, vp, i64]),
        "oracle_bf16_to_f32_n": (None, [vp, vp, i64]),
        "oracle_f16_to_f32_n": (None, [vp, vp, i64]),
        "oracle_matrixMulCPU": (None, [vp, vp, vp, ci]),
        "oracle_gemm_f32_ijk": (None, [i64, i64, i64, vp, i64, vp, i64, vp, i64, i64, i64]),
        "oracle_gemm_f32": (None, [i64, i64, i64, vp, i64, vp, i64, vp, i64]),
        "oracle_gemm_f64_rows": (None, [i64, i64, vp, i64, vp, i64, vp, vp, i64, i64, i64]),
        "oracle_gemm_i8_i32": (None, [i64, i64, i64, vp, i64, vp, i64, ci, vp, i64]),
        "oracle_gemm_i8_i64_ijk": (None, [i64, i64, i64, vp, i64, vp, i64, ci, vp, i64]),
        "oracle_dequant_f32": (None, [i64, i64, vp, i64, vp, ci, vp, ci, vp, i64]),
        "oracle_dequant_bf16": (None, [i64, i64, vp, i64, vp, ci, vp, ci, vp, i64]),
        "oracle_quantize_rows_i8": (None, [i64, i64, vp, i64, vp, i64, vp]),
        "oracle_checkResult": (i64, [vp, vp, ci, f32, ci]),
        "oracle_linear_f32": (None, [i64, i64, i64, vp, vp, vp, ci, vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def _p(a: np.ndarray):
    return a.ctypes.data_as(C.c_void_p)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads() -> int:
    return int(lib.oracle_num_threads())


# ---- generators (quantization/GEMM_*.cu fill kernels) --------------------------------
def hash64(idx: int, seed: int) -> int:
    return int(lib.oracle_hash64(idx, seed))


def fill_random_f32(count, seed, lo=-1.0, hi=1.0):
    out = np.empty(count, np.float32)
    lib.oracle_fill_random_f32(_p(out), count, seed, lo, hi)
    return out


def fill_random_bf16(count, seed, lo=-1.0, hi=1.0):
    out = np.empty(count, np.uint16)
    lib.oracle_fill_random_bf16(_p(out), count, seed, lo, hi)
    return out


def fill_random_f16(count, seed, lo=-1.0, hi=1.0):
    out = np.empty(count, np.uint16)
    lib.oracle_fill_random_f16(_p(out), count, seed, lo, hi)
    return out


def fill_random_i8(count, seed, lo=-127, hi=127):
    out = np.empty(count, np.int8)
    lib.oracle_fill_random_i8(_p(out), count, seed, lo, hi)
    return out


# ---- 16-bit conversions -------------------------------------------------------------
def f32_to_bf16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.oracle_f32_to_bf16_n(_p(x), _p(out), x.size)
    return out


def f32_to_f16(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib.oracle_f32_to_f16_n(_p(x), _p(out), x.size)
    return out


def bf16_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.oracle_bf16_to_f32_n(_p(h), _p(out), h.size)
    return out


def f16_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib.oracle_f16_to_f32_n(_p(h), _p(out), h.size)
    return out


# ---- GEMMs ----------------------------------------------------------------------------
def matrixMulCPU(A, B):
    """The reference function itself (square, fp32)."""
    A = _c(A, np.float32)
    B = _c(B, np.float32)
    w = A.shape[0]
    assert A.shape == (w, w) and B.shape == (w, w)
    Cm = np.empty((w, w), np.float32)
    lib.oracle_matrixMulCPU(_p(Cm), _p(A), _p(B), w)
    return Cm


def gemm_f32_ijk(A, B, row0=0, row1=None):
    A = _c(A, np.float32)
    B = _c(B, np.float32)
    M, K = A.shape
    N = B.shape[1]
    row1 = M if row1 is None else row1
    Cm = np.zeros((M, N), np.float32)
    lib.oracle_gemm_f32_ijk(M, N, K, _p(A), K, _p(B), N, _p(Cm), N, row0, row1)
    return Cm


def gemm_f32(A, B):
    A = _c(A, np.float32)
    B = _c(B, np.float32)
    M, K = A.shape
    N = B.shape[1]
    assert B.shape[0] == K
    Cm = np.empty((M, N), np.float32)
    lib.oracle_gemm_f32(M, N, K, _p(A), K, _p(B), N, _p(Cm), N)
    return Cm


def gemm_f64(A, B, rows=None, with_abs=False):
    """fp64 GEMM of float inputs.  ``rows`` = (row0, row1) restricts the output rows."""
    A = _c(A, np.float32)
    B = _c(B, np.float32)
    M, K = A.shape
    N = B.shape[1]
    assert B.shape[0] == K
    r0, r1 = (0, M) if rows is None else rows
    Cm = np.empty((r1 - r0, N), np.float64)
    S = np.empty((r1 - r0, N), np.float64) if with_abs else None
    lib.oracle_gemm_f64_rows(N, K, _p(A), K, _p(B), N, _p(Cm), _p(S) if with_abs else None,
                             N, r0, r1)
    return (Cm, S) if with_abs else Cm


def gemm_i8_i32(A, B, b_is_nk=False):
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, K = A.shape
    N = B.shape[0] if b_is_nk else B.shape[1]
    assert (B.shape[1] if b_is_nk else B.shape[0]) == K
    Cm = np.empty((M, N), np.int32)
    lib.oracle_gemm_i8_i32(M, N, K, _p(A), K, _p(B), B.shape[1], int(b_is_nk), _p(Cm), N)
    return Cm


def gemm_i8_i64_ijk(A, B, b_is_nk=False):
    A = _c(A, np.int8)
    B = _c(B, np.int8)
    M, K = A.shape
    N = B.shape[0] if b_is_nk else B.shape[1]
    Cm = np.empty((M, N), np.int64)
    lib.oracle_gemm_i8_i64_ijk(M, N, K, _p(A), K, _p(B), B.shape[1], int(b_is_nk), _p(Cm), N)
    return Cm


# ---- epilogue / quantizer / compare ---------------------------------------------------
def dequant(acc, sa, sb, out_dtype="f32", sa_per_row=None, sb_per_col=None):
    acc = _c(acc, np.int32)
    M, N = acc.shape
    sa = _c(np.atleast_1d(sa), np.float32)
    sb = _c(np.atleast_1d(sb), np.float32)
    per_row = (sa.size == M and sa.size > 1) if sa_per_row is None else sa_per_row
    per_col = (sb.size == N and sb.size > 1) if sb_per_col is None else sb_per_col
    assert sa.size == (M if per_row else 1) and sb.size == (N if per_col else 1)
    if out_dtype == "f32":
        out = np.empty((M, N), np.float32)
        lib.oracle_dequant_f32(M, N, _p(acc), N, _p(sa), int(per_row), _p(sb), int(per_col),
                               _p(out), N)
    elif out_dtype == "bf16":
        out = np.empty((M, N), np.uint16)
        lib.oracle_dequant_bf16(M, N, _p(acc), N, _p(sa), int(per_row), _p(sb), int(per_col),
                                _p(out), N)
    else:
        raise ValueError(out_dtype)
    return out


def quantize_rows_i8(x):
    x = _c(x, np.float32)
    rows, cols = x.shape
    q = np.empty((rows, cols), np.int8)
    s = np.empty(rows, np.float32)
    lib.oracle_quantize_rows_i8(rows, cols, _p(x), cols, _p(q), cols, _p(s))
    return q, s


def linear_f32(X, W, bias=None, relu=False):
    """MNIST MLP forward layer (MNIST/mnist_nn.cu:10-24, 27-33, 36-49)."""
    X = _c(X, np.float32)
    W = _c(W, np.float32)
    M, K = X.shape
    N = W.shape[1]
    assert W.shape[0] == K
    b = _c(bias, np.float32) if bias is not None else None
    out = np.empty((M, N), np.float32)
    lib.oracle_linear_f32(M, N, K, _p(X), _p(W), _p(b) if b is not None else None, int(relu), _p(out))
    return out


def checkResult(gpu, cpu, eps=1e-5, verbose=False):
    """True when every entry agrees within the absolute ``eps`` (matmulTensor.cu:18-28)."""
    gpu = _c(gpu, np.float32)
    cpu = _c(cpu, np.float32)
    w = gpu.shape[0]
    return lib.oracle_checkResult(_p(gpu), _p(cpu), w, eps, int(verbose)) < 0

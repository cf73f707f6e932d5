"""ctypes binding of ``include/cigemm.h``.

Every GEMM method takes device tensors (``torch.Tensor`` on the GPU), passes their raw
pointers, sizes and strides through the C ABI and returns the output tensor.  Failures of
the library raise :class:`CigemmError` carrying the status name and the handle's message.
"""
from __future__ import annotations

import ctypes as C
import enum
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libcigemm.so")
_SUITE = os.path.join(_HERE, "gemm_suite")

B_KN, B_NK = 0, 1
ACT_NONE, ACT_RELU = 0, 1
ALGO_DEFAULT, ALGO_GENERIC, ALGO_TILE, ALGO_SKINNY, ALGO_SMALL, ALGO_MFMA_ANY = -1, 0, 1, 2, 3, 4
SCALE_TENSOR, SCALE_VECTOR = 0, 1
OUT_F32, OUT_BF16 = 0, 1


class Status(enum.IntEnum):
    SUCCESS = 0
    NOT_INITIALIZED = 1
    ALLOC_FAILED = 3
    INVALID_VALUE = 7
    ARCH_MISMATCH = 8
    MAPPING_ERROR = 11
    EXECUTION_FAILED = 13
    INTERNAL_ERROR = 14
    NOT_SUPPORTED = 15
    LICENSE_ERROR = 16


class CigemmError(RuntimeError):
    def __init__(self, status: int, message: str, where: str):
        self.status = Status(status) if status in Status._value2member_map_ else status
        name = getattr(self.status, "name", str(status))
        super().__init__(f"{where}: CIGEMM_STATUS_{name}" + (f" ({message})" if message else ""))


def library_path() -> str:
    return _LIB


def suite_path() -> str:
    return _SUITE


def build_library(jobs: int = 8) -> str:
    """Compile the HIP sources in ``csrc/`` for gfx950 (works without a GPU)."""
    subprocess.run(["make", "-C", os.path.join(_HERE, "csrc"), f"-j{jobs}", "-B", "all"],
                   check=True)
    return _LIB


_lib = None

# name -> (restype, argtypes); must list every symbol include/cigemm.h declares.
_i64, _u64, _vp, _ci, _f32 = C.c_int64, C.c_uint64, C.c_void_p, C.c_int, C.c_float
SIGNATURES = {
    "cigemmCreate": (_ci, [C.POINTER(_vp)]),
    "cigemmDestroy": (_ci, [_vp]),
    "cigemmSetStream": (_ci, [_vp, _vp]),
    "cigemmGetStream": (_ci, [_vp, C.POINTER(_vp)]),
    "cigemmResetWorkspace": (_ci, [_vp]),
    "cigemmGetStatusString": (C.c_char_p, [_ci]),
    "cigemmGetLastErrorString": (C.c_char_p, [_vp]),
    "cigemmGetVersion": (_ci, []),
    "cigemmGetLastKernelName": (C.c_char_p, [_vp]),
    "cigemmGetLastPlan": (C.c_int, [_vp, C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "cigemm_matrixMulTiled": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int]),
    "cigemm_matrixMulMatrixCores": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int]),
    "cigemm_matrixMulMatrixCoresBfloat16": (C.c_int, [_vp, _vp, _vp, _vp, C.c_int]),
    "cigemmSetAlgo": (C.c_int, [_vp, C.c_int]),
    "cigemmGetAlgo": (C.c_int, [_vp, C.POINTER(C.c_int)]),
    "cigemm_gemm_f32": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "cigemm_gemm_f16": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "cigemm_gemm_bf16": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]),
    "cigemm_gemm_bf16_static": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64,
                                      C.c_char_p, C.c_size_t]),
    "cigemm_gemm_i8_i32": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _ci, _vp, _i64]),
    "cigemm_gemm_i8_dequant": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _ci, _vp, _ci,
                                     _vp, _ci, _vp, _ci, _i64, _vp, _i64]),
    "cigemm_linear_f32": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _ci, _vp, _i64]),
    "cigemm_fill_random_f32": (_ci, [_vp, _vp, _i64, _u64, _f32, _f32]),
    "cigemm_fill_random_bf16": (_ci, [_vp, _vp, _i64, _u64, _f32, _f32]),
    "cigemm_fill_random_f16": (_ci, [_vp, _vp, _i64, _u64, _f32, _f32]),
    "cigemm_fill_random_i8": (_ci, [_vp, _vp, _i64, _u64, _ci, _ci]),
    "cigemm_quantize_rows_i8": (_ci, [_vp, _i64, _i64, _vp, _i64, _vp, _i64, _vp]),
}


def load_library():
    """dlopen ``libcigemm.so`` (built in-tree) and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB):
        raise FileNotFoundError(
            f"{_LIB} is not built; run `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C cudaintro_amd/csrc`.  There is no CPU fallback.")
    lib = C.CDLL(_LIB)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _torch():
    import torch
    return torch


def gemm_bf16_static(A, B, out=None, stream=None):
    """``cigemm_gemm_bf16_static``: the decode-shape bf16 GEMM without a handle and without any
    allocation inside the library (``out`` is allocated here, by torch, when not given)."""
    torch = _torch()
    lib = load_library()
    assert A.dtype == torch.bfloat16 and B.dtype == torch.bfloat16
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    s = torch.cuda.current_stream() if stream is None else stream
    err = C.create_string_buffer(256)
    st = lib.cigemm_gemm_bf16_static(_vp(s.cuda_stream), M, N, K, A.data_ptr(), Handle._ld(A),
                                     B.data_ptr(), Handle._ld(B), out.data_ptr(), Handle._ld(out),
                                     err, len(err))
    if st != 0:
        raise CigemmError(st, err.value.decode(), "cigemm_gemm_bf16_static")
    return out


class Handle:
    """Owns one ``cigemmHandle_t`` bound to the current device and to torch's current stream."""

    def __init__(self, stream=None):
        self.lib = load_library()
        h = _vp()
        st = self.lib.cigemmCreate(C.byref(h))
        if st != 0:
            raise CigemmError(st, "", "cigemmCreate")
        self._h = h
        torch = _torch()
        s = torch.cuda.current_stream() if stream is None else stream
        self.set_stream(s.cuda_stream)

    # -- plumbing ---------------------------------------------------------------------------
    def close(self):
        if getattr(self, "_h", None):
            self.lib.cigemmDestroy(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def _check(self, st, where):
        if st != 0:
            raise CigemmError(st, self.lib.cigemmGetLastErrorString(self._h).decode(), where)

    def set_stream(self, raw_stream: int):
        self._check(self.lib.cigemmSetStream(self._h, _vp(raw_stream)), "cigemmSetStream")

    def reset_workspace(self):
        """Zero the split-K arrival counters and exchange words (after a failure seen elsewhere)."""
        self._check(self.lib.cigemmResetWorkspace(self._h), "cigemmResetWorkspace")

    def set_algo(self, algo: int):
        """Restrict following GEMM calls to one kernel family (``ALGO_*``)."""
        self._check(self.lib.cigemmSetAlgo(self._h, algo), "cigemmSetAlgo")

    def get_algo(self) -> int:
        v = C.c_int(0)
        self._check(self.lib.cigemmGetAlgo(self._h, C.byref(v)), "cigemmGetAlgo")
        return v.value

    def algo(self, algo: int):
        """Context manager: ``with h.algo(ALGO_TILE): ...`` and back to the previous choice."""
        import contextlib

        @contextlib.contextmanager
        def scope():
            prev = self.get_algo()
            self.set_algo(algo)
            try:
                yield self
            finally:
                self.set_algo(prev)

        return scope()

    @property
    def raw(self):
        return self._h

    @property
    def last_kernel(self) -> str:
        return self.lib.cigemmGetLastKernelName(self._h).decode()

    @property
    def last_plan(self):
        """(tile rows, K ranges) of the last GEMM when the LDS-tiled kernel ran, else (0, 0)."""
        rows, splits = C.c_int(0), C.c_int(0)
        self._check(self.lib.cigemmGetLastPlan(self._h, C.byref(rows), C.byref(splits)),
                    "cigemmGetLastPlan")
        return rows.value, splits.value

    # -- GEMMs ------------------------------------------------------------------------------
    @staticmethod
    def _ld(t):
        assert t.dim() == 2 and (t.shape[1] <= 1 or t.stride(1) == 1), "rows must be contiguous"
        return t.stride(0) if t.shape[0] > 1 else max(t.shape[1], t.stride(0), 1)

    def _gemm(self, fn, A, B, out, out_dtype):
        torch = _torch()
        M, K = A.shape
        K2, N = B.shape
        assert K == K2
        if out is None:
            out = torch.empty((M, N), dtype=out_dtype, device=A.device)
        st = getattr(self.lib, fn)(self._h, M, N, K, A.data_ptr(), self._ld(A), B.data_ptr(),
                                   self._ld(B), out.data_ptr(), self._ld(out))
        self._check(st, fn)
        return out

    def gemm_f32(self, A, B, out=None):
        torch = _torch()
        assert A.dtype == torch.float32 and B.dtype == torch.float32
        return self._gemm("cigemm_gemm_f32", A, B, out, torch.float32)

    def linear_f32(self, X, W, bias=None, act=ACT_NONE, out=None):
        """out = act(bias + X @ W) with W stored K x N (input-major)."""
        torch = _torch()
        assert X.dtype == torch.float32 and W.dtype == torch.float32
        M, K = X.shape
        K2, N = W.shape
        assert K == K2 and (bias is None or (bias.dtype == torch.float32 and bias.numel() == N))
        if out is None:
            out = torch.empty((M, N), dtype=torch.float32, device=X.device)
        st = self.lib.cigemm_linear_f32(self._h, M, N, K, X.data_ptr(), self._ld(X), W.data_ptr(),
                                        self._ld(W), bias.data_ptr() if bias is not None else None,
                                        act, out.data_ptr(), self._ld(out))
        self._check(st, "cigemm_linear_f32")
        return out

    def gemm_f16(self, A, B, out=None):
        torch = _torch()
        assert A.dtype == torch.float16 and B.dtype == torch.float16
        return self._gemm("cigemm_gemm_f16", A, B, out, torch.float16)

    # -- study kernels (TileProgramming demo) -------------------------------------------------
    def matrixMulTiled(self, A, B):
        torch = _torch()
        w = A.shape[0]
        assert A.dtype == torch.float32 and A.shape == (w, w) and B.shape == (w, w)
        assert A.is_contiguous() and B.is_contiguous()
        Cm = torch.empty((w, w), dtype=torch.float32, device=A.device)
        st = self.lib.cigemm_matrixMulTiled(self._h, Cm.data_ptr(), A.data_ptr(), B.data_ptr(), w)
        self._check(st, "cigemm_matrixMulTiled")
        return Cm

    def matrixMulMatrixCores(self, A, B):
        """A, B fp16 or bf16 square tensors; fp32 result."""
        torch = _torch()
        w = A.shape[0]
        assert A.dtype == B.dtype and A.dtype in (torch.float16, torch.bfloat16)
        assert A.shape == (w, w) and B.shape == (w, w) and A.is_contiguous() and B.is_contiguous()
        name = ("cigemm_matrixMulMatrixCores" if A.dtype == torch.float16
                else "cigemm_matrixMulMatrixCoresBfloat16")
        Cm = torch.empty((w, w), dtype=torch.float32, device=A.device)
        st = getattr(self.lib, name)(self._h, A.data_ptr(), B.data_ptr(), Cm.data_ptr(), w)
        self._check(st, name)
        return Cm

    def gemm_bf16(self, A, B, out=None):
        torch = _torch()
        assert A.dtype == torch.bfloat16 and B.dtype == torch.bfloat16
        return self._gemm("cigemm_gemm_bf16", A, B, out, torch.bfloat16)

    def gemm_i8_i32(self, A, B, b_layout=B_KN, out=None):
        torch = _torch()
        assert A.dtype == torch.int8 and B.dtype == torch.int8
        M, K = A.shape
        N = B.shape[0] if b_layout == B_NK else B.shape[1]
        assert (B.shape[1] if b_layout == B_NK else B.shape[0]) == K
        if out is None:
            out = torch.empty((M, N), dtype=torch.int32, device=A.device)
        st = self.lib.cigemm_gemm_i8_i32(self._h, M, N, K, A.data_ptr(), self._ld(A),
                                         B.data_ptr(), self._ld(B), b_layout, out.data_ptr(),
                                         self._ld(out))
        self._check(st, "cigemm_gemm_i8_i32")
        return out

    def gemm_i8_dequant(self, A, B, scale_a, scale_b, b_layout=B_KN, out_type=OUT_F32, out=None,
                        dump_acc=False):
        """Returns ``out`` or ``(out, acc)`` when ``dump_acc``.  A scale tensor with one
        element is per-tensor, otherwise per-row (A) / per-column (B)."""
        torch = _torch()
        M, K = A.shape
        N = B.shape[0] if b_layout == B_NK else B.shape[1]
        assert (B.shape[1] if b_layout == B_NK else B.shape[0]) == K
        assert scale_a.dtype == torch.float32 and scale_b.dtype == torch.float32
        assert scale_a.numel() in (1, M) and scale_b.numel() in (1, N)
        ma = SCALE_VECTOR if scale_a.numel() == M and M > 1 else SCALE_TENSOR
        mb = SCALE_VECTOR if scale_b.numel() == N and N > 1 else SCALE_TENSOR
        if out is None:
            out = torch.empty((M, N), device=A.device,
                              dtype=torch.bfloat16 if out_type == OUT_BF16 else torch.float32)
        acc = torch.empty((M, N), dtype=torch.int32, device=A.device) if dump_acc else None
        st = self.lib.cigemm_gemm_i8_dequant(
            self._h, M, N, K, A.data_ptr(), self._ld(A), B.data_ptr(), self._ld(B), b_layout,
            scale_a.data_ptr(), ma, scale_b.data_ptr(), mb, out.data_ptr(), out_type,
            self._ld(out), acc.data_ptr() if dump_acc else None, N if dump_acc else 0)
        self._check(st, "cigemm_gemm_i8_dequant")
        return (out, acc) if dump_acc else out

    # -- generators / quantizer ---------------------------------------------------------------
    def fill_random(self, out, seed, lo=-1.0, hi=1.0):
        torch = _torch()
        name = {torch.float32: "cigemm_fill_random_f32", torch.bfloat16: "cigemm_fill_random_bf16",
                torch.float16: "cigemm_fill_random_f16", torch.int8: "cigemm_fill_random_i8"}[out.dtype]
        if out.dtype == torch.int8:
            lo, hi = int(lo), int(hi)
        assert out.is_contiguous()
        self._check(getattr(self.lib, name)(self._h, out.data_ptr(), out.numel(), seed, lo, hi), name)
        return out

    def quantize_rows_i8(self, x, out=None):
        torch = _torch()
        assert x.dtype == torch.float32 and x.dim() == 2
        rows, cols = x.shape
        if out is None:
            q = torch.empty((rows, cols), dtype=torch.int8, device=x.device)
            s = torch.empty((rows,), dtype=torch.float32, device=x.device)
        else:
            q, s = out
            assert q.dtype == torch.int8 and q.shape == x.shape and s.dtype == torch.float32
        st = self.lib.cigemm_quantize_rows_i8(self._h, rows, cols, x.data_ptr(), self._ld(x),
                                              q.data_ptr(), self._ld(q), s.data_ptr())
        self._check(st, "cigemm_quantize_rows_i8")
        return q, s

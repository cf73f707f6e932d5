"""ctypes binding of ``include/cigemm_probe.h``: the measurement aids in ``libcigemm_probe.so``.

Not part of the drop-in library.  ``bench.py`` and the probe tests load it beside
``libcigemm.so``; every function takes a :class:`cudaintro_amd.Handle`.
"""
from __future__ import annotations

import ctypes as C
import os

from . import cigemm
from .cigemm import OUT_F32, SCALE_TENSOR, SCALE_VECTOR, CigemmError, Handle

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_HERE, "libcigemm_probe.so")
_lib = None

_i64, _vp, _ci = C.c_int64, C.c_void_p, C.c_int
_gemm = [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64]
# name -> (restype, argtypes); must list every symbol include/cigemm_probe.h declares.
SIGNATURES = {
    "cigemm_probe_mfma": (_ci, [_vp, _ci, _ci, _ci, C.POINTER(C.c_int64)]),
    "cigemm_probe_issue_cost": (_ci, [_vp, _ci, _ci, _ci, _ci, _ci, _ci, _ci, _ci, C.POINTER(C.c_double)]),
    "cigemm_probe_tile_phases": (_ci, [_vp, _ci, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _i64,
                                       C.POINTER(C.c_double)]),
    "cigemm_probe_gemm_bf16_paired": (_ci, _gemm),
    "cigemm_probe_gemm_f16_paired": (_ci, _gemm),
    "cigemm_probe_gemm_i8_i32_paired": (_ci, _gemm),
    "cigemm_probe_gemm_i8_dequant_paired": (_ci, [_vp, _i64, _i64, _i64, _vp, _i64, _vp, _i64, _vp, _ci,
                                                  _vp, _ci, _vp, _ci, _i64, _vp, _i64]),
    "cigemm_probe_dirty_workspace": (_ci, [_vp, _ci, C.c_uint32, _ci]),
    "cigemm_probe_force_tile_plan": (_ci, [_vp, _ci, _ci]),
}


def library_path() -> str:
    return _LIB


def load_library():
    global _lib
    if _lib is not None:
        return _lib
    cigemm.load_library()
    if not os.path.exists(_LIB):
        raise FileNotFoundError(f"{_LIB} is not built; run `make -C cudaintro_amd/csrc`")
    lib = C.CDLL(_LIB)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _check(h: Handle, st: int, where: str):
    if st != 0:
        raise CigemmError(st, h.lib.cigemmGetLastErrorString(h.raw).decode(), where)


_KINDS = {"bf16": 0, "f16": 1, "i8": 2, "bf16_16x16": 3, "f16_16x16": 4, "i8_16x16": 5, "f32": 6}


def mfma(h: Handle, kind: str, random_bits: bool, iters: int) -> int:
    """Launch the register-resident matrix-core loop; returns the operations it performs."""
    ops = C.c_int64(0)
    _check(h, load_library().cigemm_probe_mfma(h.raw, _KINDS[kind], int(random_bits), iters, C.byref(ops)),
           "cigemm_probe_mfma")
    return ops.value


def issue_cost(h: Handle, n_dma: int, n_lds_reads: int, barrier: bool, workgroups: int, iters: int,
               placement: int = 0, mfma: bool = True, src_kib_per_wave: int = 8):
    """Cycles per 32-matrix-instruction stage with the given companions; see cigemm_probe.h."""
    res = (C.c_double * 4)()
    _check(h, load_library().cigemm_probe_issue_cost(h.raw, n_dma, n_lds_reads, int(barrier), placement,
                                                     int(mfma), src_kib_per_wave, workgroups, iters, res), "cigemm_probe_issue_cost")
    return dict(zip(("cycles_per_stage", "cycles_per_stage_slowest_wave", "clock_ghz", "launch_us"), list(res)))


PHASE_KEYS = ("prologue_us", "main_loop_us", "epilogue_us", "first_start_to_last_end_us",
              "cycles_per_stage", "main_loop_clock_ghz", "first_epilogue_to_last_end_us", "workgroups",
              "slowest_xcd_clock_ghz", "fastest_xcd_clock_ghz", "mean_unit_end_us", "units")


def tile_phases(h: Handle, A, B, out, paired=False, b_nk=False, same_tile=False):
    """One instrumented launch of the 256-row tile kernel (bf16, fp16 or int8 K x N -> int32), or
    with ``paired`` of its two-workgroups-per-unit form (bf16, int8), or with ``b_nk`` of the
    192-row kernel over int8 N x K weights; the phase figures as a dict."""
    import torch
    if b_nk:
        assert A.dtype == torch.int8 and not paired
        kind = 5
    elif A.dtype == torch.float16:
        assert not paired
        kind = 4
    else:
        kind = {torch.bfloat16: 0, torch.int8: 1}[A.dtype] + (2 if paired else 0)
    if same_tile:
        assert kind in (0, 1, 4)
        kind += 16
    M, K = A.shape
    N = B.shape[0] if b_nk else B.shape[1]
    ph = (C.c_double * 12)()
    st = load_library().cigemm_probe_tile_phases(h.raw, kind, M, N, K, A.data_ptr(), Handle._ld(A),
                                                 B.data_ptr(), Handle._ld(B), out.data_ptr(),
                                                 Handle._ld(out), ph)
    _check(h, st, "cigemm_probe_tile_phases")
    return dict(zip(PHASE_KEYS, list(ph)))


def gemm16_paired(h: Handle, A, B, out=None):
    import torch
    assert A.dtype == B.dtype and A.dtype in (torch.bfloat16, torch.float16)
    name = "cigemm_probe_gemm_bf16_paired" if A.dtype == torch.bfloat16 else "cigemm_probe_gemm_f16_paired"
    M, K = A.shape
    N = B.shape[1]
    if out is None:
        out = torch.empty((M, N), dtype=A.dtype, device=A.device)
    st = getattr(load_library(), name)(h.raw, M, N, K, A.data_ptr(), Handle._ld(A), B.data_ptr(),
                                       Handle._ld(B), out.data_ptr(), Handle._ld(out))
    _check(h, st, name)
    return out


def gemm_i8_i32_paired(h: Handle, A, B, out=None):
    import torch
    M, K = A.shape
    N = B.shape[1]
    if out is None:
        out = torch.empty((M, N), dtype=torch.int32, device=A.device)
    st = load_library().cigemm_probe_gemm_i8_i32_paired(h.raw, M, N, K, A.data_ptr(), Handle._ld(A),
                                                        B.data_ptr(), Handle._ld(B), out.data_ptr(),
                                                        Handle._ld(out))
    _check(h, st, "cigemm_probe_gemm_i8_i32_paired")
    return out


def gemm_i8_dequant_paired(h: Handle, A, B, scale_a, scale_b, out_type=OUT_F32, out=None, dump_acc=False):
    import torch
    M, K = A.shape
    N = B.shape[1]
    ma = SCALE_VECTOR if scale_a.numel() == M and M > 1 else SCALE_TENSOR
    mb = SCALE_VECTOR if scale_b.numel() == N and N > 1 else SCALE_TENSOR
    if out is None:
        out = torch.empty((M, N), device=A.device,
                          dtype=torch.float32 if out_type == OUT_F32 else torch.bfloat16)
    acc = torch.empty((M, N), dtype=torch.int32, device=A.device) if dump_acc else None
    st = load_library().cigemm_probe_gemm_i8_dequant_paired(
        h.raw, M, N, K, A.data_ptr(), Handle._ld(A), B.data_ptr(), Handle._ld(B), scale_a.data_ptr(), ma,
        scale_b.data_ptr(), mb, out.data_ptr(), out_type, Handle._ld(out),
        acc.data_ptr() if dump_acc else None, N if dump_acc else 0)
    _check(h, st, "cigemm_probe_gemm_i8_dequant_paired")
    return (out, acc) if dump_acc else out


def dirty_workspace(h: Handle, count: int, value: int, mark_dirty: bool):
    _check(h, load_library().cigemm_probe_dirty_workspace(h.raw, count, value, int(mark_dirty)),
           "cigemm_probe_dirty_workspace")


def force_tile_plan(h: Handle, tile_rows: int, k_ranges: int = 1):
    """Imposes the tile kernel's plan on the handle's following calls; tile_rows = 0 hands the
    choice back to the library."""
    _check(h, load_library().cigemm_probe_force_tile_plan(h.raw, tile_rows, k_ranges),
           "cigemm_probe_force_tile_plan")

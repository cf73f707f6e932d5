"""Synthetic inputs of the benchmark configurations (host side, numpy).

The reference suite only knows one workload, 4096^3 filled by its hash generator
(quantization/GEMM_*.cu:20-25, 41-46).  The configurations below are the additional
shapes this build is measured on; they are generated on the host with numpy's PCG64 from a
fixed seed so the identical arrays can feed the GPU library and a CPU checker.

Nothing here touches the GPU; callers upload the arrays themselves.
"""
from __future__ import annotations

import numpy as np


def _rng(seed: int) -> np.random.Generator:
    return np.random.Generator(np.random.PCG64(seed))


def f32_to_bf16_bits(x: np.ndarray) -> np.ndarray:
    """Round-to-nearest-even narrowing of finite fp32 values to bfloat16 bit patterns."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def bf16_bits_to_f32(h: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(h, np.uint16).astype(np.uint32) << 16).view(np.float32)


def quantize_rows_absmax(x: np.ndarray):
    """Symmetric per-row int8: s = absmax/127 (1 for a zero row), q = clip(rint(x/s))."""
    x = np.ascontiguousarray(x, np.float32)
    amax = np.abs(x).max(axis=1)
    s = np.where(amax > 0, amax / np.float32(127.0), np.float32(1.0)).astype(np.float32)
    q = np.clip(np.rint(x / s[:, None]), -127, 127).astype(np.int8)
    return q, s


def fp32_uniform(M=512, N=512, K=512, seed=0):
    """fp32 A, B i.i.d. uniform[-1, 1)."""
    r = _rng(seed)
    A = r.uniform(-1.0, 1.0, size=(M, K)).astype(np.float32)
    B = r.uniform(-1.0, 1.0, size=(K, N)).astype(np.float32)
    return A, B


def int8_uniform(M=4096, N=4096, K=4096, seed=1):
    """int8 A (M x K), B (K x N) uniform over the 255 values [-127, 127]; scales 1/127."""
    r = _rng(seed)
    A = r.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = r.integers(-127, 128, size=(K, N), dtype=np.int8)
    s = np.array([1.0 / 127.0], np.float32)
    return A, B, s, s.copy()


def normal_16bit(M=8192, N=8192, K=8192, seed=2, kind="bf16", sigma_b=1.0):
    """N(0,1) A and N(0,sigma_b) B drawn in fp32, rounded to `kind`; returns bit patterns."""
    r = _rng(seed)
    A = r.standard_normal(size=(M, K), dtype=np.float32)
    B = r.standard_normal(size=(K, N), dtype=np.float32)
    if sigma_b != 1.0:
        B *= np.float32(sigma_b)
    if kind == "bf16":
        return f32_to_bf16_bits(A), f32_to_bf16_bits(B)
    if kind == "f16":
        return A.astype(np.float16).view(np.uint16), B.astype(np.float16).view(np.uint16)
    raise ValueError(kind)


def widen_16bit(bits: np.ndarray, kind: str) -> np.ndarray:
    if kind == "bf16":
        return bf16_bits_to_f32(bits)
    return np.ascontiguousarray(bits, np.uint16).view(np.float16).astype(np.float32)


def quantized_linear(M=2048, K=4096, N=11008, seed=3, sigma_w=1.0):
    """Prefill-shaped quantized linear layer: activations X (M x K) ~ N(0,1) with per-row
    absmax scales, weights W (N x K, each output channel contiguous) ~ N(0,sigma_w) with
    per-output-channel absmax scales.  Returns (Xq, sx, Wq, sw)."""
    r = _rng(seed)
    X = r.standard_normal(size=(M, K), dtype=np.float32)
    W = r.standard_normal(size=(N, K), dtype=np.float32)
    if sigma_w != 1.0:
        W *= np.float32(sigma_w)
    Xq, sx = quantize_rows_absmax(X)
    Wq, sw = quantize_rows_absmax(W)
    return Xq, sx, Wq, sw


def skinny_bf16(M, N=8192, K=8192, seed=4):
    """Decode-shaped bf16 GEMM: x (M x K) ~ N(0,1), W (K x N) ~ N(0, 0.02)."""
    return normal_16bit(M, N, K, seed=seed, kind="bf16", sigma_b=0.02)


def skinny_int8(M, N=8192, K=8192, seed=4):
    """Decode-shaped int8 GEMM: weights W (N x K) ~ N(0,0.02) per-channel quantized,
    activations x (M x K) ~ N(0,1) per-row quantized."""
    return quantized_linear(M, K, N, seed=seed, sigma_w=0.02)


# 2*M*N*K operations of one GEMM call.
def gemm_ops(M, N, K) -> float:
    return 2.0 * M * N * K


def skinny_bytes(M, N, K, w_bytes, a_bytes, out_bytes, scale_bytes=0) -> int:
    """Algorithmic HBM bytes of one skinny GEMM: weights + activations + outputs (+ scales)."""
    return K * N * w_bytes + M * K * a_bytes + M * N * out_bytes + scale_bytes

"""int8 GEMM through the C ABI: int32 accumulators bit-exact against the oracle, dequantized
outputs bit-exact against the canonical epilogue."""
import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import workloads as wl
from gpu_util import bits

pytestmark = pytest.mark.gpu


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("b_nk", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1), (2, 3, 7), (17, 33, 65), (129, 65, 33), (64, 64, 4096),
                                   (255, 257, 127), (256, 256, 128), (256, 512, 384), (768, 256, 1024),
                                   (1024, 1024, 1024), (64, 256, 64), (128, 512, 192), (192, 256, 320),
                                   (320, 768, 128), (2048, 2816, 256), (33, 16, 64), (100, 272, 128), (257, 1040, 192),
                                   (20000, 512, 64), (500, 48, 4096)])
def test_accumulators_bit_exact(handle, torch_gpu, oracle, rng, b_nk, shape):
    M, N, K = shape
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(N, K) if b_nk else (K, N), dtype=np.int8)
    C = handle.gemm_i8_i32(dev(torch_gpu, A), dev(torch_gpu, B), ci.B_NK if b_nk else ci.B_KN)
    np.testing.assert_array_equal(C.cpu().numpy(), oracle.gemm_i8_i32(A, B, b_nk))
    if M > 32 and N % 16 == 0 and K % 64 == 0:
        assert "mfma" in handle.last_kernel, handle.last_kernel


@pytest.mark.parametrize("b_nk", [False, True])
def test_extremes_no_overflow(handle, torch_gpu, b_nk):
    M, N, K = 256, 256, 8192
    A = np.full((M, K), 127, np.int8)
    B = np.full((N, K) if b_nk else (K, N), 127, np.int8)
    lay = ci.B_NK if b_nk else ci.B_KN
    C = handle.gemm_i8_i32(dev(torch_gpu, A), dev(torch_gpu, B), lay).cpu().numpy()
    assert (C == 16129 * K).all()
    C = handle.gemm_i8_i32(dev(torch_gpu, -A), dev(torch_gpu, B), lay).cpu().numpy()
    assert (C == -16129 * K).all()


@pytest.mark.parametrize("b_nk", [False, True])
def test_onehot(handle, torch_gpu, rng, b_nk):
    M, N, K = 512, 512, 512
    Bkn = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    perm = rng.integers(0, K, size=M)
    A = np.zeros((M, K), np.int8)
    A[np.arange(M), perm] = 1
    B = np.ascontiguousarray(Bkn.T) if b_nk else Bkn
    C = handle.gemm_i8_i32(dev(torch_gpu, A), dev(torch_gpu, B), ci.B_NK if b_nk else ci.B_KN)
    np.testing.assert_array_equal(C.cpu().numpy(), Bkn[perm].astype(np.int32))


@pytest.mark.parametrize("b_nk", [False, True])
@pytest.mark.parametrize("out_type", ["f32", "bf16"])
@pytest.mark.parametrize("modes", [("tensor", "tensor"), ("row", "col"), ("row", "tensor"), ("tensor", "col")])
@pytest.mark.parametrize("shape", [(256, 256, 256), (33, 65, 129), (512, 768, 640)])
def test_dequant_bit_exact(handle, torch_gpu, oracle, rng, b_nk, out_type, modes, shape):
    M, N, K = shape
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(N, K) if b_nk else (K, N), dtype=np.int8)
    sa = rng.uniform(1e-3, 5e-2, M if modes[0] == "row" else 1).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N if modes[1] == "col" else 1).astype(np.float32)
    out, acc = handle.gemm_i8_dequant(dev(torch_gpu, A), dev(torch_gpu, B), dev(torch_gpu, sa),
                                      dev(torch_gpu, sb), ci.B_NK if b_nk else ci.B_KN,
                                      ci.OUT_BF16 if out_type == "bf16" else ci.OUT_F32, dump_acc=True)
    acc_ref = oracle.gemm_i8_i32(A, B, b_nk)
    np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
    expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=modes[0] == "row",
                            sb_per_col=modes[1] == "col")
    got = bits(torch_gpu, out) if out_type == "bf16" else out.cpu().numpy()
    np.testing.assert_array_equal(got, expect)
    # without the accumulator dump the output is the same
    out2 = handle.gemm_i8_dequant(dev(torch_gpu, A), dev(torch_gpu, B), dev(torch_gpu, sa),
                                  dev(torch_gpu, sb), ci.B_NK if b_nk else ci.B_KN,
                                  ci.OUT_BF16 if out_type == "bf16" else ci.OUT_F32)
    assert torch_gpu.equal(out, out2)


def test_config_int8_4096(handle, torch_gpu, oracle, parity_stats):
    """int8 4096^3, uniform [-127,127] seed 1, per-tensor scales 1/127, fp32 out."""
    A, B, sa, sb = wl.int8_uniform(4096, 4096, 4096, seed=1)
    out, acc = handle.gemm_i8_dequant(dev(torch_gpu, A), dev(torch_gpu, B), dev(torch_gpu, sa),
                                      dev(torch_gpu, sb), ci.B_KN, ci.OUT_F32, dump_acc=True)
    assert "mfma" in handle.last_kernel
    acc_ref = oracle.gemm_i8_i32(A, B)
    np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
    np.testing.assert_array_equal(out.cpu().numpy(), oracle.dequant(acc_ref, sa, sb))
    raw = handle.gemm_i8_i32(dev(torch_gpu, A), dev(torch_gpu, B))
    np.testing.assert_array_equal(raw.cpu().numpy(), acc_ref)
    parity_stats["C2_int8_4096_dequant_f32"] = {"accumulators_bit_exact": True, "outputs_bit_exact": True,
                                               "entries_compared": int(acc_ref.size)}


def test_config_quantized_linear(handle, torch_gpu, oracle, parity_stats):
    """Prefill-shaped quantized linear: M=2048, K=4096, N=11008, per-row x per-channel
    scales, bf16 out."""
    Xq, sx, Wq, sw = wl.quantized_linear(2048, 4096, 11008, seed=3)
    out, acc = handle.gemm_i8_dequant(dev(torch_gpu, Xq), dev(torch_gpu, Wq), dev(torch_gpu, sx),
                                      dev(torch_gpu, sw), ci.B_NK, ci.OUT_BF16, dump_acc=True)
    assert "mfma" in handle.last_kernel
    acc_ref = oracle.gemm_i8_i32(Xq, Wq, b_is_nk=True)
    np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
    np.testing.assert_array_equal(bits(torch_gpu, out), oracle.dequant(acc_ref, sx, sw, out_dtype="bf16"))
    parity_stats["C4_int8_linear_2048x11008x4096_bf16"] = {
        "kernel": handle.last_kernel, "accumulators_bit_exact": True, "outputs_bit_exact": True,
        "entries_compared": int(acc_ref.size)}


def test_quantize_then_gemm_device_pipeline(handle, torch_gpu, oracle, rng):
    """Quantizer and GEMM chained on the device equal the host pipeline."""
    X = rng.normal(size=(256, 512)).astype(np.float32)
    W = rng.normal(size=(768, 512)).astype(np.float32)
    xq, sx = handle.quantize_rows_i8(dev(torch_gpu, X))
    wq, sw = handle.quantize_rows_i8(dev(torch_gpu, W))
    out = handle.gemm_i8_dequant(xq, wq, sx, sw, ci.B_NK, ci.OUT_F32)
    Xq, sxh = oracle.quantize_rows_i8(X)
    Wq, swh = oracle.quantize_rows_i8(W)
    expect = oracle.dequant(oracle.gemm_i8_i32(Xq, Wq, True), sxh, swh)
    np.testing.assert_array_equal(out.cpu().numpy(), expect)
    # and the quantized product approximates the fp32 product
    ref = X.astype(np.float64) @ W.astype(np.float64).T
    assert np.abs(out.cpu().numpy() - ref).max() < 0.05 * np.abs(ref).max()


@pytest.mark.parametrize("b_nk", [False, True])
def test_config_int8_8192(handle, torch_gpu, oracle, b_nk):
    """int8 8192^3 (the headline size), uniform [-127, 127] from seed 1.  The whole result is
    pinned by exact integer identities that touch every element -- Freivalds projections
    C.x = A.(B.x) in int64 and the checksum of checksums sum(C) = colsum(A) . rowsum(B) --
    and a stratified sample of full rows and columns equals the oracle bit for bit."""
    n = 8192
    A, B, _, _ = wl.int8_uniform(n, n, n, seed=1)
    Bs = np.ascontiguousarray(B.T) if b_nk else B           # stored operand
    C = handle.gemm_i8_i32(dev(torch_gpu, A), dev(torch_gpu, Bs), ci.B_NK if b_nk else ci.B_KN)
    assert "mfma" in handle.last_kernel and handle.last_plan == (256, 1)
    C = C.cpu().numpy()
    A64, B64, C64 = A.astype(np.int64), B.astype(np.int64), C.astype(np.int64)
    r = np.random.Generator(np.random.PCG64(11))
    for _ in range(4):
        x = r.integers(-3, 4, size=n).astype(np.int64)
        np.testing.assert_array_equal(C64 @ x, A64 @ (B64 @ x))
        y = r.integers(-3, 4, size=n).astype(np.int64)
        np.testing.assert_array_equal(y @ C64, (y @ A64) @ B64)
    assert int(C.sum(dtype=np.int64)) == int(A64.sum(axis=0) @ B64.sum(axis=1))
    rows = np.array([0, 1, 31, 32, 255, 256, 257, 4095, 4096, 8190, 8191])
    np.testing.assert_array_equal(C[rows], oracle.gemm_i8_i32(np.ascontiguousarray(A[rows]), B, False))
    cols = np.array([0, 3, 4, 127, 128, 255, 256, 4097, 8191])
    np.testing.assert_array_equal(C[:, cols],
                                  oracle.gemm_i8_i32(A, np.ascontiguousarray(B[:, cols]), False))

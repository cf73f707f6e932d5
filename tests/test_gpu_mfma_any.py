"""The any-shape matrix-core kernel (CIGEMM_ALGO_MFMA_ANY): 16-bit and int8 calls with an odd N
or K, leading dimensions and pointers with no alignment beyond the element's, matrices smaller
than a tile.  int8 bit for bit against the CPU loop, 16-bit bit for bit on exact-arithmetic
inputs and within the K-scaled bound on normal ones; the padding around every operand is NaN
(127 for int8) and the output sits inside a sentinel-filled buffer."""
import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import bits, error_bound_16

pytestmark = pytest.mark.gpu

VALS = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
SHAPES = [(1, 1, 1), (3, 5, 7), (64, 63, 64), (129, 131, 67), (300, 257, 1000), (128, 128, 33),
          (17, 1000, 129), (260, 4, 2049),
          # few tiles and a long K: run as K ranges into the workspace plus a reduction launch
          (1, 2047, 2050), (16, 1000, 4097), (130, 257, 3001)]
SPLIT = {(1, 2047, 2050), (16, 1000, 4097), (130, 257, 3001), (260, 4, 2049), (300, 257, 1000)}


def embed(torch, a, dtype, off, pad, fill):
    """`a` placed at element offset `off` of a flat buffer, rows `a.shape[1] + pad` apart."""
    r, c = a.shape
    ld = c + pad
    flat = torch.full((off + r * ld + 3,), fill, dtype=dtype, device="cuda")
    view = flat[off: off + r * ld].view(r, ld)[:, :c]
    src = torch.from_numpy(np.ascontiguousarray(a)).cuda()
    view.copy_(src.view(dtype) if src.dtype != dtype else src)
    return flat, view


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_any_shape_16bit(handle, torch_gpu, oracle, rng, kind, M, N, K):
    torch = torch_gpu
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    tdt = torch.bfloat16 if kind == "bf16" else torch.float16
    npv = np.int16
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    for exact in (True, False):
        if exact:
            Af, Bf = rng.choice(VALS, size=(M, K)), rng.choice(VALS, size=(K, N))
        else:
            Af = rng.standard_normal((M, K)).astype(np.float32)
            Bf = rng.standard_normal((K, N)).astype(np.float32)
        Ab, Bb = narrow(Af), narrow(Bf)
        _, a = embed(torch, Ab.view(npv), tdt, 1, 3, float("nan"))
        _, b = embed(torch, Bb.view(npv), tdt, 3, 1, float("nan"))
        flat, out = embed(torch, np.zeros((M, N), npv), tdt, 1, 5, 0.0)
        flat.fill_(3.0)
        for algo in (ci.ALGO_MFMA_ANY, ci.ALGO_DEFAULT):
            flat.fill_(3.0)
            with handle.algo(algo):
                fn(a, b, out=out)
            assert "mfma_any" in handle.last_kernel, handle.last_kernel
            assert handle.last_kernel.endswith("_splitk") == ((M, N, K) in SPLIT), handle.last_kernel
            got = bits(torch, out)
            if exact:
                np.testing.assert_array_equal(got, narrow(oracle.gemm_f32(widen(Ab), widen(Bb))))
            else:
                ref, S = oracle.gemm_f64(widen(Ab), widen(Bb), with_abs=True)
                err = np.abs(widen(got).astype(np.float64) - ref)
                assert (err <= error_bound_16(ref, S, K, kind)).all()
            f = bits(torch, flat)
            guard = np.ones(f.shape, bool)
            for i in range(M):
                guard[1 + i * (N + 5): 1 + i * (N + 5) + N] = False
            assert (f[guard] == narrow(np.float32(3.0))).all()


@pytest.mark.parametrize("layout", [ci.B_KN, ci.B_NK])
@pytest.mark.parametrize("M,N,K", SHAPES)
def test_any_shape_int8(handle, torch_gpu, oracle, rng, layout, M, N, K):
    torch = torch_gpu
    nk = layout == ci.B_NK
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(N, K) if nk else (K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(A, B, b_is_nk=nk)
    _, a = embed(torch, A, torch.int8, 1, 3, 127)
    _, b = embed(torch, B, torch.int8, 5, 1, 127)
    flat, out = embed(torch, np.zeros((M, N), np.int32), torch.int32, 1, 3, -9)
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    for algo in (ci.ALGO_MFMA_ANY, ci.ALGO_DEFAULT):
        flat.fill_(-9)
        with handle.algo(algo):
            handle.gemm_i8_i32(a, b, layout, out=out)
            assert "mfma_any" in handle.last_kernel, handle.last_kernel
            np.testing.assert_array_equal(out.cpu().numpy(), acc_ref)
            f = flat.cpu().numpy()
            guard = np.ones(f.shape, bool)
            for i in range(M):
                guard[1 + i * (N + 3): 1 + i * (N + 3) + N] = False
            assert (f[guard] == -9).all()
            for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
                y, acc = handle.gemm_i8_dequant(a, b, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                                layout, ot, dump_acc=True)
                assert "mfma_any" in handle.last_kernel and "dequant" in handle.last_kernel
                np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
                expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=True, sb_per_col=True)
                got = bits(torch, y) if out_type == "bf16" else y.cpu().numpy()
                np.testing.assert_array_equal(got, expect)


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_any_shape_f32(handle, torch_gpu, oracle, rng, M, N, K):
    """fp32: within the scaled 1e-5 tolerance of the CPU loop on uniform inputs, bit for bit on
    exact-arithmetic inputs; with and without bias + ReLU."""
    torch = torch_gpu
    for exact in (True, False):
        if exact:
            A, B = rng.choice(VALS, size=(M, K)), rng.choice(VALS, size=(K, N))
        else:
            A = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
            B = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
        bias = rng.choice(VALS, size=N) if exact else rng.uniform(-1, 1, size=N).astype(np.float32)
        _, a = embed(torch, A, torch.float32, 1, 3, float("nan"))
        _, b = embed(torch, B, torch.float32, 3, 1, float("nan"))
        flat, out = embed(torch, np.zeros((M, N), np.float32), torch.float32, 1, 5, 0.0)
        for algo in (ci.ALGO_MFMA_ANY, ci.ALGO_DEFAULT):
            for with_bias in (False, True):
                flat.fill_(3.0)
                with handle.algo(algo):
                    if with_bias:
                        handle.linear_f32(a, b, torch.from_numpy(bias).cuda(), ci.ACT_RELU, out=out)
                        cpu = oracle.linear_f32(A, B, bias, True)
                    else:
                        handle.gemm_f32(a, b, out=out)
                        cpu = oracle.gemm_f32(A, B)
                assert "f32_mfma_any" in handle.last_kernel, handle.last_kernel
                got = out.cpu().numpy()
                if exact:
                    np.testing.assert_array_equal(got, cpu)
                else:
                    plain = oracle.gemm_f32(A, B).astype(np.float64)
                    rms = float(np.sqrt(np.mean(plain ** 2)))
                    lim = 1e-5 * np.maximum(np.abs(plain), rms) + 1e-30
                    assert (np.abs(got.astype(np.float64) - cpu) <= lim).all()
                f = flat.cpu().numpy()
                guard = np.ones(f.shape, bool)
                for i in range(M):
                    guard[1 + i * (N + 5): 1 + i * (N + 5) + N] = False
                assert (f[guard] == 3.0).all()


def test_any_shape_kernel_is_the_fallback_not_the_first_choice(handle, torch_gpu):
    """Aligned shapes keep the LDS-DMA tile kernel and the small fp32 kernel."""
    torch = torch_gpu
    a = torch.zeros((256, 256), dtype=torch.bfloat16, device="cuda")
    handle.gemm_bf16(a, a)
    assert "mfma_any" not in handle.last_kernel and "_mfma_" in handle.last_kernel
    f = torch.zeros((512, 512), dtype=torch.float32, device="cuda")
    handle.gemm_f32(f, f)
    assert "mfma_any" not in handle.last_kernel
    f = torch.zeros((4096, 64), dtype=torch.float32, device="cuda")
    handle.gemm_f32(f, torch.zeros((64, 4096), dtype=torch.float32, device="cuda"))
    assert "x256x16_w" in handle.last_kernel

"""The LDS-tiled matrix-core kernel on shapes that do not fill its units: a K whose last 64-byte
stage is only partly filled (the rest is fetched as zeros, never read from memory) and, for
16-bit types, an N that leaves the last 16-byte piece of a row half inside the matrix.  All
through CIGEMM_ALGO_TILE, so that a call the tile kernel does not take fails instead of falling
to the any-shape kernel.  The operands sit inside larger arrays whose padding is NaN (127 for
int8): anything read from beyond K would poison the result."""
import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import probe
from gpu_util import bits, error_bound_16

pytestmark = pytest.mark.gpu

VALS = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)


def padded(torch, a, dtype, row_pad, col_pad, fill):
    """Device copy of `a` inside a larger array filled with `fill`; returns the view."""
    r, c = a.shape
    big = torch.full((r + row_pad, c + col_pad), fill, dtype=dtype, device="cuda")
    src = torch.from_numpy(np.ascontiguousarray(a))
    if dtype == torch.bfloat16:
        src = src.view(torch.int16).view(torch.bfloat16)
    big[:r, :c] = src.cuda().view(dtype) if src.dtype != dtype else src.cuda()
    return big[:r, :c]


def dev16_padded(torch, b, kind, row_pad, col_pad):
    if kind == "bf16":
        return padded(torch, b.view(np.int16), torch.bfloat16, row_pad, col_pad, float("nan"))
    return padded(torch, b.view(np.float16), torch.float16, row_pad, col_pad, float("nan"))


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M,N", [(256, 256), (100, 264), (513, 1032), (64, 2048)])
@pytest.mark.parametrize("K", [8, 16, 24, 40, 72, 104, 1000, 2048 + 16, 4096 + 24])
def test_k_tail_16bit(handle, torch_gpu, oracle, rng, kind, M, N, K):
    torch = torch_gpu
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    exact = K <= 1000
    if exact:      # exact arithmetic: bit-equal to the CPU loop whatever the summation order
        Af, Bf = rng.choice(VALS, size=(M, K)), rng.choice(VALS, size=(K, N))
    else:
        Af = rng.standard_normal((M, K)).astype(np.float32)
        Bf = rng.standard_normal((K, N)).astype(np.float32)
    Ab, Bb = narrow(Af), narrow(Bf)
    # A: 8 / 24 NaN columns after column K - 1; B: 3 NaN rows after row K - 1
    a = dev16_padded(torch, Ab, kind, 1, 8 if K % 16 else 24)
    b = dev16_padded(torch, Bb, kind, 3, 8)
    out = torch.full((M + 1, N + 8), 3.0, dtype=a.dtype, device="cuda")
    with handle.algo(ci.ALGO_TILE):
        fn(a, b, out=out[:M, :N])
    assert handle.last_plan[0] > 0      # (a long K may run as several K ranges: the last holds the tail)
    o = bits(torch, out)
    if exact:
        np.testing.assert_array_equal(o[:M, :N], narrow(oracle.gemm_f32(widen(Ab), widen(Bb))))
    else:
        ref, S = oracle.gemm_f64(widen(Ab), widen(Bb), with_abs=True)
        err = np.abs(widen(o[:M, :N]).astype(np.float64) - ref)
        assert (err <= error_bound_16(ref, S, K, kind)).all()
    three = narrow(np.float32(3.0))
    assert (o[M:] == three).all() and (o[:, N:] == three).all()


@pytest.mark.parametrize("layout", [ci.B_KN, ci.B_NK])
@pytest.mark.parametrize("M,N", [(256, 256), (100, 272), (300, 1040)])
@pytest.mark.parametrize("K", [16, 32, 48, 80, 144, 208, 1024 + 16, 4096 + 48])
def test_k_tail_int8(handle, torch_gpu, oracle, rng, layout, M, N, K):
    torch = torch_gpu
    nk = layout == ci.B_NK
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(N, K) if nk else (K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(A, B, b_is_nk=nk)
    a = padded(torch, A, torch.int8, 1, 48, 127)
    b = padded(torch, B, torch.int8, 1, 48, 127) if nk else padded(torch, B, torch.int8, 5, 16, 127)
    with handle.algo(ci.ALGO_TILE):
        y = handle.gemm_i8_i32(a, b, layout)
        np.testing.assert_array_equal(y.cpu().numpy(), acc_ref)
        sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
        sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
        out = handle.gemm_i8_dequant(a, b, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                     layout, ci.OUT_BF16)
    np.testing.assert_array_equal(bits(torch, out), oracle.dequant(acc_ref, sa, sb, out_dtype="bf16",
                                                                   sa_per_row=True, sb_per_col=True))


@pytest.mark.parametrize("M,N", [(256, 256), (130, 260)])
@pytest.mark.parametrize("K", [4, 8, 12, 20, 44, 1000 + 4])
def test_k_tail_f32(handle, torch_gpu, oracle, rng, M, N, K):
    torch = torch_gpu
    A, B = rng.choice(VALS, size=(M, K)), rng.choice(VALS, size=(K, N))
    a = padded(torch, A, torch.float32, 1, 12, float("nan"))
    b = padded(torch, B, torch.float32, 2, 4, float("nan"))
    with handle.algo(ci.ALGO_TILE):
        C = handle.gemm_f32(a, b)
    assert "x256x16_w" in handle.last_kernel
    np.testing.assert_array_equal(C.cpu().numpy(), oracle.gemm_f32(A, B))


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M,N,K", [(256, 260, 64), (100, 4, 96), (300, 1028, 1000), (64, 252, 2048 + 8)])
def test_n_half_piece_16bit(handle, torch_gpu, oracle, rng, kind, M, N, K):
    """N % 8 == 4: the last 16-byte piece of a row of B and of C is half inside the matrix.  Rows
    stay 16-byte aligned (leading dimensions are multiples of 8); the 4 columns past N hold NaN
    in B and a sentinel in C."""
    torch = torch_gpu
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    Ab, Bb = narrow(rng.choice(VALS, size=(M, K))), narrow(rng.choice(VALS, size=(K, N)))
    a = dev16_padded(torch, Ab, kind, 0, 8)
    b = dev16_padded(torch, Bb, kind, 1, 4)
    out = torch.full((M + 1, N + 12), 3.0, dtype=a.dtype, device="cuda")
    with handle.algo(ci.ALGO_TILE):
        fn(a, b, out=out[:M, :N])
    o = bits(torch, out)
    np.testing.assert_array_equal(o[:M, :N], narrow(oracle.gemm_f32(widen(Ab), widen(Bb))))
    three = narrow(np.float32(3.0))
    assert (o[M:] == three).all() and (o[:, N:] == three).all()


def test_n_half_piece_int8_bf16_out(handle, torch_gpu, oracle, rng):
    torch = torch_gpu
    M, N, K = 200, 516, 256
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    for layout in (ci.B_KN, ci.B_NK):
        nk = layout == ci.B_NK
        B = rng.integers(-127, 128, size=(N, K) if nk else (K, N), dtype=np.int8)
        acc_ref = oracle.gemm_i8_i32(A, B, b_is_nk=nk)
        sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
        sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
        b = padded(torch, B, torch.int8, 0, 0, 127) if nk else padded(torch, B, torch.int8, 0, 12, 127)
        out = torch.full((M, N + 4), 3.0, dtype=torch.bfloat16, device="cuda")
        with handle.algo(ci.ALGO_TILE):
            handle.gemm_i8_dequant(torch.from_numpy(A).cuda(), b, torch.from_numpy(sa).cuda(),
                                   torch.from_numpy(sb).cuda(), layout, ci.OUT_BF16, out=out[:, :N])
        o = bits(torch, out)
        np.testing.assert_array_equal(o[:, :N], oracle.dequant(acc_ref, sa, sb, out_dtype="bf16",
                                                               sa_per_row=True, sb_per_col=True))
        assert (o[:, N:] == oracle.f32_to_bf16(np.float32(3.0))).all()


def test_tail_shapes_keep_the_tile_kernel_by_default(handle, torch_gpu):
    """What used to fall to the any-shape kernel now stays on the matrix cores."""
    torch = torch_gpu
    a = torch.zeros((512, 1000), dtype=torch.bfloat16, device="cuda")
    b = torch.zeros((1000, 520), dtype=torch.bfloat16, device="cuda")
    handle.gemm_bf16(a, b)
    assert "_mfma_" in handle.last_kernel, handle.last_kernel
    a8 = torch.zeros((512, 1008), dtype=torch.int8, device="cuda")
    b8 = torch.zeros((1008, 512), dtype=torch.int8, device="cuda")
    handle.gemm_i8_i32(a8, b8, ci.B_KN)
    assert "_mfma_" in handle.last_kernel, handle.last_kernel


@pytest.mark.parametrize("rows,ranges", [(64, 2), (128, 3), (192, 5), (256, 7), (128, 16)])
@pytest.mark.parametrize("K", [1000, 2048 + 16, 4096 + 24, 4096 - 40])
def test_k_tail_in_the_last_k_range(handle, torch_gpu, oracle, rng, rows, ranges, K):
    """Split plans imposed on a K with a tail: ranges of an even number of whole stages, the last
    one shorter and ending in a partly filled stage.  Exact inputs: bit-equal to the CPU loop for
    bf16 (K x N), int8 (both layouts) and fp32."""
    torch = torch_gpu
    M, N = 200, 528
    try:
        probe.force_tile_plan(handle, rows, ranges)
        # bf16
        Af, Bf = rng.choice(VALS, size=(M, K)), rng.choice(VALS, size=(K, N))
        Ab, Bb = oracle.f32_to_bf16(Af), oracle.f32_to_bf16(Bf)
        a, b = dev16_padded(torch, Ab, "bf16", 1, 24), dev16_padded(torch, Bb, "bf16", 3, 8)
        out = torch.full((M + 1, N + 8), 3.0, dtype=a.dtype, device="cuda")
        with handle.algo(ci.ALGO_TILE):
            handle.gemm_bf16(a, b, out=out[:M, :N])
        got_rows, got_ranges = handle.last_plan
        assert got_rows == rows and 1 < got_ranges <= ranges, handle.last_plan
        np.testing.assert_array_equal(bits(torch, out)[:M, :N], oracle.f32_to_bf16(
            oracle.gemm_f32(oracle.bf16_to_f32(Ab), oracle.bf16_to_f32(Bb))))
        # fp32 (K in floats: the same byte counts at a quarter of the elements)
        Kf = K // 2
        Af, Bf = rng.choice(VALS, size=(M, Kf)), rng.choice(VALS, size=(Kf, N))
        a, b = padded(torch, Af, torch.float32, 1, 12, float("nan")), padded(torch, Bf, torch.float32, 3, 8, float("nan"))
        with handle.algo(ci.ALGO_TILE):
            c = handle.gemm_f32(a, b)
        assert handle.last_plan[0] == rows and handle.last_plan[1] > 1, handle.last_plan
        np.testing.assert_array_equal(c.cpu().numpy(), oracle.gemm_f32(Af, Bf))
        # int8, both layouts
        for layout in (ci.B_KN, ci.B_NK):
            nk = layout == ci.B_NK
            K8 = 2 * K
            A = rng.integers(-127, 128, size=(M, K8), dtype=np.int8)
            B = rng.integers(-127, 128, size=(N, K8) if nk else (K8, N), dtype=np.int8)
            a = padded(torch, A, torch.int8, 1, 48, 127)
            b = padded(torch, B, torch.int8, 1, 48, 127) if nk else padded(torch, B, torch.int8, 5, 16, 127)
            with handle.algo(ci.ALGO_TILE):
                y = handle.gemm_i8_i32(a, b, layout)
            assert handle.last_plan[0] == rows and handle.last_plan[1] > 1, handle.last_plan
            np.testing.assert_array_equal(y.cpu().numpy(), oracle.gemm_i8_i32(A, B, b_is_nk=nk))
    finally:
        probe.force_tile_plan(handle, 0)

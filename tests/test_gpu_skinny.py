"""Skinny (decode-shape) GEMMs, M <= 32, through the C ABI: the split-K kernels against the
oracle.  int8 accumulators and dequantized outputs bit-exact; 16-bit within the K-scaled bound
and bit-exact on exact-arithmetic inputs; repeated calls (the arrival counters must return to
zero) give identical results."""
import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import workloads as wl
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu


def widen(oracle, b, kind):
    return oracle.bf16_to_f32(b) if kind == "bf16" else oracle.f16_to_f32(b)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M", [1, 2, 8, 17, 32])
@pytest.mark.parametrize("N,K", [(256, 128), (512, 1024), (8192, 8192), (2048, 4096 + 32)])
def test_skinny_16bit(handle, torch_gpu, oracle, kind, M, N, K):
    torch = torch_gpu
    xb, wb = wl.normal_16bit(M, N, K, seed=4, kind=kind, sigma_b=0.02)
    x, w = to_dev(torch, xb, kind), to_dev(torch, wb, kind)
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    y = fn(x, w)
    assert "skinny" in handle.last_kernel, handle.last_kernel
    ref, S = oracle.gemm_f64(widen(oracle, xb, kind), widen(oracle, wb, kind), with_abs=True)
    got = widen(oracle, bits(torch, y), kind).astype(np.float64)
    err = np.abs(got - ref)
    bound = error_bound_16(ref, S, K, kind)
    assert (err <= bound).all(), float((err / bound).max())
    # a second and third call reuse the workspace and counters
    for _ in range(2):
        assert torch.equal(fn(x, w), y)


@pytest.mark.parametrize("kind", ["bf16", "f16"])
def test_skinny_16bit_exact_inputs(handle, torch_gpu, oracle, rng, kind):
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    for (M, N, K) in [(1, 256, 64), (5, 1024, 2048), (32, 8192, 1024)]:
        X = rng.choice(vals, size=(M, K))
        W = rng.choice(vals, size=(K, N))
        fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
        y = fn(to_dev(torch_gpu, narrow(X), kind), to_dev(torch_gpu, narrow(W), kind))
        assert "skinny" in handle.last_kernel
        np.testing.assert_array_equal(bits(torch_gpu, y), narrow(oracle.gemm_f32(X, W)))


@pytest.mark.parametrize("kind", ["bf16"])
def test_skinny_onehot_and_padding_rows(handle, torch_gpu, oracle, rng, kind):
    """Row m of x one-hot at k_m selects row k_m of W; rows >= M of the padded tile are never
    stored (the output buffer has guard rows)."""
    torch = torch_gpu
    M, N, K = 7, 512, 256
    Wf = oracle.bf16_to_f32(oracle.f32_to_bf16(rng.normal(size=(K, N)).astype(np.float32)))
    ks = rng.integers(0, K, size=M)
    X = np.zeros((M, K), np.float32)
    X[np.arange(M), ks] = 1.0
    out = torch.full((M + 4, N), 7.0, dtype=torch.bfloat16, device="cuda")
    handle.gemm_bf16(to_dev(torch, oracle.f32_to_bf16(X), kind), to_dev(torch, oracle.f32_to_bf16(Wf), kind),
                     out=out[:M])
    assert "skinny" in handle.last_kernel
    o = bits(torch, out)
    np.testing.assert_array_equal(o[:M], oracle.f32_to_bf16(Wf[ks]))
    assert (o[M:] == oracle.f32_to_bf16(np.float32(7.0))).all()


@pytest.mark.parametrize("M", [1, 3, 8, 32])
@pytest.mark.parametrize("N,K", [(128, 128), (1024, 512), (8192, 8192), (384, 4096 + 128)])
@pytest.mark.parametrize("out_type", ["i32", "f32", "bf16"])
def test_skinny_int8_nk(handle, torch_gpu, oracle, rng, M, N, K, out_type):
    torch = torch_gpu
    X = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(X, W, b_is_nk=True)
    xd, wd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda()
    if out_type == "i32":
        for _ in range(2):
            y = handle.gemm_i8_i32(xd, wd, ci.B_NK)
            assert "skinny" in handle.last_kernel, handle.last_kernel
            np.testing.assert_array_equal(y.cpu().numpy(), acc_ref)
        return
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    ot = ci.OUT_BF16 if out_type == "bf16" else ci.OUT_F32
    out, acc = handle.gemm_i8_dequant(xd, wd, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                      ci.B_NK, ot, dump_acc=True)
    assert "skinny" in handle.last_kernel, handle.last_kernel
    np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
    expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=M > 1, sb_per_col=True)
    got = bits(torch, out) if out_type == "bf16" else out.cpu().numpy()
    np.testing.assert_array_equal(got, expect)


@pytest.mark.parametrize("M", [1, 5, 8, 9, 16, 17, 32])
@pytest.mark.parametrize("N,K", [(8192, 512), (8192 + 128, 1536), (8192, 4096 + 128), (128, 128), (256, 640),
                                 (32, 256), (8192 + 96, 1024), (160, 16384 + 640),
                                 (2048, 16384 + 384), (256, 16384 + 512), (1024, 32768 + 128),
                                 (11008, 1024),
                                 # few slabs: rows of x in tiles of 8 or 16 with workgroups of their own
                                 (2048, 1536), (4096, 1152), (1024, 2048 + 128)])
def test_skinny_int8_without_split_k(handle, torch_gpu, oracle, rng, M, N, K):
    """The kernel that splits K over the waves of a workgroup instead of over workgroups, with
    8, 16 or 32 rows of x per stage and a last stage of one to four k-chunks.  A few slabs of
    a very long K (the last two shapes) go to the split-K kernel; same bits either way."""
    torch = torch_gpu
    if torch.cuda.get_device_properties(0).multi_processor_count > 256:
        pytest.skip("the shapes assume at most 256 compute units")
    X = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(X, W, b_is_nk=True)
    xd, wd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda()
    expect_kw = N >= 2048 or K <= 16384 or N % 128 != 0
    out = torch.full((M + 2, N + 4), -9, dtype=torch.int32, device="cuda")
    for _ in range(2):
        handle.gemm_i8_i32(xd, wd, ci.B_NK, out=out[:M, :N])
        assert ("kwaves" in handle.last_kernel) == expect_kw, handle.last_kernel
        o = out.cpu().numpy()
        np.testing.assert_array_equal(o[:M, :N], acc_ref)
        assert (o[M:] == -9).all() and (o[:, N:] == -9).all()
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
        y, acc = handle.gemm_i8_dequant(xd, wd, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                        ci.B_NK, ot, dump_acc=True)
        assert ("kwaves" in handle.last_kernel) == expect_kw, handle.last_kernel
        np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
        expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=M > 1, sb_per_col=True)
        got = bits(torch, y) if out_type == "bf16" else y.cpu().numpy()
        np.testing.assert_array_equal(got, expect)


def test_config_skinny_decode(handle, torch_gpu, oracle, parity_stats):
    """The decode-shaped configurations: M in {1, 8, 32}, N = K = 8192, bf16 weights N(0,0.02)
    and int8 weights with per-channel scales."""
    torch = torch_gpu
    for M in (1, 8, 32):
        xb, wb = wl.skinny_bf16(M, 8192, 8192, seed=4)
        y = handle.gemm_bf16(to_dev(torch, xb, "bf16"), to_dev(torch, wb, "bf16"))
        assert "skinny" in handle.last_kernel
        ref, S = oracle.gemm_f64(oracle.bf16_to_f32(xb), oracle.bf16_to_f32(wb), with_abs=True)
        got = oracle.bf16_to_f32(bits(torch, y)).astype(np.float64)
        ratio = np.abs(got - ref) / error_bound_16(ref, S, 8192, "bf16")
        parity_stats[f"C5_skinny_bf16_M{M}"] = {"kernel": handle.last_kernel,
                                                "max_err_over_bound": float(ratio.max()),
                                                "mean_err_over_bound": float(ratio.mean())}
        assert (ratio <= 1.0).all()
        xq, sx, wq, sw = wl.skinny_int8(M, 8192, 8192, seed=4)
        out, acc = handle.gemm_i8_dequant(torch.from_numpy(xq).cuda(), torch.from_numpy(wq).cuda(),
                                          torch.from_numpy(sx).cuda(), torch.from_numpy(sw).cuda(),
                                          ci.B_NK, ci.OUT_BF16, dump_acc=True)
        assert "skinny" in handle.last_kernel
        acc_ref = oracle.gemm_i8_i32(xq, wq, b_is_nk=True)
        np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
        np.testing.assert_array_equal(bits(torch, out),
                                      oracle.dequant(acc_ref, sx, sw, out_dtype="bf16", sa_per_row=M > 1))
        parity_stats[f"C5_skinny_int8_M{M}"] = {"kernel": handle.last_kernel,
                                                "accumulators_bit_exact": True, "outputs_bit_exact": True}


@pytest.mark.parametrize("shape", [(5, 1024, 2048), (8, 8192, 8192)])
def test_skinny_workspace_reuse_with_alternating_inputs(handle, torch_gpu, oracle, rng, shape):
    """The split-K kernel's partials and arrival counters live in the handle's workspace: two
    different problems of one shape called X, Y, X, Y on one handle, each checked against the
    oracle (exact-arithmetic inputs: any summation order gives the same bits).  A stale partial
    or a counter that did not return to zero would show as the other problem's values."""
    torch = torch_gpu
    M, N, K = shape
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    probs = []
    for _ in range(2):
        X, W = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
        # keep |sums| small enough that fp32 partial sums stay exact at K = 8192
        W[rng.random(size=W.shape) < 0.5] = 0
        probs.append((to_dev(torch, oracle.f32_to_bf16(X), "bf16"), to_dev(torch, oracle.f32_to_bf16(W), "bf16"),
                      oracle.f32_to_bf16(oracle.gemm_f32(X, W))))
    assert not np.array_equal(probs[0][2], probs[1][2])
    for i in range(6):
        x, w, want = probs[i & 1]
        y = handle.gemm_bf16(x, w)
        assert "skinny" in handle.last_kernel, handle.last_kernel
        np.testing.assert_array_equal(bits(torch, y), want, err_msg=f"call {i}")


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M,N,K,kernel", [
    (1, 256, 64, "32x64_kwaves"), (3, 512, 1024, "32x64_kwaves"), (32, 2048, 8192, "32x64_kwaves"),
    (32, 256, 3072, "32x64_kwaves"), (16, 8192, 1024, "32x64_kwaves"),
    # large weight matrices (at least 32 slabs of 128 columns, 2048 k, more than 4096 x 4096
    # weights): 128-column slabs
    (8, 8192, 8192, "32x128_kwaves"), (16, 8192, 4096, "32x128_kwaves"), (17, 4096, 8192, "32x128_kwaves"),
    (5, 16384, 2048, "32x128_kwaves"), (32, 8192, 8192, "32x128_kwaves"),
    (17, 4096, 4096, "32x64_kwaves"), (17, 8192, 1024, "32x64_kwaves"), (32, 8192, 2048, "32x64_kwaves"),
    (4, 1024, 4096 + 32, "32x256_ring8"),                                     # K not in whole 64-row stages
    (3, 320, 192, "32x64_kwaves"), (20, 8192 + 64, 128, "32x64_kwaves"),     # N in whole lines, not in 256s
    (32, 16384 + 192, 64, "32x64_kwaves"), (9, 8192 + 64, 4096, "32x64_kwaves"),
    # K ranges that fill the chip once, uneven when the stage count does not divide: 40 slabs x 6
    # ranges of 80 stages (13 or 14 each), 70 slabs x 3 of 25 stages (8 + 8 + 9), 108 slabs x 2
    (3, 5120, 5120, "32x128_kwaves"), (16, 5120, 13824, "32x128_kwaves"), (5, 4480, 1600, "32x64_kwaves"),
    (8, 13824, 5120, "32x128_kwaves"),
    # more workgroups than compute units, two to a unit: 86 slabs x 5 ranges of 64 stages (12 or 13
    # each), 96 x 5, 129 slabs of 64 columns x 3; 172 slabs in one range each
    (8, 11008, 4096, "32x128_kwaves"), (32, 12288, 4096, "32x128_kwaves"), (20, 8192 + 64, 4096, "32x64_kwaves"),
    (2, 22016, 4096, "32x128_kwaves"),
])
def test_skinny_16bit_both_kernels_exact_inputs(handle, torch_gpu, oracle, rng, kind, M, N, K, kernel):
    """The two 16-bit decode kernels (64-column slabs with K over the waves; 256-column slabs with
    K over workgroups): which one the shape gets, and bit-equality with the CPU loop on
    exact-arithmetic inputs, three calls in a row over guard rows."""
    torch = torch_gpu
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    X, W = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
    W[rng.random(size=W.shape) < 0.5] = 0
    want = narrow(oracle.gemm_f32(X, W))
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    out = torch.full((M + 2, N), 7.0, dtype=torch.bfloat16 if kind == "bf16" else torch.float16, device="cuda")
    x, w = to_dev(torch, narrow(X), kind), to_dev(torch, narrow(W), kind)
    for _ in range(3):
        fn(x, w, out=out[:M])
        assert handle.last_kernel == f"{kind}_skinny_{kernel}", handle.last_kernel
        got = bits(torch, out)
        np.testing.assert_array_equal(got[:M], want)
        assert (got[M:] == narrow(np.float32(7.0))).all()


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("M,N,K,forced,expect", [
    # one workgroup on every compute unit: 32 slabs x 8 ranges, 64 x 4 (counter exchange), 128 x 2
    # (exchange words), 256 x 1 -> the decode kernel with two tiles of x
    (33, 4096, 4096, False, "64x128_kwaves"), (64, 8192, 4096, False, "64x128_kwaves"),
    (47, 16384, 2048, False, "64x128_kwaves"), (64, 32768, 2048, False, "64x128_kwaves"),
    # any other grid: the tile kernel, unless the family is forced
    (40, 11008, 4096, False, None), (64, 5120, 5120, False, None),
    (40, 11008, 4096, True, "64x128_kwaves"), (64, 5120, 5120, True, "64x128_kwaves"),
    (33, 13824, 2048, True, "64x128_kwaves"),
])
def test_skinny_16bit_two_tiles_of_x(handle, torch_gpu, oracle, rng, kind, M, N, K, forced, expect):
    """33 to 64 rows of x: the K-over-the-waves kernel with two 32-row tiles per wave where its
    grid is exactly one workgroup per compute unit (or when forced), bit-equal to the CPU loop on
    exact-arithmetic inputs, three calls in a row over guard rows."""
    torch = torch_gpu
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("the shapes assume 256 compute units")
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    X, W = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
    W[rng.random(size=W.shape) < 0.5] = 0
    W[:, 128:256] = 0                      # a slab of zero sums (the exchange words' empty state)
    want = narrow(oracle.gemm_f32(X, W))
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    out = torch.full((M + 2, N), 7.0, dtype=torch.bfloat16 if kind == "bf16" else torch.float16, device="cuda")
    x, w = to_dev(torch, narrow(X), kind), to_dev(torch, narrow(W), kind)
    with handle.algo(ci.ALGO_SKINNY if forced else ci.ALGO_DEFAULT):
        for _ in range(3):
            fn(x, w, out=out[:M])
            if expect:
                assert handle.last_kernel == f"{kind}_skinny_{expect}", handle.last_kernel
            else:
                assert "skinny" not in handle.last_kernel, handle.last_kernel
            got = bits(torch, out)
            np.testing.assert_array_equal(got[:M], want)
            assert (got[M:] == narrow(np.float32(7.0))).all()


@pytest.mark.parametrize("M,N,K,forced", [(33, 8192, 8192, False), (64, 16384, 4096, False),
                                          (50, 4096, 11008, False), (64, 11008, 4096, True),
                                          (48, 4096, 2048, True)])
def test_skinny_int8_kn_two_tiles_of_x(handle, torch_gpu, oracle, rng, M, N, K, forced):
    """int8 K x N weights with 33 to 64 rows of x: raw accumulators and both dequantized output
    types, bit for bit."""
    torch = torch_gpu
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("the shapes assume 256 compute units")
    X = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    W = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(X, W, b_is_nk=False)
    xd, wd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda()
    out = torch.full((M + 2, N + 4), -9, dtype=torch.int32, device="cuda")
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    with handle.algo(ci.ALGO_SKINNY if forced else ci.ALGO_DEFAULT):
        for _ in range(2):
            handle.gemm_i8_i32(xd, wd, ci.B_KN, out=out[:M, :N])
            assert handle.last_kernel == "i8_skinny_64x128_kwaves_kn", handle.last_kernel
            o = out.cpu().numpy()
            np.testing.assert_array_equal(o[:M, :N], acc_ref)
            assert (o[M:] == -9).all() and (o[:, N:] == -9).all()
        for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
            y, acc = handle.gemm_i8_dequant(xd, wd, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                            ci.B_KN, ot, dump_acc=True)
            assert handle.last_kernel == "i8_skinny_64x128_kwaves_kn_dequant", handle.last_kernel
            np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
            expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=True, sb_per_col=True)
            got = bits(torch, y) if out_type == "bf16" else y.cpu().numpy()
            np.testing.assert_array_equal(got, expect)


@pytest.mark.parametrize("N,K,kernel", [(16384, 4096, "32x128"), (8192 - 64, 1024, "32x64")])
@pytest.mark.parametrize("zero_part", ["all", "first_range", "second_range", "columns"])
def test_two_range_exchange_with_zero_partial_sums(handle, torch_gpu, oracle, rng, zero_part, N, K, kernel):
    """128 slabs of 128 columns over 64 stages, or 127 slabs of 64 columns over 16 stages, get two
    K ranges each, which meet through one atomic exchange per pair of outputs; a pair of +0.0 partial sums
    looks like the exchange word's empty state and travels as -0.0.  Weights that are zero over a
    whole K range, over everything, or in some columns give such pairs; the results must equal
    the CPU loop's bits (+0.0 where the sum is zero), three calls in a row (every word returns to
    empty)."""
    torch = torch_gpu
    M = 3
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    X, W = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
    W[rng.random(size=W.shape) < 0.5] = 0
    if zero_part == "all":
        W[:] = 0
    elif zero_part == "first_range":
        W[:K // 2] = 0
    elif zero_part == "second_range":
        W[K // 2:] = 0
    else:
        W[:, ::3] = 0
        W[:, 1000:1100] = 0
    want = oracle.f32_to_bf16(oracle.gemm_f32(X, W))
    x, w = to_dev(torch, oracle.f32_to_bf16(X), "bf16"), to_dev(torch, oracle.f32_to_bf16(W), "bf16")
    for _ in range(3):
        y = handle.gemm_bf16(x, w)
        assert handle.last_kernel == f"bf16_skinny_{kernel}_kwaves", handle.last_kernel
        np.testing.assert_array_equal(bits(torch, y), want)


@pytest.mark.parametrize("M", [1, 5, 8, 16, 17, 32])
@pytest.mark.parametrize("N,K", [(128, 128), (1024, 512), (8192, 8192), (256, 4096 + 128), (2048, 1024),
                                 (8192 + 128, 1024 + 128)])
def test_skinny_int8_kn(handle, torch_gpu, oracle, rng, M, N, K):
    """int8 K x N weights at M <= 32: the K-over-the-waves kernel with 128-column slabs, one to
    sixteen K ranges per slab; raw accumulators (into a guarded buffer, twice) and both
    dequantized output types, bit for bit."""
    torch = torch_gpu
    X = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    W = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(X, W, b_is_nk=False)
    xd, wd = torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda()
    out = torch.full((M + 2, N + 4), -9, dtype=torch.int32, device="cuda")
    for _ in range(2):
        handle.gemm_i8_i32(xd, wd, ci.B_KN, out=out[:M, :N])
        assert handle.last_kernel == "i8_skinny_32x128_kwaves_kn", handle.last_kernel
        o = out.cpu().numpy()
        np.testing.assert_array_equal(o[:M, :N], acc_ref)
        assert (o[M:] == -9).all() and (o[:, N:] == -9).all()
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
        y, acc = handle.gemm_i8_dequant(xd, wd, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                        ci.B_KN, ot, dump_acc=True)
        assert handle.last_kernel == "i8_skinny_32x128_kwaves_kn_dequant", handle.last_kernel
        np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
        expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=M > 1, sb_per_col=True)
        got = bits(torch, y) if out_type == "bf16" else y.cpu().numpy()
        np.testing.assert_array_equal(got, expect)

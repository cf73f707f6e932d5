"""Seeded random shapes, leading dimensions and pointer offsets through every GEMM entry point
(default kernel choice), each result checked against the oracle: int8 bit for bit, fp32 within
the scaled 1e-5 tolerance of the CPU loop, fp16/bf16 within the accumulation bound of fp64."""
import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu

SEEN = set()   # kernel families the random cases reached (checked by the last test)
ALGOS = (ci.ALGO_DEFAULT, ci.ALGO_GENERIC, ci.ALGO_TILE, ci.ALGO_SMALL, ci.ALGO_SKINNY, ci.ALGO_MFMA_ANY)


def each_family(handle, call):
    """Run `call()` under every kernel family that takes it; yields after each successful run."""
    ran = 0
    for algo in ALGOS:
        with handle.algo(algo):
            try:
                call()
            except ci.CigemmError as e:
                assert "NOT_SUPPORTED" in str(e), str(e)
                assert algo not in (ci.ALGO_DEFAULT, ci.ALGO_GENERIC)
                continue
        SEEN.add(handle.last_kernel)
        ran += 1
        yield algo
    assert ran >= 2


def draw_dim(r, big):
    kind = r.integers(0, 5)
    if kind == 0:
        return int(r.integers(1, 40))
    if kind == 1:
        return int(r.choice([32, 64, 128, 256, 512]))
    if kind == 2:
        return int(r.choice([4, 8, 16, 48, 96, 260, 264, 320]))
    return int(r.integers(1, big))


def cases(seed, n, big_mn=420, big_k=900):
    """Half of the cases are arbitrary; the other half keep every size, padding and offset a
    multiple of 64 elements so that the aligned (MFMA) families take them."""
    r = np.random.Generator(np.random.PCG64(seed))
    out = []
    for i in range(n):
        if i % 2:
            M = int(r.choice([int(r.integers(1, big_mn)), int(r.integers(1, 33)), int(r.integers(1, 33)), 32, 64, 256, 300]))
            N = int(r.choice([128, 256, 256, 384, 512, int(r.integers(1, 7)) * 64]))
            K = int(r.integers(1, 13)) * 64
            pads = tuple(int(r.choice([0, 64, 128])) for _ in range(3))
            offs = tuple(int(r.choice([0, 64])) for _ in range(3))
        else:
            M, N, K = draw_dim(r, big_mn), draw_dim(r, big_mn), draw_dim(r, big_k)
            pads = tuple(int(r.choice([0, 0, 1, 4, 8, 16])) for _ in range(3))
            offs = tuple(int(r.choice([0, 0, 0, 1, 4, 16])) for _ in range(3))
        out.append((M, N, K, pads, offs))
    return out


def place(torch, a, pad, off, kind=None):
    """Copy `a` into a larger device buffer: row stride cols + pad, first element at `off`."""
    rows, cols = a.shape
    ld = cols + pad
    flat = np.zeros(off + rows * ld + 8, a.dtype)
    view = np.lib.stride_tricks.as_strided(flat[off:], shape=(rows, cols),
                                           strides=(ld * a.itemsize, a.itemsize))
    view[...] = a
    d = to_dev(torch, flat, kind)
    return d[off:off + rows * ld].view(rows, ld)[:, :cols] if pad else d[off:off + rows * cols].view(rows, cols)


def out_buffer(torch, rows, cols, pad, off, dtype, fill):
    ld = cols + pad
    flat = torch.full((off + rows * ld + 8,), fill, dtype=dtype, device="cuda")
    body = flat[off:off + rows * ld].view(rows, ld)
    return flat, body[:, :cols]


@pytest.mark.parametrize("case", cases(101, 60), ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}")
def test_random_f32(handle, torch_gpu, oracle, case):
    torch = torch_gpu
    M, N, K, pads, offs = case
    r = np.random.Generator(np.random.PCG64(M * 7919 + N * 104729 + K))
    A = r.uniform(-1, 1, size=(M, K)).astype(np.float32)
    B = r.uniform(-1, 1, size=(K, N)).astype(np.float32)
    a, b = place(torch, A, pads[0], offs[0]), place(torch, B, pads[1], offs[1])
    cpu = oracle.gemm_f32(A, B)
    rms = float(np.sqrt(np.mean(cpu.astype(np.float64) ** 2)))
    lim = 1e-5 * np.maximum(np.abs(cpu.astype(np.float64)), rms) + 1e-30
    ld = N + pads[2]
    box = {}

    def call():
        box["flat"], box["C"] = out_buffer(torch, M, N, pads[2], offs[2], torch.float32, -3.0)
        handle.gemm_f32(a, b, out=box["C"])
    for _ in each_family(handle, call):
        got = box["C"].cpu().numpy().astype(np.float64)
        assert (np.abs(got - cpu) <= lim).all(), handle.last_kernel
        f = box["flat"].cpu().numpy()
        guard = np.ones(f.shape, bool)
        for i in range(M):
            guard[offs[2] + i * ld: offs[2] + i * ld + N] = False
        assert (f[guard] == -3.0).all(), handle.last_kernel    # nothing outside C was written


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("case", cases(202, 40), ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}")
def test_random_16bit(handle, torch_gpu, oracle, kind, case):
    torch = torch_gpu
    M, N, K, pads, offs = case
    r = np.random.Generator(np.random.PCG64(M * 31 + N * 17 + K))
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    Ab = narrow(r.standard_normal((M, K)).astype(np.float32))
    Bb = narrow(r.standard_normal((K, N)).astype(np.float32))
    dt = torch.bfloat16 if kind == "bf16" else torch.float16
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    a, b = place(torch, Ab, pads[0], offs[0], kind), place(torch, Bb, pads[1], offs[1], kind)
    ref, S = oracle.gemm_f64(widen(Ab), widen(Bb), with_abs=True)
    ld = N + pads[2]
    box = {}

    def call():
        box["flat"], box["C"] = out_buffer(torch, M, N, pads[2], offs[2], dt, 7.0)
        fn(a, b, out=box["C"])
    for _ in each_family(handle, call):
        got = widen(bits(torch, box["C"])).astype(np.float64)
        assert (np.abs(got - ref) <= error_bound_16(ref, S, K, kind)).all(), handle.last_kernel
        f = widen(bits(torch, box["flat"]))
        guard = np.ones(f.shape, bool)
        for i in range(M):
            guard[offs[2] + i * ld: offs[2] + i * ld + N] = False
        assert (f[guard] == 7.0).all(), handle.last_kernel


@pytest.mark.parametrize("layout", [ci.B_KN, ci.B_NK])
@pytest.mark.parametrize("case", cases(303, 40), ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}")
def test_random_int8(handle, torch_gpu, oracle, layout, case):
    torch = torch_gpu
    M, N, K, pads, offs = case
    r = np.random.Generator(np.random.PCG64(M * 13 + N * 11 + K * 5 + layout))
    A = r.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = r.integers(-127, 128, size=(N, K) if layout == ci.B_NK else (K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(A, B, b_is_nk=layout == ci.B_NK)
    a, b = place(torch, A, pads[0], offs[0]), place(torch, B, pads[1], offs[1])
    ld = N + pads[2]
    box = {}

    def call():
        box["flat"], box["C"] = out_buffer(torch, M, N, pads[2], offs[2], torch.int32, -9)
        handle.gemm_i8_i32(a, b, layout, out=box["C"])
    for _ in each_family(handle, call):
        np.testing.assert_array_equal(box["C"].cpu().numpy(), acc_ref, err_msg=handle.last_kernel)
        f = box["flat"].cpu().numpy()
        guard = np.ones(f.shape, bool)
        for i in range(M):
            guard[offs[2] + i * ld: offs[2] + i * ld + N] = False
        assert (f[guard] == -9).all(), handle.last_kernel
    # dequantizing entry point on the same operands: per-row x per-column scales, both outputs
    sa = r.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = r.uniform(1e-3, 5e-2, N).astype(np.float32)
    sad, sbd = torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda()
    for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
        expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=True,
                                sb_per_col=True)

        def call_dq():
            box["out"], box["acc"] = handle.gemm_i8_dequant(a, b, sad, sbd, layout, ot,
                                                            dump_acc=True)
        for _ in each_family(handle, call_dq):
            np.testing.assert_array_equal(box["acc"].cpu().numpy(), acc_ref,
                                          err_msg=handle.last_kernel)
            got = bits(torch, box["out"]) if out_type == "bf16" else box["out"].cpu().numpy()
            np.testing.assert_array_equal(got, expect, err_msg=handle.last_kernel)


SPLIT_PLANS = set()   # (tile rows, K ranges) the long-K cases below ran as


def long_k_cases(seed, n):
    """Batch sizes between the decode kernels' and a full round of tiles, with a K long enough
    for the tile kernel to cut it into ranges: any count of ranges, the last one shorter, and a
    K that ends inside a 64-byte stage."""
    r = np.random.Generator(np.random.PCG64(seed))
    out = []
    for _ in range(n):
        M = int(r.integers(33, 420))
        N = int(r.integers(2, 80)) * 16
        K = int(r.integers(64, 560)) * 16 + int(r.choice([0, 0, 16, 32, 48]))
        out.append((M, N, K))
    return out


@pytest.mark.parametrize("case", long_k_cases(404, 36), ids=lambda c: f"{c[0]}x{c[1]}x{c[2]}")
def test_random_long_k_split_plans(handle, torch_gpu, oracle, case):
    """Exact-arithmetic inputs: bit for bit the CPU loop whatever plan the library takes, for
    bf16, fp32 (a quarter of the k) and int8 in both layouts."""
    torch = torch_gpu
    M, N, K = case
    r = np.random.Generator(np.random.PCG64(M * 1000003 + N * 1009 + K))
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    A, B = r.choice(vals, size=(M, K)), r.choice(vals, size=(K, N))
    out = handle.gemm_bf16(to_dev(torch, oracle.f32_to_bf16(A), "bf16"), to_dev(torch, oracle.f32_to_bf16(B), "bf16"))
    SPLIT_PLANS.add(handle.last_plan)
    np.testing.assert_array_equal(bits(torch, out), oracle.f32_to_bf16(oracle.gemm_f32(A, B)),
                                  err_msg=f"{handle.last_kernel} {handle.last_plan}")
    Kf = K // 4 * 4 // 2
    Kf -= Kf % 4
    Af, Bf = r.choice(vals, size=(M, Kf)), r.choice(vals, size=(Kf, N))
    c = handle.gemm_f32(torch.from_numpy(Af).cuda(), torch.from_numpy(Bf).cuda())
    SPLIT_PLANS.add(handle.last_plan)
    np.testing.assert_array_equal(c.cpu().numpy(), oracle.gemm_f32(Af, Bf),
                                  err_msg=f"{handle.last_kernel} {handle.last_plan}")
    A8 = r.integers(-127, 128, size=(M, K), dtype=np.int8)
    for nk in (False, True):
        B8 = r.integers(-127, 128, size=(N, K) if nk else (K, N), dtype=np.int8)
        y = handle.gemm_i8_i32(torch.from_numpy(A8).cuda(), torch.from_numpy(B8).cuda(), ci.B_NK if nk else ci.B_KN)
        SPLIT_PLANS.add(handle.last_plan)
        np.testing.assert_array_equal(y.cpu().numpy(), oracle.gemm_i8_i32(A8, B8, b_is_nk=nk),
                                      err_msg=f"{handle.last_kernel} {handle.last_plan}")


def test_random_long_k_cases_reach_uneven_splits():
    """... and only if the library did cut K: several different counts of ranges, odd ones too,
    on several tile heights."""
    ranges = {p[1] for p in SPLIT_PLANS if p[0] > 0}
    rows = {p[0] for p in SPLIT_PLANS if p[1] > 1}
    assert len(ranges) >= 6 and any(s > 1 and s % 2 for s in ranges), sorted(SPLIT_PLANS)
    assert len(rows) >= 2, sorted(SPLIT_PLANS)


def test_random_cases_reach_every_family():
    """The draws above are only worth something if they exercise the fast paths too."""
    for frag in ("f32_generic", "f32_mfma_small", "x256x16_w", "bf16_generic", "bf16_mfma_",
                 "f16_mfma_", "i8_generic", "_ring4_kn", "_ring4_nk", "dequant", "bf16_skinny",
                 "f16_skinny",
                 "i8_skinny_32x32_kwaves_nk", "i8_skinny_32x32_kwaves_nk_dequant"):
        assert any(frag in k for k in SEEN), (frag, sorted(SEEN))

"""fp16 / bf16 GEMM through the C ABI: exact cases against the oracle bit for bit, random
cases against the fp64 oracle within the K-scaled bound."""
import numpy as np
import pytest

from cudaintro_amd import workloads as wl
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu
KINDS = ["bf16", "f16"]


def narrow(oracle, x, kind):
    return oracle.f32_to_bf16(x) if kind == "bf16" else oracle.f32_to_f16(x)


def widen(oracle, b, kind):
    return oracle.bf16_to_f32(b) if kind == "bf16" else oracle.f16_to_f32(b)


def run(handle, torch, Ab, Bb, kind):
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    return bits(torch, fn(to_dev(torch, Ab, kind), to_dev(torch, Bb, kind)))


def check_bound(oracle, Cb, Ab, Bb, kind, rows=None, stats=None):
    """Asserts the K-scaled bound on the given rows; returns the worst error in units of it.
    `stats` (a list) also receives every error/bound ratio of the rows."""
    A, B = widen(oracle, Ab, kind), widen(oracle, Bb, kind)
    K = A.shape[1]
    ref, S = oracle.gemm_f64(A, B, rows=rows, with_abs=True)
    got = widen(oracle, Cb, kind).astype(np.float64)
    if rows is not None:
        got = got[rows[0]:rows[1]]
    assert np.isfinite(got).all()
    err = np.abs(got - ref)
    bound = error_bound_16(ref, S, K, kind)
    worst = float((err / bound).max())
    if stats is not None:
        stats.append((err / bound).ravel())
    assert worst <= 1.0, f"error {worst:.3f} x bound"
    return worst


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(256, 256, 64), (256, 256, 128), (512, 256, 192), (256, 768, 1024),
                                   (1024, 1024, 1024), (64, 256, 32), (128, 512, 96), (192, 256, 160),
                                   (320, 1024, 64), (2048, 2816, 128)])
def test_exact_inputs_bit_exact_mfma(handle, torch_gpu, oracle, rng, kind, shape):
    """Inputs from {0, +-0.5, +-1, +-2}: every partial sum is exact in fp32, so the result
    does not depend on summation order and must equal the CPU loop bit for bit."""
    M, N, K = shape
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    A = rng.choice(vals, size=(M, K))
    B = rng.choice(vals, size=(K, N))
    Cb = run(handle, torch_gpu, narrow(oracle, A, kind), narrow(oracle, B, kind), kind)
    assert "mfma" in handle.last_kernel
    expect = narrow(oracle, oracle.gemm_f32(A, B), kind)
    np.testing.assert_array_equal(Cb, expect)


@pytest.mark.parametrize("kind", KINDS)
def test_onehot_selects_rows_and_columns(handle, torch_gpu, oracle, rng, kind):
    """A one-hot A row picks a row of B, a one-hot B column picks a column of A: every
    position of the 256x256x64 tiling is exercised by scattering the ones."""
    M = N = 512
    K = 256
    Bf = widen(oracle, narrow(oracle, rng.normal(size=(K, N)).astype(np.float32), kind), kind)
    perm = rng.integers(0, K, size=M)
    A = np.zeros((M, K), np.float32)
    A[np.arange(M), perm] = 1.0
    Cb = run(handle, torch_gpu, narrow(oracle, A, kind), narrow(oracle, Bf, kind), kind)
    np.testing.assert_array_equal(Cb, narrow(oracle, Bf[perm], kind))
    Af = widen(oracle, narrow(oracle, rng.normal(size=(M, K)).astype(np.float32), kind), kind)
    permn = rng.integers(0, K, size=N)
    B = np.zeros((K, N), np.float32)
    B[permn, np.arange(N)] = 1.0
    Cb = run(handle, torch_gpu, narrow(oracle, Af, kind), narrow(oracle, B, kind), kind)
    np.testing.assert_array_equal(Cb, narrow(oracle, Af[:, permn], kind))


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(256, 256, 512), (512, 768, 2048), (1, 1, 1), (3, 7, 17), (33, 65, 129),
                                   (129, 17, 65), (255, 257, 63), (64, 64, 4096), (33, 8, 32), (100, 264, 96),
                                   (257, 1032, 160), (5000, 520, 64), (333, 40, 2048)])
def test_random_within_bound(handle, torch_gpu, oracle, kind, shape):
    M, N, K = shape
    Ab, Bb = wl.normal_16bit(M, N, K, seed=7, kind=kind)
    Cb = run(handle, torch_gpu, Ab, Bb, kind)
    if M > 32 and N % 8 == 0 and K % 32 == 0:
        assert "mfma" in handle.last_kernel, handle.last_kernel
    check_bound(oracle, Cb, Ab, Bb, kind)


@pytest.mark.parametrize("kind", KINDS)
def test_leading_dimensions(handle, torch_gpu, oracle, rng, kind):
    torch = torch_gpu
    M, N, K = 256, 512, 320
    Ab, Bb = wl.normal_16bit(M + 5, N + 24, K + 72, seed=9, kind=kind)
    bigA, bigB = to_dev(torch, Ab, kind), to_dev(torch, Bb, kind)
    a = bigA[:M, 8:8 + K]           # lda = K + 72
    b = bigB[:K, 16:16 + N]         # ldb = N + 24
    out = torch.zeros((M, N + 16), dtype=bigA.dtype, device="cuda")
    c = out[:, 8:8 + N]
    (handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16)(a, b, out=c)
    assert "mfma" in handle.last_kernel
    check_bound(oracle, bits(torch, c), bits(torch, a), bits(torch, b), kind)
    o = bits(torch, out)
    assert (o[:, :8] == 0).all() and (o[:, 8 + N:] == 0).all()
    # an output whose rows are only 8-byte aligned is still served (by the any-shape kernel)
    out2 = torch.zeros((M, N + 8), dtype=bigA.dtype, device="cuda")
    c2 = out2[:, 4:4 + N]
    (handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16)(a, b, out=c2)
    check_bound(oracle, bits(torch, c2), bits(torch, a), bits(torch, b), kind)


@pytest.mark.parametrize("kind", KINDS)
def test_linearity_in_a_large(handle, torch_gpu, oracle, kind):
    """Size-independent property at a large size: scaling A by 2 scales C by exactly 2
    (power-of-two scaling commutes with every rounding when nothing overflows and the result
    is a normal number: entries in fp16's subnormal range are left out)."""
    torch = torch_gpu
    Ab, Bb = wl.normal_16bit(2048, 2048, 2048, seed=11, kind=kind)
    A = to_dev(torch, Ab, kind)
    B = to_dev(torch, Bb, kind)
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    C1 = fn(A, B)
    C2 = fn(A * 2, B)
    normal = C1.abs() >= 2.0 ** -13
    assert normal.float().mean() > 0.999
    assert torch.equal((C1 * 2)[normal], C2[normal])
    # and a sample of rows against fp64
    check_bound(oracle, bits(torch, C1), Ab, Bb, kind, rows=(1000, 1032))


@pytest.mark.parametrize("kind", KINDS)
def test_config_8192(handle, torch_gpu, oracle, kind, parity_stats):
    """fp16 / bf16 8192^3, N(0,1) from seed 2: stratified sample of full rows and columns
    against fp64, plus a Freivalds projection over the whole matrix."""
    torch = torch_gpu
    n = 8192
    Ab, Bb = wl.normal_16bit(n, n, n, seed=2, kind=kind)
    A, B = to_dev(torch, Ab, kind), to_dev(torch, Bb, kind)
    C = (handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16)(A, B)
    assert "mfma" in handle.last_kernel
    Cb = bits(torch, C)
    Af, Bf = widen(oracle, Ab, kind), widen(oracle, Bb, kind)
    Cf = widen(oracle, Cb, kind)
    assert np.isfinite(Cf).all()
    worst, ratios = 0.0, []
    # full rows: tile seams and corners included
    for r0 in (0, 255, 256, 4095, 4096, 8191 - 7):
        worst = max(worst, check_bound(oracle, Cb, Ab, Bb, kind, rows=(r0, r0 + 8 if r0 + 8 <= n else n),
                                       stats=ratios))
    # full columns via the transposed problem restricted to those columns
    cols = np.array([0, 31, 32, 255, 256, 4095, 4096, 8191])
    ref, S = oracle.gemm_f64(Af, np.ascontiguousarray(Bf[:, cols]), with_abs=True)
    err = np.abs(Cf[:, cols].astype(np.float64) - ref)
    col_ratio = err / error_bound_16(ref, S, n, kind)
    ratios.append(col_ratio.ravel())
    allr = np.concatenate(ratios)
    parity_stats[f"C3_{kind}_8192"] = {
        "kernel": handle.last_kernel, "sampled_entries": int(allr.size),
        "max_err_over_bound": float(allr.max()), "mean_err_over_bound": float(allr.mean()),
        "bound": "u_out*|ref64| + 2*K*2^-24*sum|a||b|, u_out = 2^-11 (fp16) / 2^-8 (bf16)"}
    assert (col_ratio <= 1.0).all()
    # the maximum leaves a factor of six of room (observed 0.16 bf16 / 0.024 fp16); a systematic
    # loss -- a k index dropped in some tile -- would move the mean (observed 0.018 / 0.0025)
    assert allr.mean() <= 0.05, allr.mean()
    # Freivalds: C.x vs A.(B.x) in fp64 for +-1 vectors; output rounding errors are
    # independent with relative size u_out, so the projection error concentrates
    r = np.random.Generator(np.random.PCG64(5))
    u_out = 2.0 ** -11 if kind == "f16" else 2.0 ** -8
    for _ in range(4):
        x = r.choice(np.array([-1.0, 1.0]), size=n)
        lhs = Cf.astype(np.float64) @ x
        rhs = Af.astype(np.float64) @ (Bf.astype(np.float64) @ x)
        scale = np.sqrt((Cf.astype(np.float64) ** 2).sum(axis=1))   # |row|_2
        assert (np.abs(lhs - rhs) <= 8 * u_out * scale).all()
    print(f"[{kind} 8192^3] worst sampled error = {worst:.3f} x bound")


@pytest.mark.parametrize("kind", KINDS)
def test_config_8192_exact(handle, torch_gpu, oracle, kind, parity_stats):
    """fp16 / bf16 8192^3 pinned exactly over the WHOLE matrix.  Inputs from {0, +-0.5, +-1, +-2}:
    every product is a multiple of 1/4 of magnitude at most 4, every partial sum of up to 8192 of
    them is below 2^17 quarter units, so fp32 accumulation is exact in ANY order and the one
    correct output is narrow(exact sum).  The exact sums come from a float64 matrix product on
    the host (exact for the same reason, in any blocking), tied to the oracle's own fp32 loop on
    a stratified sample of rows and columns; the GPU result must equal their narrowing bit for
    bit on all 8192 x 8192 entries.  One dropped, repeated or misplaced k index anywhere in the
    four rounds of tiles changes entries by at least 1/4 and fails this."""
    torch = torch_gpu
    n = 8192
    r = np.random.Generator(np.random.PCG64(21))
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    Af, Bf = r.choice(vals, size=(n, n)), r.choice(vals, size=(n, n))
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    Ab, Bb = narrow(Af), narrow(Bf)
    assert np.array_equal(widen(oracle, Ab, kind), Af)       # the inputs are exact in 16 bits
    C = (handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16)(to_dev(torch, Ab, kind), to_dev(torch, Bb, kind))
    assert "mfma" in handle.last_kernel and handle.last_plan == (256, 1)
    Cb = bits(torch, C)
    exact = Af.astype(np.float64) @ Bf.astype(np.float64)
    assert np.abs(exact).max() < 65504 and np.array_equal(exact * 4, np.rint(exact * 4))
    # the host product against the oracle's loop (k ascending, float accumulator), bit for bit
    rows = np.array([0, 1, 31, 32, 255, 256, 257, 4095, 4096, 8190, 8191])
    np.testing.assert_array_equal(oracle.gemm_f32(np.ascontiguousarray(Af[rows]), Bf),
                                  exact[rows].astype(np.float32))
    cols = np.array([0, 3, 4, 127, 128, 255, 256, 4097, 8191])
    np.testing.assert_array_equal(oracle.gemm_f32(Af, np.ascontiguousarray(Bf[:, cols])),
                                  exact[:, cols].astype(np.float32))
    want = narrow(exact.astype(np.float32))
    diff = int((Cb != want).sum())
    parity_stats[f"C3_{kind}_8192_exact_inputs"] = {"kernel": handle.last_kernel, "entries": n * n,
                                                    "entries_differing": diff}
    assert diff == 0

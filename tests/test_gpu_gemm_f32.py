"""fp32 GEMM through the C ABI against the reference CPU GEMM (oracle)."""
import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import workloads as wl

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 3, 7, 17, 33, 65, 129]


def run(handle, torch, A, B):
    return handle.gemm_f32(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()).cpu().numpy()


def scaled_tolerance_ok(gpu, cpu, tol=1e-5):
    """|gpu - cpu| <= tol * max(|cpu|, rms(cpu)), every entry."""
    rms = float(np.sqrt(np.mean(cpu.astype(np.float64) ** 2)))
    lim = tol * np.maximum(np.abs(cpu.astype(np.float64)), rms)
    err = np.abs(gpu.astype(np.float64) - cpu.astype(np.float64))
    return bool((err <= lim).all()), float((err / lim).max())


def test_config_fp32_512(handle, torch_gpu, oracle, parity_stats):
    """fp32 512^3, U[-1,1], seed 0: within the 1e-5 scaled relative tolerance of the CPU loop."""
    A, B = wl.fp32_uniform(512, 512, 512, seed=0)
    C = run(handle, torch_gpu, A, B)
    cpu = oracle.matrixMulCPU(A, B)
    ok, worst = scaled_tolerance_ok(C, cpu)
    # the GPU is no further from fp64 than the fp32 CPU loop's own bound
    C64, S = oracle.gemm_f64(A, B, with_abs=True)
    diff = np.abs(C.astype(np.float64) - cpu.astype(np.float64))
    parity_stats["C1_fp32_512"] = {
        "kernel": handle.last_kernel,
        "max_err_over_scaled_tolerance": worst,          # the gate: <= 1
        "max_abs_diff_vs_cpu_loop": float(diff.max()),
        "mean_abs_diff_vs_cpu_loop": float(diff.mean()),
        # the reference's own compare (TileProgramming/matmulTensor.cu:18-28): absolute 1e-5;
        # reported, not gated: two fp32 summation orders differ by about that much at K = 512
        "reference_checkResult_eps_1e-5": bool(oracle.checkResult(C, cpu, eps=1e-5)),
        "max_elementwise_relative_diff": float((diff / np.maximum(np.abs(cpu), 1e-30)).max()),
        "gpu_max_abs_err_vs_fp64": float(np.abs(C - C64).max()),
        "cpu_loop_max_abs_err_vs_fp64": float(np.abs(cpu - C64).max()),
    }
    assert ok, f"worst error {worst:.3f} x tolerance ({handle.last_kernel})"
    assert (np.abs(C - C64) <= 512 * 2.0 ** -24 * S).all()


@pytest.mark.parametrize("M", SIZES)
@pytest.mark.parametrize("N,K", [(1, 1), (3, 129), (17, 7), (33, 65), (129, 33), (65, 2)])
def test_ragged_shapes(handle, torch_gpu, oracle, rng, M, N, K):
    A = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
    C = run(handle, torch_gpu, A, B)
    cpu = oracle.gemm_f32(A, B)
    ok, worst = scaled_tolerance_ok(C, cpu)
    assert ok, f"{M}x{N}x{K}: {worst}"


def test_exact_inputs_are_bit_exact(handle, torch_gpu, oracle, rng):
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    for (M, N, K) in [(64, 64, 64), (256, 256, 256), (130, 70, 1000), (512, 512, 512), (64, 256, 16),
                      (192, 512, 48), (2048, 2816, 32)]:
        A = rng.choice(vals, size=(M, K))
        B = rng.choice(vals, size=(K, N))
        np.testing.assert_array_equal(run(handle, torch_gpu, A, B), oracle.gemm_f32(A, B))


def test_identity_onehot_leading_dims(handle, torch_gpu, oracle, rng):
    torch = torch_gpu
    n = 96
    A = rng.normal(size=(n, n)).astype(np.float32)
    I = np.eye(n, dtype=np.float32)
    np.testing.assert_array_equal(run(handle, torch, A, I), A)
    np.testing.assert_array_equal(run(handle, torch, I, A), A)
    # ld > cols: operate on sub-blocks of larger device buffers, output into a padded buffer
    big_a = torch.from_numpy(rng.normal(size=(50, 100)).astype(np.float32)).cuda()
    big_b = torch.from_numpy(rng.normal(size=(70, 90)).astype(np.float32)).cuda()
    out = torch.full((50, 64), -7.0, dtype=torch.float32, device="cuda")
    a, b, c = big_a[:, 10:80], big_b[:, 5:45], out[:, 3:43]
    handle.gemm_f32(a, b, out=c)
    cpu = oracle.gemm_f32(a.cpu().numpy(), b.cpu().numpy())
    ok, worst = scaled_tolerance_ok(c.cpu().numpy(), cpu)
    assert ok, worst
    o = out.cpu().numpy()
    assert (o[:, :3] == -7.0).all() and (o[:, 43:] == -7.0).all()   # nothing outside C touched


def test_generic_kernel_equals_cpu_loop_bit_for_bit(handle, torch_gpu, oracle, rng):
    """The any-shape kernel adds one separately rounded product at a time in ascending k,
    the same order as the reference CPU loop."""
    A = rng.uniform(-1, 1, size=(77, 300)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(300, 91)).astype(np.float32)
    with handle.algo(ci.ALGO_GENERIC):
        C = run(handle, torch_gpu, A, B)
    assert "generic" in handle.last_kernel
    np.testing.assert_array_equal(C, oracle.gemm_f32(A, B))


def test_k_zero_and_empty(handle, torch_gpu):
    torch = torch_gpu
    A = torch.empty((4, 0), dtype=torch.float32, device="cuda")
    B = torch.empty((0, 5), dtype=torch.float32, device="cuda")
    out = torch.full((4, 5), 3.0, dtype=torch.float32, device="cuda")
    handle.gemm_f32(A, B, out=out)
    assert (out.cpu().numpy() == 0).all()          # empty sum
    handle.gemm_f32(torch.empty((0, 3), dtype=torch.float32, device="cuda"),
                    torch.empty((3, 5), dtype=torch.float32, device="cuda"))


MFMA_ALGOS = [pytest.param(ci.ALGO_TILE, id="tile"), pytest.param(ci.ALGO_SMALL, id="small")]


@pytest.mark.parametrize("algo", MFMA_ALGOS)
def test_mfma_path_onehot_and_bound(handle, torch_gpu, oracle, rng, algo):
    """Both fp32 MFMA kernels: one-hot rows/columns select exactly, random inputs stay within
    the fp32 summation bound of fp64, leading dimensions and guard columns are respected."""
    torch = torch_gpu
    M, N, K = 512, 768, 272
    with handle.algo(algo):
        Bf = rng.normal(size=(K, N)).astype(np.float32)
        perm = rng.integers(0, K, size=M)
        A = np.zeros((M, K), np.float32)
        A[np.arange(M), perm] = 1.0
        C = run(handle, torch, A, Bf)
        assert ("small" in handle.last_kernel) == (algo == ci.ALGO_SMALL), handle.last_kernel
        assert "mfma" in handle.last_kernel
        np.testing.assert_array_equal(C, Bf[perm])
        Af = rng.normal(size=(M, K)).astype(np.float32)
        permn = rng.integers(0, K, size=N)
        B = np.zeros((K, N), np.float32)
        B[permn, np.arange(N)] = 1.0
        np.testing.assert_array_equal(run(handle, torch, Af, B), Af[:, permn])
        # sub-blocks of larger buffers
        bigA = torch.from_numpy(rng.normal(size=(M, K + 40)).astype(np.float32)).cuda()
        bigB = torch.from_numpy(rng.normal(size=(K, N + 12)).astype(np.float32)).cuda()
        out = torch.full((M, N + 8), -3.0, dtype=torch.float32, device="cuda")
        a, b, c = bigA[:, 8:8 + K], bigB[:, 4:4 + N], out[:, 4:4 + N]
        handle.gemm_f32(a, b, out=c)
        assert "mfma" in handle.last_kernel
    ref, S = oracle.gemm_f64(a.cpu().numpy(), b.cpu().numpy(), with_abs=True)
    assert (np.abs(c.cpu().numpy() - ref) <= K * 2.0 ** -24 * S).all()
    o = out.cpu().numpy()
    assert (o[:, :4] == -3.0).all() and (o[:, 4 + N:] == -3.0).all()


def ragged_check(handle, torch, oracle, rng, algo, shape, pad_cols=4):
    M, N, K = shape
    A = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
    out = torch.full((M + 3, N + pad_cols), -9.0, dtype=torch.float32, device="cuda")
    with handle.algo(algo):
        handle.gemm_f32(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), out=out[:M, :N])
        name = handle.last_kernel
    o = out.cpu().numpy()
    ref, S = oracle.gemm_f64(A, B, with_abs=True)
    assert (np.abs(o[:M, :N] - ref) <= K * 2.0 ** -24 * S + 1e-30).all()
    assert (o[M:] == -9.0).all() and (o[:, N:] == -9.0).all()
    return name


@pytest.mark.parametrize("shape", [(33, 4, 16), (100, 260, 48), (257, 1028, 64), (20000, 512, 784), (1000, 12, 512)])
def test_tile_kernel_ragged_shapes(handle, torch_gpu, oracle, rng, shape):
    """Any M, N a multiple of 4, K a multiple of 16 go through the MFMA tile kernel with
    clamped loads and masked stores; guard rows/columns of the output stay untouched."""
    name = ragged_check(handle, torch_gpu, oracle, rng, ci.ALGO_TILE, shape)
    assert "x256x16_w" in name, name


@pytest.mark.parametrize("shape", [(33, 4, 16), (100, 260, 48), (257, 1028, 64), (1000, 12, 512),
                                   (1, 1, 8), (31, 33, 8), (100, 10, 64), (65, 37, 24),
                                   (20000, 10, 512), (7, 1000, 40)])
@pytest.mark.parametrize("pad_cols", [4, 1])
def test_small_kernel_ragged_shapes(handle, torch_gpu, oracle, rng, shape, pad_cols):
    """Any M and N, K a multiple of 8, go through the 32x32 k-split kernel; output rows need
    no alignment (pad_cols = 1 gives an odd leading dimension)."""
    name = ragged_check(handle, torch_gpu, oracle, rng, ci.ALGO_SMALL, shape, pad_cols)
    assert "small" in name, name


@pytest.mark.parametrize("shape", [(64, 1, 16), (65, 3, 48), (1000, 10, 784), (20000, 10, 512), (333, 16, 2048),
                                   (127, 13, 1040), (4097, 7, 32)])
@pytest.mark.parametrize("pad_cols", [4, 1])
def test_narrow_kernel_ragged_shapes(handle, torch_gpu, oracle, rng, shape, pad_cols):
    """N <= 16, K a multiple of 16 up to 2048, M >= 64: the 16x16 form of the small kernel
    (each wave keeps its share of B in registers); guard rows / columns stay untouched."""
    name = ragged_check(handle, torch_gpu, oracle, rng, ci.ALGO_SMALL, shape, pad_cols)
    assert "small_16x16" in name, name


@pytest.mark.parametrize("shape", [(63, 10, 512), (1000, 17, 512), (1000, 10, 2064), (1000, 10, 520)])
def test_narrow_kernel_gate(handle, torch_gpu, oracle, rng, shape):
    """Just outside the 16x16 form's conditions (M, N, K share per wave, K % 16) the 32x32
    form runs."""
    name = ragged_check(handle, torch_gpu, oracle, rng, ci.ALGO_SMALL, shape)
    assert "small_32x32" in name, name


def test_narrow_kernel_onehot_bias_relu(handle, torch_gpu, oracle, rng):
    """One-hot operands pick single elements (every index of the fragment layout), exact
    inputs make bias + ReLU comparable bit for bit."""
    torch = torch_gpu
    M, N, K = 200, 10, 784
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    X = rng.choice(vals, size=(M, K))
    Wm = np.zeros((K, N), np.float32)
    ks = rng.integers(0, K, size=N)
    Wm[ks, np.arange(N)] = 1.0                      # column n copies column ks[n] of X
    with handle.algo(ci.ALGO_SMALL):
        out = handle.gemm_f32(torch.from_numpy(X).cuda(), torch.from_numpy(Wm).cuda()).cpu().numpy()
        assert "small_16x16" in handle.last_kernel
        np.testing.assert_array_equal(out, X[:, ks])
        Wd = rng.choice(vals, size=(K, N))
        bias = rng.choice(vals, size=N)
        L = handle.linear_f32(torch.from_numpy(X).cuda(), torch.from_numpy(Wd).cuda(),
                              torch.from_numpy(bias).cuda(), ci.ACT_RELU).cpu().numpy()
        assert "small_16x16" in handle.last_kernel
    np.testing.assert_array_equal(L, oracle.linear_f32(X, Wd, bias, True))


def test_narrow_kernel_weights_inside_a_wider_matrix(handle, torch_gpu, oracle, rng):
    """Contiguous, aligned weights pass through LDS as 16-byte pieces; a column slice of a
    wider matrix (other leading dimension, unaligned start) is read element by element.
    Both give the same bits."""
    torch = torch_gpu
    M, N, K = 500, 10, 512
    X = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    wide = rng.uniform(-1, 1, size=(K, 24)).astype(np.float32)
    Wc = np.ascontiguousarray(wide[:, 3:3 + N])
    xd, wd = torch.from_numpy(X).cuda(), torch.from_numpy(wide).cuda()
    with handle.algo(ci.ALGO_SMALL):
        a = handle.gemm_f32(xd, torch.from_numpy(Wc).cuda()).cpu().numpy()
        assert "small_16x16" in handle.last_kernel
        b = handle.gemm_f32(xd, wd[:, 3:3 + N]).cpu().numpy()
        assert "small_16x16" in handle.last_kernel
    np.testing.assert_array_equal(a, b)
    ref, S = oracle.gemm_f64(X, Wc, with_abs=True)
    assert (np.abs(a - ref) <= K * 2.0 ** -24 * S + 1e-30).all()


def test_default_choice_by_shape(handle, torch_gpu):
    """Small problems and narrow outputs go to the 32x32 kernel, large ones to 256-column
    tiles, what neither takes to the any-shape matrix-core kernel."""
    torch = torch_gpu
    def kernel_for(M, N, K):
        handle.gemm_f32(torch.zeros((M, K), device="cuda"), torch.zeros((K, N), device="cuda"))
        return handle.last_kernel
    assert handle.get_algo() == ci.ALGO_DEFAULT
    assert "small" in kernel_for(512, 512, 512)
    assert "small" in kernel_for(1024, 1024, 1024)
    assert "small_16x16" in kernel_for(20000, 10, 512)
    assert "x256x16_w" in kernel_for(2048, 2048, 2048)
    assert "x256x16_w" in kernel_for(4096, 4096, 64)
    assert "x256x16_w" in kernel_for(20000, 512, 784)
    assert kernel_for(512, 512, 4096).endswith("_splitk")      # long K: tile kernel, K split
    assert kernel_for(256, 1024, 8192).endswith("_splitk")
    assert "mfma_any" in kernel_for(77, 91, 300)


def test_all_kernels_agree_on_exact_inputs(handle, torch_gpu, oracle, rng):
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    A = rng.choice(vals, size=(300, 128))
    B = rng.choice(vals, size=(128, 260))
    want = oracle.gemm_f32(A, B)
    for algo in (ci.ALGO_GENERIC, ci.ALGO_TILE, ci.ALGO_SMALL, ci.ALGO_DEFAULT):
        with handle.algo(algo):
            np.testing.assert_array_equal(run(handle, torch_gpu, A, B), want)

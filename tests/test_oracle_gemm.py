"""Pins the oracle's GEMMs (TileProgramming/tensor_utils.cu:34-45 and its generalisations)
with facts that do not come from the oracle's own formula: identities, one-hot selection,
inputs whose arithmetic is exact, integer closed forms, transposition, an int64 brute force
and numpy's independent matmul."""
import numpy as np
import pytest

SIZES = [1, 2, 3, 7, 17, 33, 65, 129]


def _exact_values(r, shape):
    """Values whose products and partial sums are exact in fp32 for K <= a few thousand."""
    return r.choice(np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32), size=shape)


def test_matrixMulCPU_identity_and_onehot(oracle, rng):
    w = 37
    A = rng.normal(size=(w, w)).astype(np.float32)
    I = np.eye(w, dtype=np.float32)
    np.testing.assert_array_equal(oracle.matrixMulCPU(A, I), A)
    np.testing.assert_array_equal(oracle.matrixMulCPU(I, A), A)
    # one-hot row i0 of A selects row k0 of B; catches any transposed operand or index
    E = np.zeros((w, w), np.float32)
    E[5, 11] = 1.0
    C = oracle.matrixMulCPU(E, A)
    expect = np.zeros((w, w), np.float32)
    expect[5] = A[11]
    np.testing.assert_array_equal(C, expect)
    C = oracle.matrixMulCPU(A, E)
    expect = np.zeros((w, w), np.float32)
    expect[:, 11] = A[:, 5]
    np.testing.assert_array_equal(C, expect)


def test_matrixMulCPU_all_ones(oracle):
    w = 64
    one = np.ones((w, w), np.float32)
    np.testing.assert_array_equal(oracle.matrixMulCPU(one, one), np.full((w, w), w, np.float32))


def test_matrixMulCPU_sequential_fp32_order(oracle):
    """The accumulator is a float that adds products one by one in ascending k:
    1 + 2^-24 + 2^-24 ... stays 1 (each addend is lost), whereas any pairwise or reversed
    order, or a double accumulator, gives a larger sum."""
    w = 64
    A = np.zeros((w, w), np.float32)
    B = np.zeros((w, w), np.float32)
    A[0, :] = 1.0
    B[:, 0] = np.float32(2.0 ** -24)
    B[0, 0] = 1.0
    C = oracle.matrixMulCPU(A, B)
    assert C[0, 0] == np.float32(1.0)
    # reversed k order accumulates the small terms first: 63*2^-24 + 1 rounds up
    assert np.float32(np.float32(63 * 2.0 ** -24) + np.float32(1.0)) > np.float32(1.0)


@pytest.mark.parametrize("w", [1, 2, 17, 64, 129])
def test_fast_order_is_bit_identical_to_reference_loop(oracle, rng, w):
    A = rng.uniform(-1, 1, size=(w, w)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(w, w)).astype(np.float32)
    ref = oracle.matrixMulCPU(A, B)
    np.testing.assert_array_equal(oracle.gemm_f32(A, B), ref)
    np.testing.assert_array_equal(oracle.gemm_f32_ijk(A, B), ref)


@pytest.mark.parametrize("M", SIZES[::2])
@pytest.mark.parametrize("N", SIZES[1::2])
@pytest.mark.parametrize("K", [1, 3, 33, 129])
def test_rectangular_exact_vs_numpy(oracle, rng, M, N, K):
    A = _exact_values(rng, (M, K))
    B = _exact_values(rng, (K, N))
    expect = (A.astype(np.float64) @ B.astype(np.float64))
    np.testing.assert_array_equal(oracle.gemm_f32(A, B).astype(np.float64), expect)
    np.testing.assert_array_equal(oracle.gemm_f32_ijk(A, B).astype(np.float64), expect)
    np.testing.assert_array_equal(oracle.gemm_f64(A, B), expect)


def test_f32_close_to_f64_and_transpose(oracle, rng):
    M, N, K = 70, 50, 300
    A = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
    C32 = oracle.gemm_f32(A, B)
    C64, S = oracle.gemm_f64(A, B, with_abs=True)
    np.testing.assert_allclose(C64, A.astype(np.float64) @ B.astype(np.float64), rtol=1e-13,
                               atol=1e-13)
    np.testing.assert_allclose(S, np.abs(A).astype(np.float64) @ np.abs(B).astype(np.float64),
                               rtol=1e-13)
    # sequential fp32 summation error bound: K * 2^-24 * sum|a||b|
    assert (np.abs(C32 - C64) <= K * 2.0 ** -24 * S).all()
    # (A.B)^T = B^T.A^T holds exactly in fp64 accumulation order independent to 1e-13
    np.testing.assert_allclose(oracle.gemm_f64(B.T.copy(), A.T.copy()), C64.T, rtol=1e-12, atol=1e-12)
    # row window
    np.testing.assert_array_equal(oracle.gemm_f64(A, B, rows=(10, 20)), C64[10:20])


@pytest.mark.parametrize("b_is_nk", [False, True])
def test_int8_closed_forms(oracle, b_is_nk):
    M, N, K = 5, 6, 8192
    A = np.full((M, K), 127, np.int8)
    B = np.full((N, K) if b_is_nk else (K, N), 127, np.int8)
    assert (oracle.gemm_i8_i32(A, B, b_is_nk) == 16129 * K).all()      # 132 128 768 < 2^31
    assert (oracle.gemm_i8_i32(-A, B, b_is_nk) == -16129 * K).all()
    A = np.full((M, K), -128, np.int8)
    B = np.full((N, K) if b_is_nk else (K, N), -128, np.int8)
    assert (oracle.gemm_i8_i32(A, B, b_is_nk) == 16384 * K).all()


@pytest.mark.parametrize("b_is_nk", [False, True])
@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 7, 17), (33, 65, 129), (64, 64, 256), (17, 2, 1)])
def test_int8_vs_int64_bruteforce_and_numpy(oracle, rng, b_is_nk, shape):
    M, N, K = shape
    A = rng.integers(-128, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-128, 128, size=(N, K) if b_is_nk else (K, N), dtype=np.int8)
    got = oracle.gemm_i8_i32(A, B, b_is_nk)
    Bm = B.T if b_is_nk else B
    expect = A.astype(np.int64) @ Bm.astype(np.int64)
    np.testing.assert_array_equal(got.astype(np.int64), expect)
    np.testing.assert_array_equal(oracle.gemm_i8_i64_ijk(A, B, b_is_nk), expect)


def test_int8_onehot_layouts(oracle, rng):
    M, N, K = 9, 11, 13
    B = rng.integers(-128, 128, size=(K, N), dtype=np.int8)
    E = np.zeros((M, K), np.int8)
    E[4, 7] = 1
    C = oracle.gemm_i8_i32(E, B)
    assert (C[4] == B[7]).all() and (np.delete(C, 4, axis=0) == 0).all()
    C = oracle.gemm_i8_i32(E, np.ascontiguousarray(B.T), b_is_nk=True)
    assert (C[4] == B[7]).all()


def test_checkResult(oracle):
    """matmulTensor.cu:18-28: absolute tolerance, strict '>' comparison."""
    w = 8
    cpu = np.zeros((w, w), np.float32)
    gpu = cpu.copy()
    assert oracle.checkResult(gpu, cpu)
    gpu[3, 3] = 0.5e-5
    assert oracle.checkResult(gpu, cpu)            # below eps
    gpu[3, 3] = 2e-5
    assert not oracle.checkResult(gpu, cpu)        # above eps
    assert oracle.checkResult(gpu, cpu, eps=1e-4)
    big = np.full((w, w), 1e6, np.float32)
    assert not oracle.checkResult(big + np.float32(0.0625), big)  # absolute, not relative

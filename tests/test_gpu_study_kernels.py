"""Study kernels (TileProgramming demo counterparts) through the C ABI against the oracle.

The demo draws inputs as rand() / RAND_MAX, i.e. uniform in [0, 1], keeps an fp32 master and a
rounded 16-bit copy (TileProgramming/tensor_utils.h:50-72), and compares with matrixMulCPU of
the masters under an absolute eps (matmulTensor.cu:18-28; 1e-5, or 2e-3 for bf16).  Here the
fp32 tiled kernel is held to bit equality with matrixMulCPU; the matrix-core kernels are held
to the fp32 summation bound around an fp64 product of the rounded inputs, and the demo's own
comparison is evaluated on top.
"""
import numpy as np
import pytest

from gpu_util import to_dev

pytestmark = pytest.mark.gpu


def demo_inputs(rng, w):
    return (rng.uniform(0, 1, size=(w, w)).astype(np.float32),
            rng.uniform(0, 1, size=(w, w)).astype(np.float32))


@pytest.mark.parametrize("w", [1, 2, 31, 32, 33, 100, 257, 1024])
def test_tiled_equals_cpu_loop_bit_for_bit(handle, torch_gpu, oracle, rng, w):
    A, B = demo_inputs(rng, w)
    C = handle.matrixMulTiled(to_dev(torch_gpu, A), to_dev(torch_gpu, B)).cpu().numpy()
    assert handle.last_kernel == "study_tiled_f32_32x32"
    cpu = oracle.matrixMulCPU(A, B)
    np.testing.assert_array_equal(C, cpu)
    assert oracle.checkResult(C, cpu, eps=1e-5)          # the demo's own check


def test_tiled_signed_inputs_and_onehot(handle, torch_gpu, oracle, rng):
    w = 96
    A = rng.normal(size=(w, w)).astype(np.float32)
    B = rng.normal(size=(w, w)).astype(np.float32)
    C = handle.matrixMulTiled(to_dev(torch_gpu, A), to_dev(torch_gpu, B)).cpu().numpy()
    np.testing.assert_array_equal(C, oracle.matrixMulCPU(A, B))
    P = np.zeros((w, w), np.float32)
    perm = rng.permutation(w)
    P[np.arange(w), perm] = 1.0
    np.testing.assert_array_equal(
        handle.matrixMulTiled(to_dev(torch_gpu, P), to_dev(torch_gpu, B)).cpu().numpy(), B[perm])
    np.testing.assert_array_equal(
        handle.matrixMulTiled(to_dev(torch_gpu, A), to_dev(torch_gpu, P)).cpu().numpy(),
        A[:, np.argsort(perm)])


@pytest.mark.parametrize("kind", ["f16", "bf16"])
@pytest.mark.parametrize("w", [1, 15, 16, 33, 100, 512, 1024])
def test_matrix_cores_within_fp32_bound(handle, torch_gpu, oracle, rng, kind, w):
    A, B = demo_inputs(rng, w)
    narrow = oracle.f32_to_f16 if kind == "f16" else oracle.f32_to_bf16
    widen = oracle.f16_to_f32 if kind == "f16" else oracle.bf16_to_f32
    Ah, Bh = narrow(A), narrow(B)
    C = handle.matrixMulMatrixCores(to_dev(torch_gpu, Ah, kind), to_dev(torch_gpu, Bh, kind)).cpu().numpy()
    assert handle.last_kernel == f"study_mfma_{kind}_32x32x16"
    ref, S = oracle.gemm_f64(widen(Ah), widen(Bh), with_abs=True)
    # products of two 16-bit values are exact in fp32: only the fp32 accumulation rounds
    assert (np.abs(C - ref) <= 2 * w * 2.0 ** -24 * S + 1e-30).all()
    # the demo's comparison against the fp32 masters: dominated by the input rounding,
    # |error| <= (2u + u^2) * sum |a||b| + accumulation, u = 2^-11 (fp16) / 2^-8 (bf16)
    u = 2.0 ** -11 if kind == "f16" else 2.0 ** -8
    cpu = oracle.matrixMulCPU(A, B)
    _, Sm = oracle.gemm_f64(A, B, with_abs=True)
    assert (np.abs(C.astype(np.float64) - cpu) <= (2 * u + u * u) * Sm + 4 * w * 2.0 ** -24 * Sm).all()


@pytest.mark.parametrize("kind", ["f16", "bf16"])
def test_matrix_cores_exact_inputs_and_onehot(handle, torch_gpu, oracle, rng, kind):
    w = 200
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    A = rng.choice(vals, size=(w, w))
    B = rng.choice(vals, size=(w, w))
    narrow = oracle.f32_to_f16 if kind == "f16" else oracle.f32_to_bf16
    run = lambda X, Y: handle.matrixMulMatrixCores(to_dev(torch_gpu, narrow(X), kind),
                                                   to_dev(torch_gpu, narrow(Y), kind)).cpu().numpy()
    np.testing.assert_array_equal(run(A, B), oracle.matrixMulCPU(A, B))
    P = np.zeros((w, w), np.float32)
    perm = rng.permutation(w)
    P[np.arange(w), perm] = 1.0
    np.testing.assert_array_equal(run(P, B), B[perm])               # row selection
    np.testing.assert_array_equal(run(A, P), A[:, np.argsort(perm)])  # column selection
    # not symmetric: A.B differs from A.B^T, which a column-major read of B would give
    assert not np.array_equal(run(A, B), oracle.matrixMulCPU(A, B.T.copy()))


def test_study_kernel_arguments(handle, torch_gpu):
    import cudaintro_amd as ci
    lib, h = handle.lib, handle.raw
    a = torch_gpu.zeros((4, 4), device="cuda")
    p = a.data_ptr()
    assert lib.cigemm_matrixMulTiled(h, p, p, p, -1) == ci.Status.INVALID_VALUE
    assert lib.cigemm_matrixMulTiled(h, None, p, p, 4) == ci.Status.INVALID_VALUE
    assert lib.cigemm_matrixMulMatrixCores(h, p, None, p, 4) == ci.Status.INVALID_VALUE
    assert lib.cigemm_matrixMulMatrixCoresBfloat16(h, p, p, None, 4) == ci.Status.INVALID_VALUE
    assert lib.cigemm_matrixMulTiled(h, None, None, None, 0) == ci.Status.SUCCESS

"""Linear layer (GEMM + bias + ReLU fused) through the C ABI against the oracle's restatement
of the MNIST MLP forward kernels."""
import numpy as np
import pytest

import cudaintro_amd as ci

pytestmark = pytest.mark.gpu


def check(handle, torch, oracle, X, W, bias, relu, expect=None, algo=ci.ALGO_DEFAULT):
    with handle.algo(algo):
        out = handle.linear_f32(torch.from_numpy(X).cuda(), torch.from_numpy(W).cuda(),
                                torch.from_numpy(bias).cuda() if bias is not None else None,
                                ci.ACT_RELU if relu else ci.ACT_NONE).cpu().numpy()
    if expect is not None:
        assert expect in handle.last_kernel, handle.last_kernel
    cpu = oracle.linear_f32(X, W, bias, relu)
    # fp32 gate of the GEMM path: |gpu - cpu| <= 1e-5 * max(|cpu|, rms of the pre-activation)
    pre = oracle.linear_f32(X, W, bias, False)
    rms = float(np.sqrt(np.mean(pre.astype(np.float64) ** 2)))
    lim = 1e-5 * np.maximum(np.abs(cpu), rms)
    err = np.abs(out.astype(np.float64) - cpu)
    assert (err <= lim).all(), float((err / lim).max())
    if relu:
        assert (out >= 0).all()
    return out


def test_mnist_hidden_layer(handle, torch_gpu, oracle, rng):
    """20000 x 784 -> 512 with ReLU (MNIST/mnist_nn.h:12-15): pixel-like inputs in [0,1]."""
    X = rng.uniform(0, 1, size=(20000, 784)).astype(np.float32)
    W = (rng.normal(size=(784, 512)) * np.sqrt(2.0 / 784)).astype(np.float32)
    b = rng.normal(size=512).astype(np.float32) * 0.1
    out = check(handle, torch_gpu, oracle, X, W, b, True, expect="x256x16_w")
    assert (out == 0).mean() > 0.1      # ReLU actually clips something


def test_mnist_output_layer(handle, torch_gpu, oracle, rng):
    """20000 x 512 -> 10, no activation: N = 10 goes to the 32x32 k-split kernel."""
    X = np.maximum(rng.normal(size=(20000, 512)), 0).astype(np.float32)
    W = (rng.normal(size=(512, 10)) * 0.05).astype(np.float32)
    b = rng.normal(size=10).astype(np.float32) * 0.1
    check(handle, torch_gpu, oracle, X, W, b, False, expect="small")


@pytest.mark.parametrize("shape", [(1, 1, 1), (3, 5, 7), (64, 64, 64), (100, 48, 260), (257, 16, 12), (512, 512, 512)])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_shapes(handle, torch_gpu, oracle, rng, shape, relu, with_bias):
    M, K, N = shape
    X = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    W = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
    b = rng.uniform(-1, 1, size=N).astype(np.float32) if with_bias else None
    check(handle, torch_gpu, oracle, X, W, b, relu)


@pytest.mark.parametrize("algo,shape", [
    (ci.ALGO_GENERIC, (100, 48, 260)), (ci.ALGO_TILE, (100, 48, 260)), (ci.ALGO_SMALL, (100, 48, 260)),
    (ci.ALGO_SMALL, (257, 16, 10)), (ci.ALGO_SMALL, (40, 512, 33)), (ci.ALGO_TILE, (300, 64, 512))])
@pytest.mark.parametrize("relu", [False, True])
@pytest.mark.parametrize("with_bias", [False, True])
def test_each_kernel_family(handle, torch_gpu, oracle, rng, algo, shape, relu, with_bias):
    M, K, N = shape
    X = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    W = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
    b = rng.uniform(-1, 1, size=N).astype(np.float32) if with_bias else None
    expect = {ci.ALGO_GENERIC: "generic", ci.ALGO_TILE: "x256x16_w", ci.ALGO_SMALL: "small"}[algo]
    check(handle, torch_gpu, oracle, X, W, b, relu, expect=expect, algo=algo)


def test_exact_inputs_bit_exact(handle, torch_gpu, oracle, rng):
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    for (M, K, N) in [(128, 64, 256), (100, 32, 20), (20000, 784, 512)]:
        X = rng.choice(vals, size=(M, K))
        W = rng.choice(vals, size=(K, N))
        b = rng.choice(vals, size=N)
        out = handle.linear_f32(torch_gpu.from_numpy(X).cuda(), torch_gpu.from_numpy(W).cuda(),
                                torch_gpu.from_numpy(b).cuda(), ci.ACT_RELU).cpu().numpy()
        np.testing.assert_array_equal(out, oracle.linear_f32(X, W, b, True))


def test_bad_activation(handle, torch_gpu):
    a = torch_gpu.zeros((8, 8), device="cuda")
    with pytest.raises(ci.CigemmError, match="INVALID_VALUE"):
        handle.linear_f32(a, a, None, act=7)

"""Pins the oracle's MLP forward layer (MNIST/mnist_nn.cu:10-24, 27-33, 36-49)."""
import numpy as np


def test_bias_only_and_identity(oracle, rng):
    M, K, N = 5, 7, 7
    bias = rng.normal(size=N).astype(np.float32)
    X = rng.normal(size=(M, K)).astype(np.float32)
    # zero weights: every row of the output is the bias
    out = oracle.linear_f32(X, np.zeros((K, N), np.float32), bias)
    np.testing.assert_array_equal(out, np.broadcast_to(bias, (M, N)))
    # identity weights, no bias: output equals the input
    np.testing.assert_array_equal(oracle.linear_f32(X, np.eye(K, dtype=np.float32)), X)
    # weights are input-major: W[i][j] multiplies input i into output j
    W = np.zeros((K, N), np.float32)
    W[2, 5] = 3.0
    expect = np.zeros((M, N), np.float32)
    expect[:, 5] = 3.0 * X[:, 2]
    np.testing.assert_array_equal(oracle.linear_f32(X, W), expect)


def test_relu_and_order(oracle):
    X = np.array([[1.0, -2.0]], np.float32)
    W = np.array([[1.0, 1.0], [1.0, -1.0]], np.float32)
    bias = np.array([0.5, -4.0], np.float32)
    np.testing.assert_array_equal(oracle.linear_f32(X, W, bias), [[-0.5, -1.0]])
    np.testing.assert_array_equal(oracle.linear_f32(X, W, bias, relu=True), [[0.0, 0.0]])
    np.testing.assert_array_equal(oracle.linear_f32(-X, W, bias, relu=True), [[1.5, 0.0]])
    # the sum starts AT the bias: 2^24 + 1 + 1 stays 2^24 in fp32, whereas bias added last gives 2^24 + 2
    Xs = np.ones((1, 2), np.float32)
    Ws = np.ones((2, 1), np.float32)
    b = np.array([2.0 ** 24], np.float32)
    assert oracle.linear_f32(Xs, Ws, b)[0, 0] == np.float32(2.0 ** 24)


def test_against_numpy(oracle, rng):
    M, K, N = 33, 100, 17
    X = rng.uniform(-1, 1, size=(M, K)).astype(np.float32)
    W = rng.uniform(-1, 1, size=(K, N)).astype(np.float32)
    bias = rng.uniform(-1, 1, size=N).astype(np.float32)
    ref = X.astype(np.float64) @ W.astype(np.float64) + bias
    out = oracle.linear_f32(X, W, bias)
    S = np.abs(X).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(bias)
    assert (np.abs(out - ref) <= (K + 1) * 2.0 ** -24 * S).all()
    np.testing.assert_array_equal(oracle.linear_f32(X, W, bias, relu=True), np.maximum(out, 0))

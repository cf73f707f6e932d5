"""The build-defined dequantize epilogue and absmax quantizer of the oracle."""
import numpy as np


def test_dequant_matches_numpy_float32(oracle, rng):
    M, N = 37, 53
    acc = rng.integers(-(2 ** 27), 2 ** 27, size=(M, N)).astype(np.int32)   # beyond 2^24: conversion rounds
    sa = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
    sb = rng.uniform(1e-3, 1e-1, N).astype(np.float32)
    # numpy float32 arithmetic rounds each operation separately (no fusing)
    expect = (acc.astype(np.float32) * sa[:, None]) * sb[None, :]
    got = oracle.dequant(acc, sa, sb)
    np.testing.assert_array_equal(got, expect)
    # per-tensor
    got = oracle.dequant(acc, sa[:1], sb[:1])
    np.testing.assert_array_equal(got, (acc.astype(np.float32) * sa[0]) * sb[0])
    # mixed
    got = oracle.dequant(acc, sa, sb[:1])
    np.testing.assert_array_equal(got, (acc.astype(np.float32) * sa[:, None]) * sb[0])
    # association matters: (acc*sa)*sb != acc*(sa*sb) for some entries, and the oracle is the former
    other = acc.astype(np.float32) * (sa[:, None] * sb[None, :])
    assert (other != expect).any()


def test_dequant_bf16_is_rne_of_f32(oracle, rng):
    M, N = 16, 24
    acc = rng.integers(-(2 ** 26), 2 ** 26, size=(M, N)).astype(np.int32)
    sa = rng.uniform(1e-3, 1e-1, M).astype(np.float32)
    sb = rng.uniform(1e-3, 1e-1, N).astype(np.float32)
    f = oracle.dequant(acc, sa, sb)
    np.testing.assert_array_equal(oracle.dequant(acc, sa, sb, out_dtype="bf16"), oracle.f32_to_bf16(f))


def test_dequant_per_tensor_127(oracle):
    # acc * (1/127) * (1/127) at the int8 extremes: 16129*K / 16129 = K up to fp32 rounding
    K = 4096
    acc = np.full((2, 2), 16129 * K, np.int32)
    s = np.array([1.0 / 127.0], np.float32)
    out = oracle.dequant(acc, s, s)
    assert abs(out[0, 0] - K) <= K * 3 * 2.0 ** -24


def test_quantizer_hand_cases(oracle):
    x = np.array([
        [0.0, 0.0, 0.0, 0.0],            # zero row: scale 1, all zero
        [0.0, 0.0, 5.0, 0.0],            # single spike -> 127
        [-3.0, 3.0, 1.5, -1.5],          # +-absmax -> +-127; 1.5/(3/127) = 63.5 -> tie to even 64
        [127.0, 1.5, 2.5, -0.5],         # scale exactly 1: ties 1.5 -> 2, 2.5 -> 2, -0.5 -> -0
    ], np.float32)
    q, s = oracle.quantize_rows_i8(x)
    assert s.tolist() == [1.0, np.float32(5.0) / np.float32(127.0), np.float32(3.0) / np.float32(127.0), 1.0]
    assert q[0].tolist() == [0, 0, 0, 0]
    assert q[1].tolist() == [0, 0, 127, 0]
    assert q[2, 0] == -127 and q[2, 1] == 127 and abs(int(q[2, 2])) in (63, 64) and q[2, 2] == -q[2, 3]
    assert q[3].tolist() == [127, 2, 2, 0]


def test_quantizer_matches_workload_helper(oracle, rng):
    from cudaintro_amd import workloads as wl
    x = rng.normal(size=(64, 300)).astype(np.float32)
    q, s = oracle.quantize_rows_i8(x)
    q2, s2 = wl.quantize_rows_absmax(x)
    np.testing.assert_array_equal(s, s2)
    np.testing.assert_array_equal(q, q2)
    assert np.abs(q).max() == 127
    # reconstruction error at most half a step
    assert (np.abs(q.astype(np.float32) * s[:, None] - x) <= 0.5 * s[:, None] * (1 + 1e-6)).all()

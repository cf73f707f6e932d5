"""The oracle's input generators against known answers derived from the formula
(quantization/GEMM_fp32.cu:13-16, GEMM_bf16.cu:14-18, GEMM_fp16.cu:14-18, GEMM_int8.cu:14-18)."""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "fill_random_kat.json")))
IDX = KAT["idx"]
COUNT = max(IDX) + 1


def test_hash64(oracle):
    for seed, vals in KAT["hash64"].items():
        for i, v in zip(IDX, vals):
            assert oracle.hash64(i, int(seed, 16)) == int(v, 16)


def test_fill_f32(oracle):
    for seed, vals in KAT["f32"].items():
        a = oracle.fill_random_f32(COUNT, int(seed, 16))
        assert a.view(np.uint32)[IDX].tolist() == vals


def test_fill_bf16(oracle):
    for seed, vals in KAT["bf16"].items():
        a = oracle.fill_random_bf16(COUNT, int(seed, 16))
        assert a[IDX].tolist() == vals


def test_fill_f16(oracle):
    for seed, vals in KAT["f16"].items():
        a = oracle.fill_random_f16(COUNT, int(seed, 16))
        assert a[IDX].tolist() == vals


def test_fill_i8(oracle):
    for seed, vals in KAT["i8"].items():
        a = oracle.fill_random_i8(COUNT, int(seed, 16))
        assert a[IDX].tolist() == vals
        assert a.min() == -127 and a.max() == 127


def test_hand_checked_known_answers(oracle):
    """Hand-checked decimal values for the first elements of the 4096^2 operands."""
    a = oracle.fill_random_f32(1 << 24, 0x3234)
    np.testing.assert_array_equal(
        a[:4], np.array([0.194802642, -0.172687471, -0.540177584, -0.907667637], np.float32))
    assert a[-1] == np.float32(0.773311257)
    assert [float.hex(float(v)) for v in a[:2]] == ["0x1.8ef4b00000000p-3", "-0x1.61a9f80000000p-3"]
    i = oracle.fill_random_i8(1 << 24, 0x4234)
    assert i[:8].tolist() == [22, 34, 46, 58, -27, -15, -3, 9] and i[-1] == -3
    assert oracle.fill_random_i8(8, 0x6676).tolist() == [-53, -41, -77, -65, -102, -89, -127, -114]


def test_range_and_affine(oracle):
    a = oracle.fill_random_f32(100000, 7, lo=-1.0, hi=1.0)
    assert a.min() >= -1.0 and a.max() <= 1.0
    b = oracle.fill_random_f32(100000, 7, lo=0.0, hi=1.0)
    # lo + r*(hi-lo): with (lo,hi)=(-1,1) the product 2r is exact, so a == 2b - 1 exactly
    np.testing.assert_array_equal(a, np.float32(2.0) * b - np.float32(1.0))

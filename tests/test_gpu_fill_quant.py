"""Device generators and quantizer against the oracle, bit for bit, through the C ABI."""
import json
import os

import numpy as np
import pytest

from gpu_util import bits

pytestmark = pytest.mark.gpu
HERE = os.path.dirname(os.path.abspath(__file__))
KAT = json.load(open(os.path.join(HERE, "golden", "fill_random_kat.json")))


@pytest.mark.parametrize("count", [0, 1, 7, 255, 256, 1000003, 1 << 24])
def test_fill_f32(handle, torch_gpu, oracle, count):
    t = torch_gpu.empty(count, dtype=torch_gpu.float32, device="cuda")
    handle.fill_random(t, 0x3234)
    np.testing.assert_array_equal(t.cpu().numpy().view(np.uint32),
                                  oracle.fill_random_f32(count, 0x3234).view(np.uint32))


@pytest.mark.parametrize("dtype,seed,fn", [("bfloat16", 0x1234, "fill_random_bf16"),
                                           ("bfloat16", 0x9876, "fill_random_bf16"),
                                           ("float16", 0x2234, "fill_random_f16"),
                                           ("float16", 0x8876, "fill_random_f16")])
def test_fill_16(handle, torch_gpu, oracle, dtype, seed, fn):
    for count in (5, 4099, 1 << 24):
        t = torch_gpu.empty(count, dtype=getattr(torch_gpu, dtype), device="cuda")
        handle.fill_random(t, seed)
        np.testing.assert_array_equal(bits(torch_gpu, t), getattr(oracle, fn)(count, seed))


@pytest.mark.parametrize("seed", [0x4234, 0x6676])
def test_fill_i8(handle, torch_gpu, oracle, seed):
    for count in (3, 4097, 1 << 24):
        t = torch_gpu.empty(count, dtype=torch_gpu.int8, device="cuda")
        handle.fill_random(t, seed, -127, 127)
        np.testing.assert_array_equal(t.cpu().numpy(), oracle.fill_random_i8(count, seed))


def test_fill_golden_vectors(handle, torch_gpu):
    idx = KAT["idx"]
    n = max(idx) + 1
    for seed, vals in KAT["f32"].items():
        t = handle.fill_random(torch_gpu.empty(n, dtype=torch_gpu.float32, device="cuda"), int(seed, 16))
        assert t.cpu().numpy().view(np.uint32)[idx].tolist() == vals
    for seed, vals in KAT["bf16"].items():
        t = handle.fill_random(torch_gpu.empty(n, dtype=torch_gpu.bfloat16, device="cuda"), int(seed, 16))
        assert bits(torch_gpu, t)[idx].tolist() == vals
    for seed, vals in KAT["f16"].items():
        t = handle.fill_random(torch_gpu.empty(n, dtype=torch_gpu.float16, device="cuda"), int(seed, 16))
        assert bits(torch_gpu, t)[idx].tolist() == vals
    for seed, vals in KAT["i8"].items():
        t = handle.fill_random(torch_gpu.empty(n, dtype=torch_gpu.int8, device="cuda"), int(seed, 16), -127, 127)
        assert t.cpu().numpy()[idx].tolist() == vals


def test_fill_unaligned_and_other_range(handle, torch_gpu, oracle):
    base = torch_gpu.zeros(1000, dtype=torch_gpu.float32, device="cuda")
    handle.fill_random(base[3:903], 99, lo=0.0, hi=4.0)   # pointer 12 bytes past alignment
    got = base.cpu().numpy()
    np.testing.assert_array_equal(got[3:903], oracle.fill_random_f32(900, 99, 0.0, 4.0))
    assert (got[:3] == 0).all() and (got[903:] == 0).all()
    b = torch_gpu.zeros(1001, dtype=torch_gpu.int8, device="cuda")
    handle.fill_random(b[1:], 5, -5, 9)
    got = b.cpu().numpy()
    np.testing.assert_array_equal(got[1:], oracle.fill_random_i8(1000, 5, -5, 9))
    assert got[0] == 0


@pytest.mark.parametrize("shape", [(1, 1), (3, 5), (64, 300), (257, 4096), (2048, 4096), (7, 1028),
                                   (4, 2052), (5, 8192), (3, 16384), (2, 16388), (3, 4098)])
def test_quantize_rows(handle, torch_gpu, oracle, rng, shape):
    x = rng.normal(size=shape).astype(np.float32)
    x[0] = 0.0   # zero row
    if shape[1] >= 4:
        x[-1, :4] = [1.5, -1.5, 3.0, -3.0]
    q, s = handle.quantize_rows_i8(torch_gpu.from_numpy(x).cuda())
    qe, se = oracle.quantize_rows_i8(x)
    np.testing.assert_array_equal(s.cpu().numpy(), se)
    np.testing.assert_array_equal(q.cpu().numpy(), qe)


@pytest.mark.parametrize("pad", [4, 1])
def test_quantize_rows_of_a_wider_matrix(handle, torch_gpu, oracle, rng, pad):
    """Rows with a leading dimension above the column count: a multiple of 4 keeps the
    16-byte-piece kernel, any other falls back to the element-wise one; same bits."""
    rows, cols = 33, 1024
    wide = rng.normal(size=(rows, cols + pad)).astype(np.float32) * 3
    xd = torch_gpu.from_numpy(wide).cuda()[:, :cols]
    q, s = handle.quantize_rows_i8(xd)
    qe, se = oracle.quantize_rows_i8(np.ascontiguousarray(wide[:, :cols]))
    np.testing.assert_array_equal(s.cpu().numpy(), se)
    np.testing.assert_array_equal(q.cpu().numpy(), qe)

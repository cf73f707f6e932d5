"""The LDS-tiled kernel at each of its four tile heights (256, 192, 128, 64 rows), chosen by
the host's cost model from the shape: each height must be reachable and give the oracle's
result.  The shapes below assume a 256-CU device (the cost model counts rounds of
workgroups); K is an odd number of 64-byte stages so that the peeled last stage runs too."""
import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu

# (M, N) -> expected tile rows on 256 CUs: the height whose tiles just fill one round
HEIGHTS = [((4096, 4096), 256), ((3072, 4096), 192), ((2048, 4096), 128), ((1024, 4096), 64),
           ((3000, 4096), 192), ((1999, 4080), 128), ((4000, 4080), 256), ((1000, 4080), 64)]


def _skip_unless_256_cus(torch):
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("the expected plans are those of a 256-CU device")


@pytest.mark.parametrize("mn,rows", HEIGHTS)
def test_heights_bf16(handle, torch_gpu, oracle, rng, mn, rows):
    torch = torch_gpu
    _skip_unless_256_cus(torch)
    (M, N), K = mn, 160
    Ab = oracle.f32_to_bf16(rng.standard_normal((M, K)).astype(np.float32))
    Bb = oracle.f32_to_bf16(rng.standard_normal((K, N)).astype(np.float32))
    out = handle.gemm_bf16(to_dev(torch, Ab, "bf16"), to_dev(torch, Bb, "bf16"))
    assert handle.last_plan == (rows, 1), (handle.last_plan, handle.last_kernel)
    ref, S = oracle.gemm_f64(oracle.bf16_to_f32(Ab), oracle.bf16_to_f32(Bb), with_abs=True)
    o = oracle.bf16_to_f32(bits(torch, out)).astype(np.float64)
    assert (np.abs(o - ref) <= error_bound_16(ref, S, K, "bf16")).all()


@pytest.mark.parametrize("layout", [ci.B_KN, ci.B_NK])
@pytest.mark.parametrize("mn,rows", HEIGHTS)
def test_heights_int8(handle, torch_gpu, oracle, rng, mn, rows, layout):
    torch = torch_gpu
    _skip_unless_256_cus(torch)
    (M, N), K = mn, 192
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(N, K) if layout == ci.B_NK else (K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(A, B, b_is_nk=layout == ci.B_NK)
    a, b = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    y = handle.gemm_i8_i32(a, b, layout)
    assert handle.last_plan == (rows, 1), (handle.last_plan, handle.last_kernel)
    np.testing.assert_array_equal(y.cpu().numpy(), acc_ref)
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    out = handle.gemm_i8_dequant(a, b, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                 layout, ci.OUT_BF16)
    assert handle.last_plan == (rows, 1), (handle.last_plan, handle.last_kernel)
    expect = oracle.dequant(acc_ref, sa, sb, out_dtype="bf16", sa_per_row=True, sb_per_col=True)
    np.testing.assert_array_equal(bits(torch, out), expect)


@pytest.mark.parametrize("mn,rows", HEIGHTS)
def test_heights_f32_exact_inputs(handle, torch_gpu, oracle, rng, mn, rows):
    """Inputs from {0, +-0.5, +-1, +-2}: every partial sum is exact, so the expected result
    does not depend on the summation order and the comparison is bit for bit."""
    torch = torch_gpu
    _skip_unless_256_cus(torch)
    (M, N), K = mn, 48
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    A, B = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
    bias = rng.choice(vals, size=N)
    with handle.algo(ci.ALGO_TILE):
        L = handle.linear_f32(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(),
                              torch.from_numpy(bias).cuda(), ci.ACT_RELU).cpu().numpy()
    assert handle.last_plan == (rows, 1), (handle.last_plan, handle.last_kernel)
    np.testing.assert_array_equal(L, oracle.linear_f32(A, B, bias, True))


def test_plan_is_zero_for_other_families(handle, torch_gpu):
    torch = torch_gpu
    x = torch.zeros((4, 1024), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((1024, 1024), dtype=torch.bfloat16, device="cuda")
    handle.gemm_bf16(x, w)
    assert "skinny" in handle.last_kernel and handle.last_plan == (0, 0)

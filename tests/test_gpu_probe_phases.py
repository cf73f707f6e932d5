"""The measurement aids of libcigemm_probe.so (include/cigemm_probe.h).  The instrumented launch
of the tile kernel is the product kernel plus four timestamps per workgroup, so its output must
equal the plain entry point's bit for bit, and the figures it reduces must be self-consistent;
the register-resident loops report their operation counts and plausible cycle counts."""
import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import probe
from gpu_util import to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["bf16", "f16", "i8"])
@pytest.mark.parametrize("M,N,K", [(512, 512, 1024), (300, 272, 1008), (2048, 2048, 2048)])
def test_probe_output_equals_plain_call_and_phases_add_up(handle, torch_gpu, oracle, rng, kind, M, N, K):
    torch = torch_gpu
    if kind != "i8":
        # exact-arithmetic inputs: the plain call may split K or pick another tile height,
        # and only such inputs give the same bits in any summation order
        vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
        narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
        a = to_dev(torch, narrow(rng.choice(vals, size=(M, K))), kind)
        b = to_dev(torch, narrow(rng.choice(vals, size=(K, N))), kind)
        out = torch.zeros((M, N), dtype=a.dtype, device="cuda")
        with handle.algo(ci.ALGO_TILE):
            want = (handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16)(a, b)
    else:
        a = torch.from_numpy(rng.integers(-127, 128, size=(M, K), dtype=np.int8)).cuda()
        b = torch.from_numpy(rng.integers(-127, 128, size=(K, N), dtype=np.int8)).cuda()
        out = torch.zeros((M, N), dtype=torch.int32, device="cuda")
        with handle.algo(ci.ALGO_TILE):
            want = handle.gemm_i8_i32(a, b, ci.B_KN)
    for paired, rows, min_cycles in ((False, 256, 1024), (True, 128, 512)):
        if paired and kind == "f16":
            continue
        out.zero_()
        ph = probe.tile_phases(handle, a, b, out, paired=paired)
        assert handle.last_kernel == "tile_phase_probe"
        assert torch.equal(out.view(torch.uint8), want.view(torch.uint8))
        tiles = -(-M // rows) * -(-N // 256)
        assert ph["workgroups"] == tiles
        assert ph["prologue_us"] > 0 and ph["main_loop_us"] > 0 and ph["epilogue_us"] > 0
        # one workgroup's phases fit inside the launch; the matrix cores cannot issue a stage
        # of the tile in fewer cycles than its matrix instructions take; the clock is plausible
        assert ph["prologue_us"] + ph["main_loop_us"] + ph["epilogue_us"] <= ph["first_start_to_last_end_us"] * 1.001
        assert ph["cycles_per_stage"] >= min_cycles
        assert 0.05 < ph["main_loop_clock_ghz"] < 3.0
        # per die and per unit: the dies' clocks bracket the average, no unit ends after the launch
        assert 0.05 < ph["slowest_xcd_clock_ghz"] <= ph["main_loop_clock_ghz"] * 1.001
        assert ph["main_loop_clock_ghz"] <= ph["fastest_xcd_clock_ghz"] * 1.001 < 3.0
        assert 1 <= ph["units"] <= min(tiles, 256)
        assert 0 < ph["mean_unit_end_us"] <= ph["first_start_to_last_end_us"] * 1.001


def test_probe_same_tile_mode(handle, torch_gpu, oracle, rng):
    """kind + 16: every workgroup computes tile (0, 0); that tile of the output is right."""
    torch = torch_gpu
    M, N, K = 768, 1024, 512
    a = torch.from_numpy(rng.integers(-127, 128, size=(M, K), dtype=np.int8)).cuda()
    b = torch.from_numpy(rng.integers(-127, 128, size=(K, N), dtype=np.int8)).cuda()
    with handle.algo(ci.ALGO_TILE):
        want = handle.gemm_i8_i32(a, b, ci.B_KN)
    out = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    ph = probe.tile_phases(handle, a, b, out, same_tile=True)
    assert ph["workgroups"] == 12
    assert torch.equal(out[:256, :256], want[:256, :256])
    assert not out[256:].any() and not out[:, 256:].any()


def test_probe_nk_192_row_form(handle, torch_gpu, rng):
    """kind 5: the 192-row kernel over N x K int8 weights gives the library's bits."""
    torch = torch_gpu
    M, N, K = 600, 520, 1040
    a = torch.from_numpy(rng.integers(-127, 128, size=(M, K), dtype=np.int8)).cuda()
    b = torch.from_numpy(rng.integers(-127, 128, size=(N, K), dtype=np.int8)).cuda()
    with handle.algo(ci.ALGO_TILE):
        want = handle.gemm_i8_i32(a, b, ci.B_NK)
    out = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    ph = probe.tile_phases(handle, a, b, out, b_nk=True)
    assert torch.equal(out, want)
    assert ph["workgroups"] == -(-M // 192) * -(-N // 256) and ph["cycles_per_stage"] >= 768


def test_probe_rejects_bad_arguments(handle, torch_gpu):
    torch = torch_gpu
    a = torch.zeros((64, 60), dtype=torch.bfloat16, device="cuda")      # K * 2 not a multiple of 16
    b = torch.zeros((60, 64), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
        probe.tile_phases(handle, a, b, out)


def test_matrix_core_probe(handle, torch_gpu):
    """The register-resident loop launches on the handle's stream, reports the operation count of
    one launch, and rejects unknown kinds."""
    import ctypes
    from cudaintro_amd import Status
    lib = probe.load_library()
    ops = probe.mfma(handle, "bf16", True, 10)
    cus = torch_gpu.cuda.get_device_properties(0).multi_processor_count
    assert ops == cus * 4 * 10 * 12 * 32768
    assert probe.mfma(handle, "i8", False, 10) == 2 * ops
    assert probe.mfma(handle, "bf16_16x16", False, 10) == ops // 2
    assert probe.mfma(handle, "i8_16x16", False, 10) == ops
    torch_gpu.cuda.synchronize()
    assert handle.last_kernel == "mfma_probe"
    n = ctypes.c_int64(0)
    assert probe.mfma(handle, "f32", True, 10) == ops // 8
    assert lib.cigemm_probe_mfma(handle.raw, 7, 0, 10, ctypes.byref(n)) == Status.INVALID_VALUE
    assert lib.cigemm_probe_mfma(handle.raw, 0, 0, 0, ctypes.byref(n)) == Status.INVALID_VALUE
    assert lib.cigemm_probe_mfma(handle.raw, 0, 0, 10, None) == Status.SUCCESS
    torch_gpu.cuda.synchronize()


def test_issue_cost_probe(handle, torch_gpu):
    """32 matrix instructions of 8 passes of 4 cycles cannot issue in fewer than 1024 cycles; the
    companions (LDS-DMA, fragment reads, a barrier) can only add to that; bad arguments are
    refused before anything is launched."""
    import ctypes
    from cudaintro_amd import Status
    lib = probe.load_library()
    cus = torch_gpu.cuda.get_device_properties(0).multi_processor_count
    base = probe.issue_cost(handle, 0, 0, False, 4, 2000)
    assert handle.last_kernel == "issue_cost_probe"
    assert 1024 <= base["cycles_per_stage"] < 1100, base
    assert base["cycles_per_stage"] <= base["cycles_per_stage_slowest_wave"]
    assert 0.05 < base["clock_ghz"] < 3.0 and base["launch_us"] > 0
    full = probe.issue_cost(handle, 8, 24, True, cus, 2000)
    assert base["cycles_per_stage"] <= full["cycles_per_stage"] < 4 * 1024, full
    res = (ctypes.c_double * 4)()
    for placement in range(1, 8):
        r = probe.issue_cost(handle, 8, 24, True, cus, 500, placement=placement)
        assert 1024 <= r["cycles_per_stage"] < 4 * 1024, (placement, r)
    # without the matrix instructions the memory instructions show what they take by themselves;
    # a DMA source larger than the vector L1 costs no less than one it holds
    alone = probe.issue_cost(handle, 8, 24, True, cus, 500, mfma=False)
    alone_l2 = probe.issue_cost(handle, 8, 24, True, cus, 500, mfma=False, src_kib_per_wave=32)
    assert 0 < alone["cycles_per_stage"] < 4 * 1024 and 0 < alone_l2["cycles_per_stage"] < 8 * 1024
    for bad in ((3, 0, 0, 0, 1, 8, 4, 10), (0, 12, 0, 0, 1, 8, 4, 10), (0, 0, 2, 0, 1, 8, 4, 10),
                (0, 0, 0, 0, 1, 8, 0, 10), (0, 0, 0, 0, 1, 8, cus + 1, 10), (0, 0, 0, 0, 1, 8, 4, 0),
                (8, 24, 1, 8, 1, 8, 4, 10), (4, 24, 1, 1, 1, 8, 4, 10), (8, 24, 1, 3, 0, 8, 4, 10),
                (0, 0, 0, 0, 2, 8, 4, 10), (0, 0, 0, 0, 1, 4, 4, 10), (0, 0, 0, 0, 1, 2048, 4, 10)):
        assert lib.cigemm_probe_issue_cost(handle.raw, *bad, res) == Status.INVALID_VALUE
    assert lib.cigemm_probe_issue_cost(handle.raw, 0, 0, 0, 0, 1, 8, 4, 10, None) == Status.INVALID_VALUE
    # more DMA source than the handle's workspace holds: refused, nothing launched
    assert lib.cigemm_probe_issue_cost(handle.raw, 8, 24, 1, 0, 1, 1024, cus, 10, res) == Status.NOT_SUPPORTED

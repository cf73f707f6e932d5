"""The instrumented launch of the tile kernel (cigemm_probe_tile_phases): it is the product
kernel plus four timestamps per workgroup, so its output must equal the plain entry point's
bit for bit, and the figures it reduces must be self-consistent."""
import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import to_dev

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("kind", ["bf16", "i8"])
@pytest.mark.parametrize("M,N,K", [(512, 512, 1024), (300, 272, 1008), (2048, 2048, 2048)])
def test_probe_output_equals_plain_call_and_phases_add_up(handle, torch_gpu, oracle, rng, kind, M, N, K):
    torch = torch_gpu
    if kind == "bf16":
        # exact-arithmetic inputs: the plain call may split K or pick another tile height,
        # and only such inputs give the same bits in any summation order
        vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
        a = to_dev(torch, oracle.f32_to_bf16(rng.choice(vals, size=(M, K))), "bf16")
        b = to_dev(torch, oracle.f32_to_bf16(rng.choice(vals, size=(K, N))), "bf16")
        out = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
        with handle.algo(ci.ALGO_TILE):
            want = handle.gemm_bf16(a, b)
    else:
        a = torch.from_numpy(rng.integers(-127, 128, size=(M, K), dtype=np.int8)).cuda()
        b = torch.from_numpy(rng.integers(-127, 128, size=(K, N), dtype=np.int8)).cuda()
        out = torch.zeros((M, N), dtype=torch.int32, device="cuda")
        with handle.algo(ci.ALGO_TILE):
            want = handle.gemm_i8_i32(a, b, ci.B_KN)
    for paired, rows, min_cycles in ((False, 256, 1024), (True, 128, 512)):
        out.zero_()
        ph = handle.probe_tile_phases(a, b, out, paired=paired)
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


def test_probe_rejects_bad_arguments(handle, torch_gpu):
    torch = torch_gpu
    a = torch.zeros((64, 60), dtype=torch.bfloat16, device="cuda")      # K * 2 not a multiple of 16
    b = torch.zeros((60, 64), dtype=torch.bfloat16, device="cuda")
    out = torch.zeros((64, 64), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ci.CigemmError, match="NOT_SUPPORTED"):
        handle.probe_tile_phases(a, b, out)

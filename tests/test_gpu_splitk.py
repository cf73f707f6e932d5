"""Split-K runs of the tile kernel (few output tiles, long K): partial sums per K range in the
handle's workspace, then one reduction launch with the real epilogue."""
import re

import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu

SHAPES = [(33, 512, 2048), (64, 1024, 4096), (100, 264, 1024), (256, 2048, 8192), (300, 256, 1536)]


@pytest.mark.parametrize("kind", ["bf16", "f16"])
@pytest.mark.parametrize("shape", SHAPES)
def test_splitk_16bit(handle, torch_gpu, oracle, rng, kind, shape):
    torch = torch_gpu
    M, N, K = shape
    narrow = oracle.f32_to_bf16 if kind == "bf16" else oracle.f32_to_f16
    widen = oracle.bf16_to_f32 if kind == "bf16" else oracle.f16_to_f32
    Ab = narrow(rng.standard_normal((M, K)).astype(np.float32))
    Bb = narrow(rng.standard_normal((K, N)).astype(np.float32))
    fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
    out = torch.full((M + 2, N + 8), 3.0, dtype=torch.bfloat16 if kind == "bf16" else torch.float16,
                     device="cuda")
    for _ in range(2):      # the workspace is reused: a second call must not see stale partials
        fn(to_dev(torch, Ab, kind), to_dev(torch, Bb, kind), out=out[:M, :N])
        if K >= 2048:
            assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
        assert "_mfma_" in handle.last_kernel
        ref, S = oracle.gemm_f64(widen(Ab), widen(Bb), with_abs=True)
        o = widen(bits(torch, out))
        assert (np.abs(o[:M, :N].astype(np.float64) - ref) <= error_bound_16(ref, S, K, kind)).all()
        assert (o[M:] == 3.0).all() and (o[:, N:] == 3.0).all()


@pytest.mark.parametrize("layout", [ci.B_KN, ci.B_NK])
@pytest.mark.parametrize("shape", [(33, 512, 2048), (64, 1024, 4096), (100, 272, 1024), (256, 2048, 8192)])
def test_splitk_int8(handle, torch_gpu, oracle, rng, layout, shape):
    torch = torch_gpu
    M, N, K = shape
    A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
    B = rng.integers(-127, 128, size=(N, K) if layout == ci.B_NK else (K, N), dtype=np.int8)
    acc_ref = oracle.gemm_i8_i32(A, B, b_is_nk=layout == ci.B_NK)
    a, b = torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()
    y = handle.gemm_i8_i32(a, b, layout)
    if K >= 2048:      # short K: the plan may well keep one K range
        assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
    assert "_mfma_" in handle.last_kernel
    np.testing.assert_array_equal(y.cpu().numpy(), acc_ref)
    sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
    sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
    for out_type, ot in (("f32", ci.OUT_F32), ("bf16", ci.OUT_BF16)):
        out, acc = handle.gemm_i8_dequant(a, b, torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(),
                                          layout, ot, dump_acc=True)
        if K >= 2048:
            assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
        np.testing.assert_array_equal(acc.cpu().numpy(), acc_ref)
        expect = oracle.dequant(acc_ref, sa, sb, out_dtype=out_type, sa_per_row=True, sb_per_col=True)
        got = bits(torch, out) if out_type == "bf16" else out.cpu().numpy()
        np.testing.assert_array_equal(got, expect)


def test_splitk_f32_and_exact_inputs(handle, torch_gpu, oracle, rng):
    torch = torch_gpu
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    M, N, K = 256, 512, 4096
    A, B = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
    bias = rng.choice(vals, size=N)
    with handle.algo(ci.ALGO_TILE):
        C = handle.gemm_f32(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda()).cpu().numpy()
        assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
        np.testing.assert_array_equal(C, oracle.gemm_f32(A, B))
        L = handle.linear_f32(torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(),
                              torch.from_numpy(bias).cuda(), ci.ACT_RELU).cpu().numpy()
        assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
        np.testing.assert_array_equal(L, oracle.linear_f32(A, B, bias, True))


def test_large_shapes_do_not_split(handle, torch_gpu):
    a = torch_gpu.zeros((2048, 2048), dtype=torch_gpu.bfloat16, device="cuda")
    handle.gemm_bf16(a, a)
    rows, splits = handle.last_plan
    assert splits == 1 and not handle.last_kernel.endswith("_splitk")
    # the name carries the plan: tile rows and waves per workgroup
    assert re.fullmatch(rf"bf16_mfma_{rows}x256x32_w[48]_ring4", handle.last_kernel), handle.last_kernel


@pytest.mark.parametrize("kind", ["bf16", "i8"])
def test_splitk_workspace_reuse_with_alternating_inputs(handle, torch_gpu, oracle, rng, kind):
    """Two different problems of one shape, called X, Y, X, Y on one handle: a partial sum left
    in the workspace by the previous call would belong to the other problem and show.  The
    expected values come from the oracle (exact-arithmetic inputs: any summation order gives
    the same bits)."""
    torch = torch_gpu
    M, N, K = 64, 1024, 4096
    probs = []
    for _ in range(2):
        if kind == "bf16":
            vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
            A, B = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
            probs.append((to_dev(torch, oracle.f32_to_bf16(A), "bf16"), to_dev(torch, oracle.f32_to_bf16(B), "bf16"),
                          oracle.f32_to_bf16(oracle.gemm_f32(A, B))))
        else:
            A = rng.integers(-127, 128, size=(M, K), dtype=np.int8)
            B = rng.integers(-127, 128, size=(K, N), dtype=np.int8)
            probs.append((torch.from_numpy(A).cuda(), torch.from_numpy(B).cuda(), oracle.gemm_i8_i32(A, B)))
    assert not np.array_equal(probs[0][2], probs[1][2])
    for i in range(6):
        a, b, want = probs[i & 1]
        if kind == "bf16":
            got = bits(torch, handle.gemm_bf16(a, b))
        else:
            got = handle.gemm_i8_i32(a, b, ci.B_KN).cpu().numpy()
        assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
        np.testing.assert_array_equal(got, want, err_msg=f"call {i}")


def test_handle_recovers_after_a_failed_launch(torch_gpu, oracle, rng):
    """A split-K kernel that did not run to its end leaves arrival counters or exchange words
    non-zero.  The state is forged from the host here (a copy into the workspace; every kernel
    runs normally): a handle marked as a failed launch marks it clears them by itself before
    its next GEMM, and cigemmResetWorkspace does it on request."""
    from cudaintro_amd import probe
    torch = torch_gpu
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    cases = []
    # four K ranges per slab (partials and arrival counters); two ranges (one exchange word per
    # pair of outputs)
    for (M, N, K) in ((8, 8192, 8192), (4, 13824, 5120)):
        x = to_dev(torch, oracle.f32_to_bf16(rng.choice(vals, size=(M, K))), "bf16")
        w = to_dev(torch, oracle.f32_to_bf16(rng.choice(vals, size=(K, N)) * (rng.random((K, N)) < 0.1)), "bf16")
        cases.append((x, w))
    with ci.Handle() as h:
        want = []
        for x, w in cases:
            want.append(h.gemm_bf16(x, w).clone())
            assert "skinny" in h.last_kernel, h.last_kernel
        torch.cuda.synchronize()

        def run_all():
            outs = []
            for x, w in cases:
                y = torch.full((x.shape[0], w.shape[1]), 3.0, dtype=torch.bfloat16, device="cuda")
                outs.append(h.gemm_bf16(x, w, out=y))
            torch.cuda.synchronize()
            return outs

        # the forged state matters: without a reset the same calls come out wrong (no kernel
        # waits on these words, so nothing can hang: an output is left unwritten or mis-summed)
        probe.dirty_workspace(h, 8192, 7, mark_dirty=False)
        assert not all(torch.equal(a, b) for a, b in zip(run_all(), want))
        h.reset_workspace()
        assert all(torch.equal(a, b) for a, b in zip(run_all(), want))
        # what a call ending in CIGEMM_STATUS_EXECUTION_FAILED records: cleared without being asked
        probe.dirty_workspace(h, 8192, 7, mark_dirty=True)
        assert all(torch.equal(a, b) for a, b in zip(run_all(), want))
        assert all(torch.equal(a, b) for a, b in zip(run_all(), want))


def test_full_rounds_then_a_planned_remainder(handle, torch_gpu, oracle, rng):
    """Several rounds of tiles whose row tiles do not divide the unit count (6 x 43 tiles of 256
    rows): the columns of the full rounds run as 256-row tiles, the last tile column as a second
    launch of 64-row tiles over K ranges with its own reduction.  Exact-arithmetic inputs: bit
    for bit the CPU loop, for bf16 and for int8 with per-row x per-column scales (whose column
    scales must move with the column offset of the second launch)."""
    torch = torch_gpu
    if torch.cuda.get_device_properties(0).multi_processor_count != 256:
        pytest.skip("the expected plan is that of a 256-CU device")
    M, N, K = 1536, 11008, 1024
    vals = np.array([0, 0.5, -0.5, 1, -1, 2, -2], np.float32)
    A, B = rng.choice(vals, size=(M, K)), rng.choice(vals, size=(K, N))
    out = handle.gemm_bf16(to_dev(torch, oracle.f32_to_bf16(A), "bf16"), to_dev(torch, oracle.f32_to_bf16(B), "bf16"))
    assert re.fullmatch(r"bf16_mfma_256\+\d+x256x32_w4\+w\d_ring4(_splitk)?", handle.last_kernel), handle.last_kernel
    np.testing.assert_array_equal(bits(torch, out), oracle.f32_to_bf16(oracle.gemm_f32(A, B)))
    K8 = 4096
    A8 = rng.integers(-127, 128, size=(M, K8), dtype=np.int8)
    for nk in (False, True):
        B8 = rng.integers(-127, 128, size=(N, K8) if nk else (K8, N), dtype=np.int8)
        sa = rng.uniform(1e-3, 5e-2, M).astype(np.float32)
        sb = rng.uniform(1e-3, 5e-2, N).astype(np.float32)
        layout = ci.B_NK if nk else ci.B_KN
        y = handle.gemm_i8_dequant(torch.from_numpy(A8).cuda(), torch.from_numpy(B8).cuda(),
                                   torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda(), layout, ci.OUT_BF16)
        assert re.fullmatch(r"i8_mfma_256\+\d+x256x64_w\d\+w\d_ring4_(kn|nk)_dequant(_splitk)?", handle.last_kernel), \
            handle.last_kernel
        assert handle.last_kernel.endswith("_splitk"), handle.last_kernel
        acc = oracle.gemm_i8_i32(A8, B8, b_is_nk=nk)
        expect = oracle.dequant(acc, sa, sb, out_dtype="bf16", sa_per_row=True, sb_per_col=True)
        np.testing.assert_array_equal(bits(torch, y), expect)

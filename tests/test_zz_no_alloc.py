"""cigemm_gemm_bf16_static: the decode-shape bf16 GEMM that allocates nothing (no handle, its
split-K scratch in a fixed device array inside the library), through the C ABI, against
cigemm_gemm_bf16 on the same arguments.  Same kernel, same K ranges: the outputs must be
identical bit for bit.  Two calls in a row share the device array, the second smaller."""
import ctypes

import numpy as np
import pytest

import cudaintro_amd as ci
from cudaintro_amd import workloads as wl
from gpu_util import bits, error_bound_16, to_dev

pytestmark = pytest.mark.gpu


def test_static_entry_matches_handle_entry_two_calls(handle, torch_gpu, oracle):
    torch = torch_gpu
    # first call: 32 column slabs x 8 K ranges fill 8 MiB of the array; second call: smaller
    # in every dimension, 4 slabs x 16 ranges, over what the first call left behind
    for (M, N, K) in [(8, 8192, 8192), (3, 1024, 2048)]:
        xb, wb = wl.normal_16bit(M, N, K, seed=4 + M, kind="bf16", sigma_b=0.02)
        x, w = to_dev(torch, xb, "bf16"), to_dev(torch, wb, "bf16")
        y = torch.full((M + 2, N), 7.0, dtype=torch.bfloat16, device="cuda")
        ci.gemm_bf16_static(x, w, out=y[:M])
        with handle.algo(ci.ALGO_SKINNY):
            y_ref = handle.gemm_bf16(x, w)
        assert "skinny" in handle.last_kernel
        got = bits(torch, y)
        np.testing.assert_array_equal(got[:M], bits(torch, y_ref))
        assert (got[M:] == oracle.f32_to_bf16(np.float32(7.0))).all()
        # and against the fp64 checker on the rounded inputs
        ref, S = oracle.gemm_f64(oracle.bf16_to_f32(xb), oracle.bf16_to_f32(wb), with_abs=True)
        err = np.abs(oracle.bf16_to_f32(got[:M]).astype(np.float64) - ref)
        assert (err <= error_bound_16(ref, S, K, "bf16")).all()


@pytest.mark.parametrize("M,N,K,kernel", [
    (4, 1024, 4128, "32x256_ring8"),        # K % 64 != 0: the barrier kernel, 256-column slabs
    (8, 11008, 4096, "kwaves"),             # 128-column slabs, five K ranges: partials and counters
    (4, 13824, 5120, "kwaves"),             # two K ranges: the exchange words
    (2, 4096, 4096, "kwaves"),              # 64-column slabs
])
def test_static_entry_every_kernel_choice(handle, torch_gpu, M, N, K, kernel):
    torch = torch_gpu
    xb, wb = wl.normal_16bit(M, N, K, seed=40 + M, kind="bf16", sigma_b=0.02)
    x, w = to_dev(torch, xb, "bf16"), to_dev(torch, wb, "bf16")
    with handle.algo(ci.ALGO_SKINNY):
        y_ref = handle.gemm_bf16(x, w)
    assert kernel in handle.last_kernel, handle.last_kernel
    for _ in range(2):
        y = ci.gemm_bf16_static(x, w)
        np.testing.assert_array_equal(bits(torch, y), bits(torch, y_ref))


def test_static_entry_allocates_nothing_and_replays_from_a_graph(handle, torch_gpu):
    """Free device memory is the same before and after warm calls, and a call recorded into a HIP
    graph (after the first call on the device, which looks the array's address up) gives the
    handle entry's bits on every replay, with eager calls of other shapes in between that use the
    same device array."""
    torch = torch_gpu
    M, N, K = 8, 8192, 8192
    xb, wb = wl.normal_16bit(M, N, K, seed=12, kind="bf16", sigma_b=0.02)
    x, w = to_dev(torch, xb, "bf16"), to_dev(torch, wb, "bf16")
    xs, ws = x[:3, :2048].contiguous(), w[:2048, :1024].contiguous()
    with handle.algo(ci.ALGO_SKINNY):
        want = bits(torch, handle.gemm_bf16(x, w))
        want_s = bits(torch, handle.gemm_bf16(xs, ws))
    y = torch.zeros((M, N), dtype=torch.bfloat16, device="cuda")
    ys = torch.zeros((3, 1024), dtype=torch.bfloat16, device="cuda")
    ci.gemm_bf16_static(x, w, out=y)            # first call on the device: address look-up
    ci.gemm_bf16_static(xs, ws, out=ys)
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    for _ in range(5):
        ci.gemm_bf16_static(x, w, out=y)
        ci.gemm_bf16_static(xs, ws, out=ys)
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    np.testing.assert_array_equal(bits(torch, y), want)
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.graph(graph, stream=side):
        ci.gemm_bf16_static(x, w, out=y, stream=side)
    torch.cuda.synchronize()
    for _ in range(4):
        y.zero_()
        ci.gemm_bf16_static(xs, ws, out=ys)     # eager, another shape, same device array
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bits(torch, ys), want_s)
        graph.replay()
        torch.cuda.synchronize()
        np.testing.assert_array_equal(bits(torch, y), want)
    free2, _ = torch.cuda.mem_get_info()
    del graph


def test_static_entry_rejects_what_it_cannot_hold(torch_gpu):
    torch = torch_gpu
    x = torch.zeros((33, 64), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((64, 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ci.CigemmError) as e:
        ci.gemm_bf16_static(x, w)
    assert e.value.status == ci.Status.NOT_SUPPORTED and "maximum" in str(e.value)
    x = torch.zeros((1, 64), dtype=torch.bfloat16, device="cuda")
    w = torch.zeros((64, 16384 + 256), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ci.CigemmError) as e:
        ci.gemm_bf16_static(x, w)
    assert e.value.status == ci.Status.NOT_SUPPORTED and "16384" in str(e.value)
    # a shape outside the kernel's gate, and bad arguments: a code, no launch
    w = torch.zeros((64, 128), dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ci.CigemmError) as e:
        ci.gemm_bf16_static(x, w)
    assert e.value.status == ci.Status.NOT_SUPPORTED
    lib = ci.load_library()
    err = ctypes.create_string_buffer(128)
    st = lib.cigemm_gemm_bf16_static(None, 1, 256, 64, None, 64, None, 256, None, 256, err, 128)
    assert st == ci.Status.INVALID_VALUE and b"null" in err.value
    st = lib.cigemm_gemm_bf16_static(None, 0, 256, 64, None, 64, None, 256, None, 256, None, 0)
    assert st == ci.Status.SUCCESS
    torch.cuda.synchronize()

"""The library's calls record into a HIP graph: every entry point only launches kernels on the
handle's stream (no allocation, no memset node, no synchronisation per call), so a serving loop
can capture a sequence once and replay it.  The graph is replayed several times with eager
work and synchronisations between the replays, and every replay is checked against the eager
results: the split-K kernels leave their arrival counters and workspace ready for the next
launch without host help."""
import numpy as np
import pytest

import cudaintro_amd as ci
from gpu_util import to_dev

pytestmark = pytest.mark.gpu


def test_gemm_sequence_replays_from_a_graph(torch_gpu, oracle, rng):
    torch = torch_gpu
    side = torch.cuda.Stream()
    h = ci.Handle(stream=side)

    def bf(shape, scale=1.0):
        return to_dev(torch, oracle.f32_to_bf16((scale * rng.standard_normal(shape)).astype(np.float32)), "bf16")

    x8, w = bf((8, 2048)), bf((2048, 1024), 0.05)              # skinny kernel, split-K fix-up in the kernel
    a64, b64 = bf((64, 4096)), bf((4096, 1024), 0.05)          # tile kernel, split-K: two launches
    a5, b5 = bf((512, 256)), bf((256, 768))                    # tile kernel, one launch
    xq = torch.from_numpy(rng.integers(-127, 128, size=(4, 1024), dtype=np.int8)).cuda()
    wq = torch.from_numpy(rng.integers(-127, 128, size=(512, 1024), dtype=np.int8)).cuda()
    sx = torch.from_numpy(rng.uniform(1e-3, 1e-2, 4).astype(np.float32)).cuda()
    sw = torch.from_numpy(rng.uniform(1e-3, 1e-2, 512).astype(np.float32)).cuda()
    f1 = torch.from_numpy(rng.uniform(-1, 1, (512, 512)).astype(np.float32)).cuda()
    f2 = torch.from_numpy(rng.uniform(-1, 1, (512, 512)).astype(np.float32)).cuda()
    outs = [torch.empty((8, 1024), dtype=torch.bfloat16, device="cuda"),
            torch.empty((64, 1024), dtype=torch.bfloat16, device="cuda"),
            torch.empty((512, 768), dtype=torch.bfloat16, device="cuda"),
            torch.empty((4, 512), dtype=torch.bfloat16, device="cuda"),
            torch.empty((512, 512), dtype=torch.float32, device="cuda")]
    names = []

    def sequence():
        h.gemm_bf16(x8, w, out=outs[0]); names.append(h.last_kernel)
        h.gemm_bf16(a64, b64, out=outs[1]); names.append(h.last_kernel)
        h.gemm_bf16(a5, b5, out=outs[2]); names.append(h.last_kernel)
        h.gemm_i8_dequant(xq, wq, sx, sw, ci.B_NK, ci.OUT_BF16, out=outs[3]); names.append(h.last_kernel)
        h.gemm_f32(f1, f2, out=outs[4]); names.append(h.last_kernel)

    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        sequence()                                              # eager
    side.synchronize()
    assert "skinny" in names[0] and names[1].endswith("_splitk") and "skinny" in names[3]
    eager = [o.clone() for o in outs]

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):                  # capture on the handle's stream
        sequence()
    for replay in range(4):
        for o in outs:
            o.fill_(float("nan"))
        # eager work on the same handle between the replays: it uses the same workspace
        with torch.cuda.stream(side):
            h.gemm_bf16(a64, b64)
        side.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for k, (o, e) in enumerate(zip(outs, eager)):
            assert torch.equal(o.view(torch.int16) if o.dtype == torch.bfloat16 else o,
                               e.view(torch.int16) if e.dtype == torch.bfloat16 else e), (replay, k, names[k])
    h.close()


def test_two_handles_on_two_streams_do_not_share_state(torch_gpu, oracle, rng):
    """One handle per stream: each owns its split-K workspace and arrival counters, so the two
    streams can run split-K calls at the same time.  Forty calls alternate between the streams
    without a synchronisation in between; every output equals the one computed alone."""
    torch = torch_gpu
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    handles = [ci.Handle(stream=s) for s in streams]

    def bf(shape, scale=1.0):
        return to_dev(torch, oracle.f32_to_bf16((scale * rng.standard_normal(shape)).astype(np.float32)), "bf16")

    # a skinny call (fix-up inside the kernel) and a split-K tile call (two launches) per stream
    work = []
    for _ in streams:
        work.append([(bf((8, 4096)), bf((4096, 1024), 0.05)), (bf((64, 4096)), bf((4096, 1024), 0.05))])
    torch.cuda.synchronize()
    alone = []
    for h, s, jobs in zip(handles, streams, work):
        with torch.cuda.stream(s):
            alone.append([h.gemm_bf16(a, b).clone() for a, b in jobs])
        s.synchronize()
    assert "skinny" in handles[0].last_kernel or "splitk" in handles[0].last_kernel
    outs = [[torch.empty_like(o) for o in res] for res in alone]
    for rep in range(20):
        for i, (h, s, jobs) in enumerate(zip(handles, streams, work)):
            with torch.cuda.stream(s):
                for (a, b), o in zip(jobs, outs[i]):
                    h.gemm_bf16(a, b, out=o)
    torch.cuda.synchronize()
    for res, got in zip(alone, outs):
        for r, g in zip(res, got):
            assert torch.equal(r.view(torch.int16), g.view(torch.int16))
    for h in handles:
        h.close()

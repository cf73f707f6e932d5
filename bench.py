#!/usr/bin/env python3
"""Benchmark of the MI355X quantization-GEMM library.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu] [--reference-seconds S]

Headline (the one JSON line printed last): bf16 GEMM 8192^3, TFLOP/s = 2*M*N*K / time, inputs
resident in HBM before the timed region; one "step" is one GEMM call.  The same line carries
`per_config` (fp16 and int8 at 8192^3, int8 4096^3 with per-tensor dequant, the quantized
linear prefill shape, the skinny decode shapes in GB/s), the `roofline` of the headline
kernel (HIP-event timed on the launch stream) and the `cpu_baseline` (the CPU port of the
reference triple loop timed on a bounded slice of rows of the same problem).

One GPU only: --gpus above 1 exits with a message.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
# The CPU-baseline legs run the oracle's OpenMP loops in this process.  Worker threads that keep
# spinning after a parallel region compete with the HIP runtime's own threads: the launch-bound
# 512^3 call measured 8.9 us after such a leg and 5.9 us without.  Let them sleep instead.
os.environ.setdefault("OMP_WAIT_POLICY", "passive")

# MI355X published dense peaks: 256 CUs x 4 SIMDs x 2.4 GHz x 1024 flop/clk (16-bit), x2 for int8.
PEAK_16BIT_TFLOPS = 2516.6
PEAK_INT8_TOPS = 5033.2
PEAK_FP32_MATRIX_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0


def log(*a):
    print(*a, file=sys.stderr, flush=True)


SETTLE_SECONDS = 0.06


def time_calls(torch, fn, steps, warmup):
    """W untimed calls, then exactly `steps` calls between a synchronize on both sides.
    Returns (wall seconds, HIP-event seconds) for the timed region.

    Before the W warm-up calls the workload runs for SETTLE_SECONDS: each workload follows
    host-side input generation, the GPU has idled meanwhile, and its clocks need some 30 ms of
    work to leave the idle state (a 90 us kernel measured 8 % slow over its first 250
    launches after two idle seconds, and at its steady rate from then on)."""
    t_end = time.perf_counter() + SETTLE_SECONDS
    while time.perf_counter() < t_end:
        for _ in range(8):
            fn()
        torch.cuda.synchronize()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    return wall, e0.elapsed_time(e1) * 1e-3


def median_call_ms(torch, fn, steps):
    """Median over `steps` individually HIP-event-timed calls (each call bracketed by its own
    pair of events on the launch stream)."""
    evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
           for _ in range(steps)]
    for a, b in evs:
        a.record()
        fn()
        b.record()
    torch.cuda.synchronize()
    return float(np.median([a.elapsed_time(b) for a, b in evs]))


def graph_call_us(torch, ci, make_call, calls=24, replays=10):
    """Per-call time of `calls` library calls recorded once into a HIP graph on a side stream
    (with a handle of its own bound to that stream) and replayed: what a serving loop that
    captures its decode step sees, without per-launch host work.  make_call(handle, i) issues
    call number i."""
    side = torch.cuda.Stream()
    h = ci.Handle(stream=side)
    torch.cuda.synchronize()
    with torch.cuda.stream(side):
        for i in range(calls):
            make_call(h, i)                      # eager once: loads code objects
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for i in range(calls):
            make_call(h, i)
    for _ in range(3):
        graph.replay()
    torch.cuda.synchronize()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(replays):
        graph.replay()
    e1.record()
    torch.cuda.synchronize()
    h.close()
    return e0.elapsed_time(e1) * 1e3 / (replays * calls)


def reference_protocol(seconds):
    """The reference's own measurement (quantization/main.cu:8-31, GEMM_*.cu:59-84): the suite
    driver built beside the library, as a child process: 4096^3 per precision, device-side
    fills with the reference's seeds, one warm-up, a wall-clock loop of at least `seconds`
    sampled every 256 launches.  Returns {"BF16": TFLOP/s, ...} or None if it is not built."""
    import re
    import subprocess
    exe = os.path.join(ROOT, "cudaintro_amd", "gemm_suite")
    if not os.path.exists(exe):
        return None
    out = subprocess.run([exe, "--seconds", str(seconds)], capture_output=True, text=True,
                         timeout=60 + 8 * seconds)
    if out.returncode != 0:
        log("[bench] gemm_suite failed: " + out.stderr.strip()[-300:])
        return None
    res = {"seconds_per_precision": seconds, "size": 4096}
    for m in re.finditer(r"Ran (\d+) (\w+) GEMMs in ([\d.]+) s \(([\d.]+) TFLOP/s\)", out.stdout):
        res[m.group(2)] = float(m.group(4))
    return res


def dev16(torch, bits, kind):
    if kind == "bf16":
        return torch.from_numpy(bits.view(np.int16)).cuda().view(torch.bfloat16)
    return torch.from_numpy(bits.view(np.float16)).cuda()


def cpu_baseline_16bit(Ab, Bb, kind, target_seconds=12.0):
    """The CPU port of the reference triple loop (i-j-k, float accumulator) on the first R
    rows of the same problem; cost is exactly linear in rows."""
    import oracle
    from cudaintro_amd import workloads as wl
    A = wl.widen_16bit(Ab, kind)
    B = wl.widen_16bit(Bb, kind)
    M, K = A.shape
    N = B.shape[1]
    threads = oracle.num_threads()
    rows = max(threads, 16)
    probe = np.empty((rows, N), np.float32)
    t0 = time.perf_counter()
    oracle.lib.oracle_gemm_f32_ijk(M, N, K, A.ctypes.data, K, B.ctypes.data, N, probe.ctypes.data,
                                   N, 0, rows)
    dt = time.perf_counter() - t0
    scale = max(1, int(target_seconds / max(dt, 1e-3)))
    rows2 = min(M, rows * scale)
    rows2 -= rows2 % threads
    rows2 = max(rows2, threads)
    out = np.empty((rows2, N), np.float32)
    t0 = time.perf_counter()
    oracle.lib.oracle_gemm_f32_ijk(M, N, K, A.ctypes.data, K, B.ctypes.data, N, out.ctypes.data, N,
                                   0, rows2)
    dt = time.perf_counter() - t0
    tflops = 2.0 * rows2 * N * K / dt / 1e12
    return {"value": tflops, "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "sample": f"first {rows2} of {M} rows of the same {M}x{N}x{K} problem, "
                      f"fp32 i-j-k triple loop, {dt:.1f} s"}


def cpu_rows_baseline(run_rows, M, ops_per_row, unit, what, target_seconds=3.0):
    """Times `run_rows(r)` (the CPU port on the first r rows of the problem; cost is exactly
    linear in rows) on a bounded slice: a probe of a few rows, then as many rows as fit
    `target_seconds`.  Returns the per_config[*].cpu_baseline object and run_rows' last result."""
    import oracle
    threads = oracle.num_threads()
    rows = min(M, max(threads, 8))
    t0 = time.perf_counter()
    run_rows(rows)
    dt = time.perf_counter() - t0
    rows2 = min(M, max(rows, int(rows * target_seconds / max(dt, 1e-4))))
    if rows2 >= threads:
        rows2 -= rows2 % threads
    t0 = time.perf_counter()
    res = run_rows(rows2)
    dt = time.perf_counter() - t0
    return {"value": ops_per_row * rows2 / dt / 1e12, "unit": unit, "cores": min(threads, rows2),
            "kind": "port", "sample": f"first {rows2} of {M} rows of the same problem, {what}, {dt:.2f} s"}, res


def k_sweep(torch, ci, wl, probe, handle, steps, warmup):
    """Per-launch time of the tile kernel at several K for a fixed M x N, and the least-squares
    fit t = rounds * (a + b * stages): `a` is what one output tile costs whatever its K
    (pipeline fill, epilogue, the burst of output stores), `b` the cost of one 64-byte stage
    of k.  Prints one JSON object."""
    res = {}

    def fit(rows, cus=256):
        # rows: (K stages, tiles, seconds per launch)
        x = np.array([[np.ceil(t / cus), np.ceil(t / cus) * st] for st, t, _ in rows], np.float64)
        y = np.array([sec for _, _, sec in rows], np.float64)
        (a, b), *_ = np.linalg.lstsq(x, y, rcond=None)
        return a * 1e6, b * 1e6

    for name, sz, ks in (("int8_kn_dequant_f32_4096x4096", 4096, (1024, 2048, 4096, 8192)),
                         ("int8_kn_raw_i32_8192x8192", 8192, (2048, 4096, 8192)),
                         ("bf16_4096x4096", 4096, (1024, 2048, 4096, 8192)),
                         ("bf16_8192x8192", 8192, (2048, 4096, 8192))):
        kmax = max(ks)
        rows = []
        if name.startswith("int8"):
            Aq, Bq, sa, sb = wl.int8_uniform(sz, sz, kmax, seed=1)
            a, b = torch.from_numpy(Aq).cuda(), torch.from_numpy(Bq).cuda()
            sa_d, sb_d = torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda()
            deq = "dequant" in name
            out = torch.empty((sz, sz), device="cuda", dtype=torch.float32 if deq else torch.int32)
            for K in ks:
                av, bv = a[:, :K], b[:K]
                if deq:
                    fn = lambda: handle.gemm_i8_dequant(av, bv, sa_d, sb_d, ci.B_KN, ci.OUT_F32, out=out)  # noqa: E731
                else:
                    fn = lambda: handle.gemm_i8_i32(av, bv, ci.B_KN, out=out)  # noqa: E731
                _, e = time_calls(torch, fn, steps, warmup)
                rows.append((K // 64, (sz // 256) ** 2, e / steps))
                res.setdefault(name, {})[f"K{K}"] = {"us": e / steps * 1e6, "kernel": handle.last_kernel}
        else:
            Ab, Bb = wl.normal_16bit(sz, sz, kmax, seed=2, kind="bf16")
            a, b = dev16(torch, Ab, "bf16"), dev16(torch, Bb, "bf16")
            out = torch.empty((sz, sz), dtype=torch.bfloat16, device="cuda")
            for K in ks:
                av, bv = a[:, :K], b[:K]
                _, e = time_calls(torch, lambda: handle.gemm_bf16(av, bv, out=out), steps, warmup)
                rows.append((K // 32, (sz // 256) ** 2, e / steps))
                res.setdefault(name, {})[f"K{K}"] = {"us": e / steps * 1e6, "kernel": handle.last_kernel}
        a_us, b_us = fit(rows)
        res[name]["fit"] = {"a_us_per_tile": a_us, "b_us_per_stage": b_us}
        log(f"[k-sweep] {name}: {json.dumps(res[name])}")
        del a, b, out
    # Phases of one instrumented launch while 1, 16, 64, 128, 256 and 1024 workgroups are
    # resident (M = N from 256 to 8192 at K = 4096): the cycles per stage stay, the clock the
    # chip holds under the load does not.
    occ = {}
    r = np.random.Generator(np.random.PCG64(1))
    for kind in ("int8", "bf16"):
        for (Mo, No) in ((256, 256), (1024, 1024), (2048, 2048), (2048, 4096), (4096, 4096), (8192, 8192)):
            if kind == "int8":
                a = torch.from_numpy(r.integers(-127, 128, size=(Mo, 4096), dtype=np.int8)).cuda()
                b = torch.from_numpy(r.integers(-127, 128, size=(4096, No), dtype=np.int8)).cuda()
                o = torch.empty((Mo, No), dtype=torch.int32, device="cuda")
            else:
                a = torch.randn((Mo, 4096), device="cuda").to(torch.bfloat16)
                b = torch.randn((4096, No), device="cuda").to(torch.bfloat16)
                o = torch.empty((Mo, No), dtype=torch.bfloat16, device="cuda")
            for _ in range(20):
                ph = probe.tile_phases(handle, a, b, o)
            occ[f"{kind}_{Mo}x{No}x4096"] = ph
            log(f"[occupancy] {kind} {Mo}x{No}x4096: {json.dumps(ph)}")
            del a, b, o
    print(json.dumps({"k_sweep": res, "occupancy_sweep": occ}), flush=True)


def decode_sweep(torch, ci, handle, steps, warmup):
    """Decode GEMMs (M = 1, 16 and 32) at layer shapes of common decoder models, bf16 K x N and int8
    N x K weights: microseconds per call and weight bytes per second.  Several weight buffers
    are rotated so that the Infinity Cache cannot serve them."""
    shapes = [(4096, 4096), (11008, 4096), (4096, 11008), (12288, 4096), (5120, 5120), (13824, 5120),
              (5120, 13824), (8192, 8192), (28672, 8192), (8192, 28672), (32000, 4096)]
    res = {}
    for (N, K) in shapes:
        for M in (1, 16, 32):
            for kind in ("bf16", "int8"):
                eb = 2 if kind == "bf16" else 1
                nb = max(2, int(700e6 // (N * K * eb)) + 1)
                if kind == "bf16":
                    x = torch.randn((M, K), device="cuda").to(torch.bfloat16)
                    ws = [(torch.randn((K, N), device="cuda") * 0.02).to(torch.bfloat16) for _ in range(nb)]
                    y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
                else:
                    x = torch.randint(-127, 128, (M, K), dtype=torch.int8, device="cuda")
                    ws = [torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda") for _ in range(nb)]
                    y = torch.empty((M, N), dtype=torch.int32, device="cuda")
                it = [0]

                def fn():
                    if kind == "bf16":
                        handle.gemm_bf16(x, ws[it[0] % nb], out=y)
                    else:
                        handle.gemm_i8_i32(x, ws[it[0] % nb], ci.B_NK, out=y)
                    it[0] += 1
                w, e = time_calls(torch, fn, steps, warmup)
                name = f"{kind}_M{M}_N{N}_K{K}"
                res[name] = {"us": e / steps * 1e6, "weight_gbs": N * K * eb * steps / e / 1e9,
                             "kernel": handle.last_kernel}
                log(f"[decode-sweep] {name}: {json.dumps(res[name])}")
                del ws
    print(json.dumps({"decode_sweep": res}), flush=True)


PLAN_SWEEP_SHAPES = {
    # (N, K) of the weights: layer shapes of common decoder models
    "a": [(8192, 8192), (11008, 4096), (4096, 11008), (4096, 4096), (14336, 4096), (4096, 14336)],
    "b": [(5120, 5120), (13824, 5120), (5120, 13824), (6144, 4096), (12288, 4096), (28672, 8192),
          (8192, 28672), (10240, 8192), (2048, 2048), (3072, 8192), (8192, 3072), (7168, 7168),
          (1024, 4096), (16384, 2048), (2048, 16384)],
    "c": [(4096, 4096), (8192, 2048), (2048, 8192), (11008, 4096), (4096, 11008), (1024, 4096),
          (5120, 5120)],
    # not used when the planner's constants were chosen
    "d": [(3584, 3584), (18944, 3584), (3584, 18944), (9216, 4608), (4608, 9216), (6656, 6656)],
    "e": [(3584, 3584), (18944, 3584), (3584, 18944), (6656, 6656)],
}
PLAN_SWEEP_MS = {
    "a": (33, 64, 65, 128, 129, 192, 256, 257, 384, 512, 768, 1024, 1536, 2048),
    "b": (40, 72, 96, 128, 160, 200, 256, 320, 448, 512, 640, 896, 1024, 1280, 2048),
    "c": (40, 64, 96, 128, 192, 256, 384, 512, 768, 1024, 2048),
    "d": (48, 100, 144, 224, 288, 352, 480, 576, 704, 960, 1152, 1792),
    "e": (48, 100, 144, 224, 288, 352, 480, 576, 704, 960, 1152, 1792),
}
PLAN_SWEEP_KINDS = {"a": ("bf16", "i8nk"), "b": ("bf16", "i8nk"), "c": ("f32", "i8kn"),
                    "d": ("bf16", "i8nk"), "e": ("f32", "i8kn")}


def plan_sweep(torch, ci, probe, handle, sets, out_path):
    """Evidence for the tile kernel's planner: for every problem of the chosen sets (batch sizes
    between the decode kernels' and one full round of 256-row tiles) the library's own plan and
    every imposed (tile rows, K ranges) plan are timed; prints, per problem, how much slower the
    library's choice is than the best plan timed, and writes all timings as JSON."""
    def timed(fn, steps, warm):
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e3

    out = []
    for st in sets:
        for kind in PLAN_SWEEP_KINDS[st]:
            eb = {"bf16": 2, "f32": 4}.get(kind, 1)
            for (N, K) in PLAN_SWEEP_SHAPES[st]:
                nb = max(2, min(6, (600 << 20) // (K * N * eb)))   # rotated: no cache holds them
                if kind == "bf16":
                    ws = [(torch.randn((K, N), device="cuda") * 0.02).to(torch.bfloat16) for _ in range(nb)]
                elif kind == "f32":
                    ws = [torch.randn((K, N), device="cuda") * 0.02 for _ in range(nb)]
                else:
                    shape = (N, K) if kind == "i8nk" else (K, N)
                    ws = [torch.randint(-127, 128, shape, dtype=torch.int8, device="cuda") for _ in range(nb)]
                for M in PLAN_SWEEP_MS[st]:
                    if kind == "bf16":
                        x = torch.randn((M, K), device="cuda").to(torch.bfloat16)
                        y = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
                    elif kind == "f32":
                        x = torch.randn((M, K), device="cuda")
                        y = torch.empty((M, N), dtype=torch.float32, device="cuda")
                    else:
                        x = torch.randint(-127, 128, (M, K), dtype=torch.int8, device="cuda")
                        y = torch.empty((M, N), dtype=torch.int32, device="cuda")
                    it = [0]

                    def fn():
                        w = ws[it[0] % nb]
                        it[0] += 1
                        if kind == "bf16":
                            handle.gemm_bf16(x, w, out=y)
                        elif kind == "f32":
                            handle.gemm_f32(x, w, out=y)
                        else:
                            handle.gemm_i8_i32(x, w, ci.B_NK if kind == "i8nk" else ci.B_KN, out=y)
                    probe.force_tile_plan(handle, 0)
                    own = timed(fn, 60, 10)
                    own_kernel, own_plan = handle.last_kernel, handle.last_plan
                    plans = {}
                    if own_plan[0]:     # the tile kernel serves this problem
                        for rows in (64, 128, 192, 256):
                            if rows > 64 and rows - 64 >= M:
                                continue
                            for sp in (1, 2, 3, 4, 5, 6, 7, 8, 10, 12, 16, 20, 24, 32):
                                probe.force_tile_plan(handle, rows, sp)
                                fn()
                                torch.cuda.synchronize()
                                pl = handle.last_plan
                                key = f"{pl[0]}x{pl[1]}"
                                tiles = -(-M // rows) * -(-N // 256) * pl[1]
                                if key in plans or (tiles > 768 and pl[1] > 1):
                                    continue
                                plans[key] = round(timed(fn, 40, 10), 1)
                        probe.force_tile_plan(handle, 0)
                    rec = dict(kind=kind, M=M, N=N, K=K, own_us=round(own, 1), own_kernel=own_kernel,
                               own_plan=list(own_plan), plans=plans)
                    if plans:
                        rec["best"] = min(plans, key=plans.get)
                        rec["best_us"] = plans[rec["best"]]
                        log(f"[plan-sweep] {kind} M={M} N={N} K={K}: own {own_plan[0]}x{own_plan[1]} "
                            f"{own:.1f} us | best {rec['best']} {rec['best_us']:.1f} us | "
                            f"{100 * (own / rec['best_us'] - 1):+.1f} %")
                    out.append(rec)
                del ws
    losses = [r["own_us"] / r["best_us"] - 1 for r in out if r["plans"]]
    summary = {"problems": len(losses), "mean_loss": sum(losses) / max(1, len(losses)),
               "max_loss": max(losses, default=0.0),
               "over_5_percent": sum(1 for v in losses if v > 0.05),
               "over_10_percent": sum(1 for v in losses if v > 0.10)}
    if out_path:
        with open(out_path, "w") as f:
            json.dump(out, f)
    print(json.dumps({"plan_sweep": summary}), flush=True)


ONLY_WORKLOADS = ("bf16_8192", "fp16_8192", "int8_8192", "int8_8192_nk", "int8_4096_dequant_f32",
                  "int8_linear_2048x11008x4096_dequant_bf16", "fp32_4096")


def only_workload(torch, ci, wl, handle, name, steps, warmup):
    """One of the matrix-core-bound workloads of the benchmark by itself (same inputs, same
    protocol), for profiler runs whose statistics should cover one kernel: prints one JSON
    object with its rate, time per call and kernel."""
    if name in ("bf16_8192", "fp16_8192"):
        kind = "bf16" if name.startswith("bf16") else "f16"
        M = N = K = 8192
        a_b, b_b = wl.normal_16bit(M, N, K, seed=2, kind=kind)
        a, b = dev16(torch, a_b, kind), dev16(torch, b_b, kind)
        c = torch.empty((M, N), dtype=a.dtype, device="cuda")
        gemm = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
        fn, unit, peak = (lambda: gemm(a, b, out=c)), "TFLOP/s", PEAK_16BIT_TFLOPS
    elif name in ("int8_8192", "int8_8192_nk"):
        M = N = K = 8192
        Aq, Bq, _, _ = wl.int8_uniform(M, N, K, seed=1)
        nk = name.endswith("_nk")
        a = torch.from_numpy(Aq).cuda()
        b = torch.from_numpy(np.ascontiguousarray(Bq.T) if nk else Bq).cuda()
        c = torch.empty((M, N), dtype=torch.int32, device="cuda")
        fn, unit, peak = (lambda: handle.gemm_i8_i32(a, b, ci.B_NK if nk else ci.B_KN, out=c)), "TOP/s", PEAK_INT8_TOPS
    elif name == "int8_4096_dequant_f32":
        M = N = K = 4096
        Aq, Bq, sa, sb = wl.int8_uniform(M, N, K, seed=1)
        a, b, sa_d, sb_d = (torch.from_numpy(v).cuda() for v in (Aq, Bq, sa, sb))
        c = torch.empty((M, N), dtype=torch.float32, device="cuda")
        fn, unit, peak = (lambda: handle.gemm_i8_dequant(a, b, sa_d, sb_d, ci.B_KN, ci.OUT_F32, out=c)), "TOP/s", PEAK_INT8_TOPS
    elif name == "int8_linear_2048x11008x4096_dequant_bf16":
        M, K, N = 2048, 4096, 11008
        Xq, sx, Wq, sw = wl.quantized_linear(M, K, N, seed=3)
        a, b, sa_d, sb_d = (torch.from_numpy(v).cuda() for v in (Xq, Wq, sx, sw))
        c = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")
        fn, unit, peak = (lambda: handle.gemm_i8_dequant(a, b, sa_d, sb_d, ci.B_NK, ci.OUT_BF16, out=c)), "TOP/s", PEAK_INT8_TOPS
    else:
        M = N = K = 4096
        Af, Bf = wl.fp32_uniform(M, N, K, seed=0)
        a, b = torch.from_numpy(Af).cuda(), torch.from_numpy(Bf).cuda()
        c = torch.empty((M, N), dtype=torch.float32, device="cuda")
        fn, unit, peak = (lambda: handle.gemm_f32(a, b, out=c)), "TFLOP/s", PEAK_FP32_MATRIX_TFLOPS
    wall, ev = time_calls(torch, fn, steps, warmup)
    ops = wl.gemm_ops(M, N, K)
    rate = ops * steps / ev / 1e12
    print(json.dumps({"only": name, "value": rate, "unit": unit, "frac_of_peak": rate / peak, "peak": peak,
                      "ms": ev / steps * 1e3, "ms_wall": wall / steps * 1e3, "steps": steps, "warmup": warmup,
                      "ops_per_call": ops, "kernel": handle.last_kernel}), flush=True)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # The chip's power controller takes some 15 launches of this size to settle (the first
    # two run at boost clocks, the next dozen 15-25 % slower); the defaults time the settled
    # state, which is also what the reference's >= 10 s loop measures.
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--no-extra", action="store_true", help="headline workload only")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--reference-seconds", type=float, default=10.0,
                    help="time budget per precision of the reference's own protocol (10, as in "
                         "quantization/GEMM_bf16.cu:63; 0 skips that leg)")
    ap.add_argument("--size", type=int, default=8192, help="headline M=N=K (default 8192)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy a few times (reference point for "
                         "the FETCH_SIZE / WRITE_SIZE counters under rocprofv3 --pmc)")
    ap.add_argument("--k-sweep", action="store_true",
                    help="instead of the benchmark: time the tile kernel at several K per M x N and "
                         "fit its fixed cost per tile and its cost per stage")
    ap.add_argument("--only", choices=ONLY_WORKLOADS,
                    help="instead of the benchmark: this one workload by itself (for profiler runs)")
    ap.add_argument("--decode-sweep", action="store_true",
                    help="instead of the benchmark: decode GEMMs (M = 1, 16, 32) at layer shapes of common "
                         "decoder models, bf16 and int8")
    ap.add_argument("--plan-sweep", metavar="SETS",
                    help="instead of the benchmark: time every (tile rows, K ranges) plan of the tile "
                         "kernel against the library's own choice over the problem sets named "
                         "(letters of a..e; e.g. 'ab')")
    ap.add_argument("--plan-sweep-out", default="", help="with --plan-sweep: write all timings here (JSON)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1",
              file=sys.stderr)
        sys.exit(2)

    import torch
    import cudaintro_amd as ci
    from cudaintro_amd import probe
    from cudaintro_amd import workloads as wl

    if not torch.cuda.is_available():
        print("bench.py needs an MI355X; there is no CPU fallback", file=sys.stderr)
        sys.exit(1)
    handle = ci.Handle()
    if args.k_sweep:
        k_sweep(torch, ci, wl, probe, handle, args.steps, args.warmup)
        return
    if args.decode_sweep:
        decode_sweep(torch, ci, handle, args.steps, args.warmup)
        return
    if args.plan_sweep:
        if any(c not in PLAN_SWEEP_SHAPES for c in args.plan_sweep):
            print("--plan-sweep takes letters of: " + "".join(PLAN_SWEEP_SHAPES), file=sys.stderr)
            sys.exit(2)
        plan_sweep(torch, ci, probe, handle, args.plan_sweep, args.plan_sweep_out)
        return
    if args.only:
        only_workload(torch, ci, wl, handle, args.only, args.steps, args.warmup)
        return
    n = args.size
    per_config = {}
    mfma_probe = {}

    if args.copy_calibration:
        src = torch.ones(1 << 28, dtype=torch.float32, device="cuda")   # 1 GiB
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---- headline: bf16 n^3 -------------------------------------------------------------
    log(f"[bench] generating bf16 {n}^3 inputs")
    Ab, Bb = wl.normal_16bit(n, n, n, seed=2, kind="bf16")
    A, B = dev16(torch, Ab, "bf16"), dev16(torch, Bb, "bf16")
    C = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
    wall, ev = time_calls(torch, lambda: handle.gemm_bf16(A, B, out=C), args.steps, args.warmup)
    kernel = handle.last_kernel
    ops = wl.gemm_ops(n, n, n)
    value = ops * args.steps / wall / 1e12
    achieved = ops * args.steps / ev / 1e12
    log(f"[bench] bf16 {n}^3: {value:.1f} TFLOP/s wall, {achieved:.1f} TFLOP/s by HIP events, "
        f"kernel {kernel}")
    roofline = {"bound": "mfma", "achieved": achieved, "peak": PEAK_16BIT_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / PEAK_16BIT_TFLOPS, "traffic": None, "kernel": kernel,
                "avg_kernel_ms": ev / args.steps * 1e3}
    # where the time of one launch goes, from timestamps inside the kernel (one instrumented
    # launch of the same kernel, taken while the chip is in the state the timed loop left)
    for _ in range(3):
        phases = probe.tile_phases(handle, A, B, C)
    roofline["phases"] = phases
    # every compute die holds its own clock and gets the same number of tiles: the launch ends
    # with the slowest die, the average unit earlier
    roofline["xcd_clock_ghz_slowest_fastest"] = [phases["slowest_xcd_clock_ghz"], phases["fastest_xcd_clock_ghz"]]
    roofline["mean_unit_end_over_launch_end"] = phases["mean_unit_end_us"] / phases["first_start_to_last_end_us"]
    roofline["clock_ghz_main_loop_this_run"] = phases["main_loop_clock_ghz"]
    # matrix-core issue cycles of one 64-byte stage of the 256 x 256 tile: 32 instructions of 8
    # passes of 4 cycles per wave
    roofline["mfma_issue_fraction_of_main_loop"] = 1024.0 / phases["cycles_per_stage"]
    roofline["median_kernel_ms"] = median_call_ms(torch, lambda: handle.gemm_bf16(A, B, out=C),
                                                  max(50, args.steps))
    # What the 4.3 x re-read operand traffic costs: the same instrumented launch with every
    # workgroup on output tile (0, 0), so that no operand read leaves the L2.
    for _ in range(3):
        ph_l2 = probe.tile_phases(handle, A, B, C, same_tile=True)
    roofline["all_operands_in_l2"] = {
        "launch_us": ph_l2["first_start_to_last_end_us"], "launch_us_real_tiles": phases["first_start_to_last_end_us"],
        "main_loop_us": ph_l2["main_loop_us"], "cycles_per_stage": ph_l2["cycles_per_stage"],
        "clock_ghz": ph_l2["main_loop_clock_ghz"],
        "what": "one instrumented launch with every workgroup computing output tile (0, 0)"}
    handle.gemm_bf16(A, B, out=C)
    # HBM-side bytes per launch and the counter decomposition of the same kernel are not
    # measurable from inside this process: they come from the rocprofv3 --pmc runs of this
    # same command summarised in profiles/ (the file says which runs).  Everything copied from
    # there sits under `from_profiles`, apart from `traffic`, whose source is named beside it.
    traffic_file = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    prof = json.load(open(traffic_file)) if os.path.exists(traffic_file) else {}
    if prof:
        roofline["traffic"] = prof.get(f"bf16_{n}")
        roofline["traffic_source"] = "profiles/hbm_traffic.json"
        roofline["from_profiles"] = {key: prof[f"bf16_{n}_{key}"] for key in ("mfma_busy", "clock_ghz")
                                     if f"bf16_{n}_{key}" in prof}
        roofline["from_profiles"]["source"] = "profiles/hbm_traffic.json (rocprofv3 --pmc runs, not this run)"

    # What a register-resident loop of the same matrix instruction sustains in this run on
    # random operand bits, with no memory traffic at all: the chip is power limited on such
    # data, so this, not the datasheet peak, is the ceiling a kernel can approach.
    def sustained(kind):
        ops_box = [0]

        def fn_probe():
            ops_box[0] = probe.mfma(handle, kind, True, 20000)
        _, e_probe = time_calls(torch, fn_probe, 20, 10)
        return ops_box[0] * 20 / e_probe / 1e12

    roofline["sustained_peak"] = sustained("bf16")
    roofline["sustained_peak_what"] = ("register-resident v_mfma_f32_32x32x16_bf16 loop, random "
                                       "operand bits, one wave per SIMD, same run")
    roofline["frac_of_sustained"] = achieved / roofline["sustained_peak"]
    # The metric is quoted per dtype: bf16, fp16 and int8 at n^3, each against its datasheet peak
    # and against what the register-resident loop of its matrix instruction sustained in this run.
    per_dtype = {"bf16": {"achieved": achieved, "unit": "TFLOP/s", "peak": PEAK_16BIT_TFLOPS,
                          "frac": achieved / PEAK_16BIT_TFLOPS, "sustained_peak": roofline["sustained_peak"],
                          "frac_of_sustained": roofline["frac_of_sustained"], "kernel": kernel,
                          "ms": ev / args.steps * 1e3, "cycles_per_stage": phases["cycles_per_stage"],
                          "clock_ghz_main_loop": phases["main_loop_clock_ghz"]}}
    roofline["per_dtype"] = per_dtype

    cpu = None
    if not args.no_cpu:
        log("[bench] CPU baseline (port of the reference triple loop) ...")
        cpu = cpu_baseline_16bit(Ab, Bb, "bf16")
        log(f"[bench] CPU: {cpu['value'] * 1e3:.2f} GFLOP/s on {cpu['cores']} threads")
    del A, B, C

    if not args.no_extra:
        def run16(kind):
            a_b, b_b = wl.normal_16bit(n, n, n, seed=2, kind=kind)
            a, b = dev16(torch, a_b, kind), dev16(torch, b_b, kind)
            c = torch.empty((n, n), dtype=a.dtype, device="cuda")
            fn = handle.gemm_bf16 if kind == "bf16" else handle.gemm_f16
            w, e = time_calls(torch, lambda: fn(a, b, out=c), args.steps, args.warmup)
            t = ops * args.steps / e / 1e12
            res = {"tflops": t, "frac_of_peak": t / PEAK_16BIT_TFLOPS, "peak": PEAK_16BIT_TFLOPS,
                   "ms": e / args.steps * 1e3, "kernel": handle.last_kernel}
            for _ in range(3):
                res["phases"] = probe.tile_phases(handle, a, b, c)
            return res

        log(f"[bench] fp16 {n}^3")
        r16 = run16("f16")
        per_config[f"fp16_{n}"] = r16
        sp = sustained("f16")
        per_dtype["fp16"] = {"achieved": r16["tflops"], "unit": "TFLOP/s", "peak": PEAK_16BIT_TFLOPS,
                             "frac": r16["frac_of_peak"], "sustained_peak": sp,
                             "frac_of_sustained": r16["tflops"] / sp, "kernel": r16["kernel"], "ms": r16["ms"],
                             "cycles_per_stage": r16["phases"]["cycles_per_stage"],
                             "clock_ghz_main_loop": r16["phases"]["main_loop_clock_ghz"]}
        log(f"[bench] fp16 {n}^3: {json.dumps(per_dtype['fp16'])}")

        # The same headline problem on the two-workgroups-per-unit form of the tile kernel
        # (libcigemm_probe.so; the library never chooses it): more matrix instructions issued
        # per cycle, a lower clock under the power limit.  Recorded as the measured reason for
        # the default's choice.
        a_b, b_b = wl.normal_16bit(n, n, n, seed=2, kind="bf16")
        a, b = dev16(torch, a_b, "bf16"), dev16(torch, b_b, "bf16")
        c = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
        w, e = time_calls(torch, lambda: probe.gemm16_paired(handle, a, b, out=c), args.steps, args.warmup)
        name_p = handle.last_kernel
        t = ops * args.steps / e / 1e12
        for _ in range(3):
            ph = probe.tile_phases(handle, a, b, c, paired=True)
        per_config[f"bf16_{n}_two_workgroups_per_unit"] = {
            "tflops": t, "frac_of_peak": t / PEAK_16BIT_TFLOPS, "peak": PEAK_16BIT_TFLOPS,
            "ms": e / args.steps * 1e3, "ms_over_default": e / args.steps / (ev / args.steps),
            "kernel": name_p, "phases": ph,
            # two workgroups share a unit's matrix cores: 2 x 512 issue cycles per stage pair
            "mfma_issue_fraction_of_main_loop": 1024.0 / ph["cycles_per_stage"]}
        del a, b, c

        # shapes that do not fill the kernel's units: a K whose last 64-byte stage holds one
        # 16-byte piece, an N whose last column tile holds 8 columns (no alignment cliff wanted)
        for (Mx, Nx, Kx) in ((n, n, n + 8), (n, n + 8, n)):
            a_b, b_b = wl.normal_16bit(Mx, Nx, Kx, seed=2, kind="bf16")
            a, b = dev16(torch, a_b, "bf16"), dev16(torch, b_b, "bf16")
            c = torch.empty((Mx, Nx), dtype=torch.bfloat16, device="cuda")
            steps_x = max(10, args.steps // 4)
            w, e = time_calls(torch, lambda: handle.gemm_bf16(a, b, out=c), steps_x, max(5, args.warmup // 4))
            t = wl.gemm_ops(Mx, Nx, Kx) * steps_x / e / 1e12
            per_config[f"bf16_{Mx}x{Nx}x{Kx}"] = {"tflops": t, "frac_of_peak": t / PEAK_16BIT_TFLOPS,
                                                   "peak": PEAK_16BIT_TFLOPS, "ms": e / steps_x * 1e3,
                                                   "ms_over_aligned": e / steps_x / (ev / args.steps),
                                                   "kernel": handle.last_kernel}
            del a, b, c
        # shapes no aligned kernel takes (odd N: rows of B and C at every 2-byte alignment; odd K:
        # rows of A): the any-shape matrix-core kernel, and the scalar kernel it took them from
        for (Mx, Nx, Kx) in ((4096, 4095, 4096), (4096, 4096, 4095)):
            a_b, b_b = wl.normal_16bit(Mx, Nx, Kx, seed=2, kind="bf16")
            a, b = dev16(torch, a_b, "bf16"), dev16(torch, b_b, "bf16")
            c = torch.empty((Mx, Nx), dtype=torch.bfloat16, device="cuda")
            w, e = time_calls(torch, lambda: handle.gemm_bf16(a, b, out=c), 20, 5)
            t = wl.gemm_ops(Mx, Nx, Kx) * 20 / e / 1e12
            name_a = handle.last_kernel
            with handle.algo(ci.ALGO_GENERIC):
                w, e_s = time_calls(torch, lambda: handle.gemm_bf16(a, b, out=c), 3, 1)
            per_config[f"bf16_{Mx}x{Nx}x{Kx}_unaligned"] = {
                "tflops": t, "frac_of_peak": t / PEAK_16BIT_TFLOPS, "peak": PEAK_16BIT_TFLOPS,
                "ms": e / 20 * 1e3, "kernel": name_a,
                "scalar_kernel_tflops": wl.gemm_ops(Mx, Nx, Kx) * 3 / e_s / 1e12}
            del a, b, c
        per_config[f"bf16_{n}"] = {"tflops": achieved, "frac_of_peak": achieved / PEAK_16BIT_TFLOPS,
                                   "peak": PEAK_16BIT_TFLOPS, "ms": ev / args.steps * 1e3,
                                   "kernel": kernel}
        # the same for fp32: every dimension odd
        Mx, Nx, Kx = 4095, 4097, 4099
        a = torch.from_numpy(np.random.Generator(np.random.PCG64(5)).uniform(-1, 1, (Mx, Kx)).astype(np.float32)).cuda()
        b = torch.from_numpy(np.random.Generator(np.random.PCG64(6)).uniform(-1, 1, (Kx, Nx)).astype(np.float32)).cuda()
        c = torch.empty((Mx, Nx), dtype=torch.float32, device="cuda")
        w, e = time_calls(torch, lambda: handle.gemm_f32(a, b, out=c), 10, 3)
        name_a = handle.last_kernel
        with handle.algo(ci.ALGO_GENERIC):
            w, e_s = time_calls(torch, lambda: handle.gemm_f32(a, b, out=c), 3, 1)
        t = wl.gemm_ops(Mx, Nx, Kx) * 10 / e / 1e12
        per_config[f"fp32_{Mx}x{Nx}x{Kx}_unaligned"] = {
            "tflops": t, "frac_of_peak": t / PEAK_FP32_MATRIX_TFLOPS, "peak": PEAK_FP32_MATRIX_TFLOPS,
            "ms": e / 10 * 1e3, "kernel": name_a,
            "scalar_kernel_tflops": wl.gemm_ops(Mx, Nx, Kx) * 3 / e_s / 1e12}
        del a, b, c

        def run_i8(name, M, N, K, make, dequant):
            log(f"[bench] {name}")
            Aq, Bq, sa, sb, lay, out_t = make()
            a, b = torch.from_numpy(Aq).cuda(), torch.from_numpy(Bq).cuda()
            if dequant:
                sa_d, sb_d = torch.from_numpy(sa).cuda(), torch.from_numpy(sb).cuda()
                out = torch.empty((M, N), device="cuda",
                                  dtype=torch.bfloat16 if out_t == ci.OUT_BF16 else torch.float32)
                fn = lambda: handle.gemm_i8_dequant(a, b, sa_d, sb_d, lay, out_t, out=out)  # noqa: E731
            else:
                out = torch.empty((M, N), dtype=torch.int32, device="cuda")
                fn = lambda: handle.gemm_i8_i32(a, b, lay, out=out)  # noqa: E731
            w, e = time_calls(torch, fn, args.steps, args.warmup)
            t = wl.gemm_ops(M, N, K) * args.steps / e / 1e12
            per_config[name] = {"tops": t, "frac_of_peak": t / PEAK_INT8_TOPS, "peak": PEAK_INT8_TOPS,
                                "ms": e / args.steps * 1e3, "kernel": handle.last_kernel}
            if lay == ci.B_KN or "192x256" in handle.last_kernel:
                # phases of the same tile kernel with raw int32 output (the same bytes per
                # output element as the fp32 dequantized one)
                o32 = out if not dequant else torch.empty((M, N), dtype=torch.int32, device="cuda")
                for _ in range(3):
                    ph = probe.tile_phases(handle, a, b, o32, b_nk=lay == ci.B_NK)
                per_config[name]["phases_raw_i32_out"] = ph
                del o32
            if not args.no_cpu:
                # the int8 -> int32 twin of the reference's CPU loop on a slice of rows, timed;
                # the same rows of the GPU result are compared with it (bit-exact or not)
                import oracle
                nk = lay == ci.B_NK
                base, acc_ref = cpu_rows_baseline(lambda r: oracle.gemm_i8_i32(Aq[:r], Bq, b_is_nk=nk), M,
                                                  2.0 * N * K, "TOP/s", "int8 x int8 -> int32 loop")
                r = acc_ref.shape[0]
                if dequant:
                    bf = out_t == ci.OUT_BF16
                    want = oracle.dequant(acc_ref, sa[:r] if sa.size > 1 else sa, sb,
                                          out_dtype="bf16" if bf else "f32",
                                          sa_per_row=sa.size > 1, sb_per_col=sb.size > 1)
                    got = out[:r].view(torch.int16).cpu().numpy().view(np.uint16) if bf else out[:r].cpu().numpy()
                else:
                    want, got = acc_ref, out[:r].cpu().numpy()
                base["gpu_rows_bit_exact"] = bool(np.array_equal(got, want))
                per_config[name]["cpu_baseline"] = base

        def mk_square(sz, seed):
            def f():
                Aq, Bq, sa, sb = wl.int8_uniform(sz, sz, sz, seed=seed)
                return Aq, Bq, sa, sb, ci.B_KN, ci.OUT_F32
            return f

        def mk_linear():
            Xq, sx, Wq, sw = wl.quantized_linear(2048, 4096, 11008, seed=3)
            return Xq, Wq, sx, sw, ci.B_NK, ci.OUT_BF16

        def mk_square_nk(sz, seed):
            def f():
                Aq, Bq, sa, sb = wl.int8_uniform(sz, sz, sz, seed=seed)
                return Aq, np.ascontiguousarray(Bq.T), sa, sb, ci.B_NK, ci.OUT_F32
            return f

        run_i8(f"int8_{n}_raw_i32", n, n, n, mk_square(n, 1), False)
        r8 = per_config[f"int8_{n}_raw_i32"]
        sp = sustained("i8")
        per_dtype["int8"] = {"achieved": r8["tops"], "unit": "TOP/s", "peak": PEAK_INT8_TOPS,
                             "frac": r8["frac_of_peak"], "sustained_peak": sp,
                             "frac_of_sustained": r8["tops"] / sp, "kernel": r8["kernel"], "ms": r8["ms"],
                             "cycles_per_stage": r8["phases_raw_i32_out"]["cycles_per_stage"],
                             "clock_ghz_main_loop": r8["phases_raw_i32_out"]["main_loop_clock_ghz"]}
        log(f"[bench] int8 {n}^3: {json.dumps(per_dtype['int8'])}")
        # the same problem with the weights stored N x K (each output channel contiguous: the
        # layout of the quantized linear layer)
        run_i8(f"int8_{n}_nk_raw_i32", n, n, n, mk_square_nk(n, 1), False)
        run_i8("int8_4096_dequant_f32", 4096, 4096, 4096, mk_square(4096, 1), True)
        run_i8("int8_linear_2048x11008x4096_dequant_bf16", 2048, 11008, 4096, mk_linear, True)

        # fp32 anchor and the reference's own 4096^3
        for sz in (512, 4096):
            Af, Bf = wl.fp32_uniform(sz, sz, sz, seed=0)
            a, b = torch.from_numpy(Af).cuda(), torch.from_numpy(Bf).cuda()
            c = torch.empty((sz, sz), dtype=torch.float32, device="cuda")
            steps = args.steps if sz == 512 else max(2, args.steps // 4)
            w, e = time_calls(torch, lambda: handle.gemm_f32(a, b, out=c), steps, max(2, args.warmup // 4))
            t = wl.gemm_ops(sz, sz, sz) * steps / e / 1e12
            per_config[f"fp32_{sz}"] = {"tflops": t, "frac_of_peak": t / PEAK_FP32_MATRIX_TFLOPS,
                                        "peak": PEAK_FP32_MATRIX_TFLOPS, "ms": e / steps * 1e3,
                                        "kernel": handle.last_kernel}
            if sz == 512 and not args.no_cpu:
                # the reference's own CPU check at its own size: matrixMulCPU, one thread
                import oracle
                t0 = time.perf_counter()
                oracle.matrixMulCPU(Af, Bf)
                dt = time.perf_counter() - t0
                per_config["fp32_512"]["cpu_matrixMulCPU_one_thread_ms"] = dt * 1e3
                per_config["fp32_512"]["cpu_gflops"] = wl.gemm_ops(sz, sz, sz) / dt / 1e9

        # MLP forward layers of the reference's MNIST demo on the fp32 GEMM with the fused
        # bias + ReLU epilogue (MNIST/mnist_nn.h:12-15: batch 20000, 784 -> 512 -> 10)
        r = np.random.Generator(np.random.PCG64(5))
        for name, (Mb, Kb, Nb), act in (("mnist_hidden_20000x784x512_bias_relu", (20000, 784, 512), ci.ACT_RELU),
                                        ("mnist_output_20000x512x10_bias", (20000, 512, 10), ci.ACT_NONE)):
            x = torch.from_numpy(r.uniform(0, 1, size=(Mb, Kb)).astype(np.float32)).cuda()
            wgt = torch.from_numpy((r.standard_normal((Kb, Nb)) * 0.05).astype(np.float32)).cuda()
            bias = torch.from_numpy(r.standard_normal(Nb).astype(np.float32)).cuda()
            o = torch.empty((Mb, Nb), dtype=torch.float32, device="cuda")
            w_, e = time_calls(torch, lambda: handle.linear_f32(x, wgt, bias, act, out=o), args.steps, args.warmup)
            t = wl.gemm_ops(Mb, Nb, Kb) * args.steps / e / 1e12
            per_config[name] = {"tflops": t, "frac_of_peak": t / PEAK_FP32_MATRIX_TFLOPS,
                                "peak": PEAK_FP32_MATRIX_TFLOPS, "ms": e / args.steps * 1e3,
                                "kernel": handle.last_kernel}
            if Nb <= 16:   # a narrow output layer streams its activations: HBM is the bound
                nbytes = 4 * (Mb * Kb + Kb * Nb + Mb * Nb + Nb)
                gbs = nbytes * args.steps / e / 1e9
                per_config[name].update({"gbs": gbs, "frac_of_hbm_peak": gbs / PEAK_HBM_GBS,
                                         "bytes": nbytes})

        # the steps either side of the int8 GEMM: device fills and the absmax row quantizer
        # (HBM-bound; algorithmic bytes = what is written, resp. 4 + 1 bytes per element)
        fb = torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda")
        w_, e = time_calls(torch, lambda: handle.fill_random(fb, 0x1234), args.steps, args.warmup)
        gbs = fb.numel() * 2 * args.steps / e / 1e9
        per_config["fill_random_bf16_8192x8192"] = {"gbs": gbs, "frac_of_peak": gbs / PEAK_HBM_GBS,
                                                    "peak": PEAK_HBM_GBS, "us": e / args.steps * 1e6,
                                                    "bytes": fb.numel() * 2}
        del fb
        # C2 is one round of tiles whose 64 MiB of fp32 output all units store at the same time,
        # with the matrix cores idle: its floor on this chip is the main loop plus the output's
        # bytes at the rate the fill kernel (a pure store stream) reached in this run.
        c2 = per_config["int8_4096_dequant_f32"]
        out_bytes = 4096 * 4096 * 4
        floor_us = c2["phases_raw_i32_out"]["main_loop_us"] + out_bytes / (gbs * 1e9) * 1e6
        c2["floor_us"] = floor_us
        c2["floor_what"] = ("main loop of the instrumented launch + 64 MiB of output at the fill kernel's "
                            "write rate of this run")
        c2["frac_of_floor"] = floor_us / (c2["ms"] * 1e3)
        c2["floor_tops"] = wl.gemm_ops(4096, 4096, 4096) / floor_us / 1e6
        for rows_q, cols_q in ((2048, 4096), (8192, 8192)):
            xq_ = torch.from_numpy(r.standard_normal((rows_q, cols_q)).astype(np.float32)).cuda()
            outq = (torch.empty((rows_q, cols_q), dtype=torch.int8, device="cuda"),
                    torch.empty((rows_q,), dtype=torch.float32, device="cuda"))
            w_, e = time_calls(torch, lambda: handle.quantize_rows_i8(xq_, out=outq), args.steps, args.warmup)
            nbytes = rows_q * cols_q * 5 + rows_q * 4
            gbs = nbytes * args.steps / e / 1e9
            per_config[f"quantize_rows_i8_{rows_q}x{cols_q}"] = {
                "gbs": gbs, "frac_of_peak": gbs / PEAK_HBM_GBS, "peak": PEAK_HBM_GBS,
                "us": e / args.steps * 1e6, "bytes": nbytes}
            del xq_, outq

        # skinny decode shapes: HBM-bound.  Rotate over several distinct weight buffers so the
        # working set (> 256 MB) cannot sit in the Infinity Cache between calls.
        for M in (1, 8, 32):
            xb, wb = wl.skinny_bf16(M, 8192, 8192, seed=4)
            x = dev16(torch, xb, "bf16")
            ws = [dev16(torch, wb, "bf16") for _ in range(4)]
            y = torch.empty((M, 8192), dtype=torch.bfloat16, device="cuda")
            it = [0]

            def fn():
                handle.gemm_bf16(x, ws[it[0] & 3], out=y)
                it[0] += 1
            steps = max(args.steps, 40)
            w, e = time_calls(torch, fn, steps, max(4, args.warmup))
            nbytes = wl.skinny_bytes(M, 8192, 8192, 2, 2, 2)
            gbs = nbytes * steps / e / 1e9
            per_config[f"skinny_bf16_M{M}"] = {"gbs": gbs, "frac_of_peak": gbs / PEAK_HBM_GBS,
                                               "peak": PEAK_HBM_GBS, "us": e / steps * 1e6,
                                               "bytes": nbytes, "kernel": handle.last_kernel}
            if not args.no_cpu:
                # the reference's fp32 i-j-k loop on the widened inputs, on the rows that fit
                import oracle
                xf, wf = wl.widen_16bit(xb, "bf16"), wl.widen_16bit(wb, "bf16")
                base, cpu_rows = cpu_rows_baseline(lambda r: oracle.gemm_f32_ijk(xf, wf, 0, r)[:r], M,
                                                   2.0 * 8192 * 8192, "TFLOP/s", "fp32 i-j-k triple loop",
                                                   target_seconds=2.0)
                r = cpu_rows.shape[0]
                got = wl.bf16_bits_to_f32(y[:r].view(torch.int16).cpu().numpy().view(np.uint16))
                base["gpu_rows_max_abs_diff"] = float(np.abs(got - cpu_rows).max())
                base["cpu_rows_rms"] = float(np.sqrt(np.mean(cpu_rows.astype(np.float64) ** 2)))
                per_config[f"skinny_bf16_M{M}"]["cpu_baseline"] = base
            del ws
            xq, sx, wq, sw = wl.skinny_int8(M, 8192, 8192, seed=4)
            xd, sxd, swd = torch.from_numpy(xq).cuda(), torch.from_numpy(sx).cuda(), torch.from_numpy(sw).cuda()
            wqs = [torch.from_numpy(wq).cuda() for _ in range(6)]
            yo = torch.empty((M, 8192), dtype=torch.bfloat16, device="cuda")

            def fn8():
                handle.gemm_i8_dequant(xd, wqs[it[0] % 6], sxd, swd, ci.B_NK, ci.OUT_BF16, out=yo)
                it[0] += 1
            w, e = time_calls(torch, fn8, steps, max(6, args.warmup))
            nbytes = wl.skinny_bytes(M, 8192, 8192, 1, 1, 2, scale_bytes=4 * 8192)
            gbs = nbytes * steps / e / 1e9
            per_config[f"skinny_int8_M{M}"] = {"gbs": gbs, "frac_of_peak": gbs / PEAK_HBM_GBS,
                                               "peak": PEAK_HBM_GBS, "us": e / steps * 1e6,
                                               "bytes": nbytes, "kernel": handle.last_kernel}
            if not args.no_cpu:
                import oracle
                base, acc_ref = cpu_rows_baseline(lambda r: oracle.gemm_i8_i32(xq[:r], wq, b_is_nk=True), M,
                                                  2.0 * 8192 * 8192, "TOP/s", "int8 x int8 -> int32 loop",
                                                  target_seconds=1.0)
                r = acc_ref.shape[0]
                want = oracle.dequant(acc_ref, sx[:r] if M > 1 else sx, sw, out_dtype="bf16",
                                      sa_per_row=M > 1, sb_per_col=True)
                base["gpu_rows_bit_exact"] = bool(np.array_equal(
                    yo[:r].view(torch.int16).cpu().numpy().view(np.uint16), want))
                per_config[f"skinny_int8_M{M}"]["cpu_baseline"] = base
            del wqs
            # the same weights stored K x N (the reference's own operand order): the decode
            # kernel with 128-column slabs and four K ranges per slab
            wts = [torch.from_numpy(np.ascontiguousarray(wq.T)).cuda() for _ in range(6)]

            def fn8kn():
                handle.gemm_i8_dequant(xd, wts[it[0] % 6], sxd, swd, ci.B_KN, ci.OUT_BF16, out=yo)
                it[0] += 1
            w, e = time_calls(torch, fn8kn, steps, max(6, args.warmup))
            per_config[f"skinny_int8_kn_M{M}"] = {"gbs": nbytes * steps / e / 1e9,
                                                  "frac_of_peak": nbytes * steps / e / 1e9 / PEAK_HBM_GBS,
                                                  "peak": PEAK_HBM_GBS, "us": e / steps * 1e6,
                                                  "bytes": nbytes, "kernel": handle.last_kernel}
            del wts
        # small-batch shapes between the decode and the square configurations: few output
        # tiles and a long K, run as split-K (weights still dominate the traffic)
        for M in (64, 256):
            xb, wb = wl.skinny_bf16(M, 8192, 8192, seed=4)
            x = dev16(torch, xb, "bf16")
            ws = [dev16(torch, wb, "bf16") for _ in range(4)]
            y = torch.empty((M, 8192), dtype=torch.bfloat16, device="cuda")
            it = [0]

            def fnb():
                handle.gemm_bf16(x, ws[it[0] & 3], out=y)
                it[0] += 1
            w, e = time_calls(torch, fnb, args.steps, args.warmup)
            nbytes = wl.skinny_bytes(M, 8192, 8192, 2, 2, 2)
            per_config[f"batch_bf16_M{M}"] = {"tflops": wl.gemm_ops(M, 8192, 8192) * args.steps / e / 1e12,
                                              "gbs": nbytes * args.steps / e / 1e9,
                                              "frac_of_peak": nbytes * args.steps / e / 1e9 / PEAK_HBM_GBS,
                                              "peak": PEAK_HBM_GBS, "us": e / args.steps * 1e6,
                                              "bytes": nbytes, "kernel": handle.last_kernel}
            del ws

        # The decode shape once more, as replays of a captured HIP graph.  Last of the GEMM
        # measurements on purpose: once a second stream has been used in the process, eager
        # launches on the first one take a few microseconds longer each.
        xb, wb = wl.skinny_bf16(1, 8192, 8192, seed=4)
        x = dev16(torch, xb, "bf16")
        ws = [dev16(torch, wb, "bf16") for _ in range(4)]
        y = torch.empty((1, 8192), dtype=torch.bfloat16, device="cuda")
        per_config["skinny_bf16_M1"]["us_replayed_from_graph"] = graph_call_us(
            torch, ci, lambda hh, i: hh.gemm_bf16(x, ws[i & 3], out=y))
        del ws
        xq, sx, wq, sw = wl.skinny_int8(1, 8192, 8192, seed=4)
        xd, sxd, swd = torch.from_numpy(xq).cuda(), torch.from_numpy(sx).cuda(), torch.from_numpy(sw).cuda()
        wqs = [torch.from_numpy(wq).cuda() for _ in range(6)]
        yo = torch.empty((1, 8192), dtype=torch.bfloat16, device="cuda")
        per_config["skinny_int8_M1"]["us_replayed_from_graph"] = graph_call_us(
            torch, ci, lambda hh, i: hh.gemm_i8_dequant(xd, wqs[i % 6], sxd, swd, ci.B_NK,
                                                        ci.OUT_BF16, out=yo))
        del wqs

        if args.reference_seconds > 0:
            log("[bench] the reference's protocol (gemm_suite, 4096^3) ...")
            torch.cuda.synchronize()
            ref = reference_protocol(args.reference_seconds)
            if ref:
                per_config["reference_protocol_4096"] = ref

        # What the matrix cores sustain with no memory traffic at all, at the clock the chip
        # holds under that load, on constant and on random operand bits.
        probe_res = {}
        for kind in ("bf16", "f16", "i8", "f32"):
            for rnd in (False, True):
                ops_box = [0]

                def fnp():
                    ops_box[0] = probe.mfma(handle, kind, rnd, 5000 if kind == "f32" else 20000)
                w, e = time_calls(torch, fnp, 20, 10)
                probe_res[f"{kind}_{'random' if rnd else 'constant'}_bits"] = ops_box[0] * 20 / e / 1e12
        mfma_probe.update(probe_res)
        # What the other instructions of the tile kernel's stage cost in matrix-core issue time:
        # cycles per 32 matrix instructions (1024 when nothing delays them) with n LDS-DMA
        # instructions, the stage's 24 LDS fragment reads and its barrier added, all units busy.
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        issue = {}

        def ic(key, *a, **kw):
            for _ in range(2):
                r_ic = probe.issue_cost(handle, *a, **kw)
            issue[key] = round(r_ic["cycles_per_stage"], 1)

        for n_dma, n_lds, bar in ((0, 0, 0), (8, 0, 0), (0, 24, 0), (0, 0, 1), (8, 24, 0)):
            ic(f"dma{n_dma}_lds{n_lds}_bar{bar}", n_dma, n_lds, bool(bar), cus, 4000)
        # all three, with the DMA instructions back to back after the barrier (placement 0) and in
        # every second slot (placement 1, what the tile kernel does), sources the L1 holds or not
        ic("dma8_lds24_bar1_back_to_back", 8, 24, True, cus, 4000)
        ic("dma8_lds24_bar1_spread", 8, 24, True, cus, 4000, placement=1)
        ic("dma8_lds24_bar1_spread_l2_source", 8, 24, True, cus, 4000, placement=1, src_kib_per_wave=32)
        ic("dma8_lds24_bar1_spread_one_workgroup", 8, 24, True, 1, 4000, placement=1)
        # the stage's memory instructions without its matrix instructions
        ic("no_mfma_dma8", 8, 0, True, cus, 4000, mfma=False, placement=1, src_kib_per_wave=32)
        ic("no_mfma_lds24", 0, 24, True, cus, 4000, mfma=False)
        ic("no_mfma_dma8_lds24", 8, 24, True, cus, 4000, mfma=False, placement=1, src_kib_per_wave=32)
        mfma_probe["issue_cost_cycles_per_stage"] = issue
        roofline["issue_ceiling"] = 1024.0 / issue["dma8_lds24_bar1_spread_l2_source"]
        roofline["issue_ceiling_what"] = ("1024 matrix-core issue cycles per stage / cycles per stage of a "
                                          "register-resident loop with the stage's 8 LDS-DMA instructions (every "
                                          "second slot, L2 sources), 24 LDS fragment reads and barrier, same run")
        for k, v in per_config.items():
            log(f"[bench]   {k}: {json.dumps(v)}")
        log(f"[bench]   register-resident MFMA loop, T(FL)OP/s: {json.dumps(probe_res)}")
        log(f"[bench]   issue cost, cycles per stage: {json.dumps(issue)}")

    # The line printed last holds the figures; the full per-configuration records (phases, CPU
    # baselines, samples) were logged above.  One entry per configuration: value, unit, fraction
    # of its roofline, time per call, kernel.
    def compact(v):
        if not isinstance(v, dict) or not any(k in v for k in ("tflops", "tops", "gbs")):
            return v
        key = "tflops" if "tflops" in v else "tops" if "tops" in v else "gbs"
        out = {"value": round(v[key], 2), "unit": {"tflops": "TFLOP/s", "tops": "TOP/s", "gbs": "GB/s"}[key],
               "frac_of_peak": round(v["frac_of_peak"], 4)}
        us = v["us"] if "us" in v else v["ms"] * 1e3
        out["us"] = round(us, 2)
        if "kernel" in v:
            out["kernel"] = v["kernel"]
        for extra in ("us_replayed_from_graph", "ms_over_default", "ms_over_aligned", "scalar_kernel_tflops",
                      "floor_us", "frac_of_floor", "cpu_gflops"):
            if extra in v:
                out[extra] = round(v[extra], 4)
        base = v.get("cpu_baseline")
        if base:
            out["cpu"] = {"value": float(f"{base['value']:.4g}"), "unit": base["unit"], "cores": base["cores"]}
            for flag in ("gpu_rows_bit_exact",):
                if flag in base:
                    out["cpu"][flag] = base[flag]
        return out

    line = {
        "metric": "GEMM TFLOPS/TOPS at 8192^3 per dtype (int8/bf16/fp16) + % of MFMA peak",
        "value": value,
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": wall / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"bf16 GEMM M=N=K={n}, N(0,1) inputs rounded to bf16, fp32 accumulate, "
                               "bf16 out, row-major", "M": n, "N": n, "K": n},
        "roofline": roofline,
        "cpu_baseline": cpu,
    }
    # the metric's three dtypes, flat (beside roofline.per_dtype)
    for dt, rec in per_dtype.items():
        pkey = f"{dt}_{n}"
        if f"{pkey}_mfma_busy" in prof:
            rec["from_profiles"] = {"mfma_busy": prof[f"{pkey}_mfma_busy"], "clock_ghz": prof[f"{pkey}_clock_ghz"],
                                    "traffic": prof.get(pkey)}
        unit = "tflops" if dt != "int8" else "tops"
        line[f"{dt}_{n}_{unit}"] = rec["achieved"]
        line[f"{dt}_{n}_frac_of_peak"] = rec["frac"]
        line[f"{dt}_{n}_frac_of_sustained"] = rec["frac_of_sustained"]
        roofline[f"{dt}_{n}_achieved"] = rec["achieved"]
        roofline[f"{dt}_{n}_frac"] = rec["frac"]
    line["per_config"] = {k: compact(v) for k, v in per_config.items()}
    line["mfma_only_probe"] = mfma_probe
    # the BASELINE configurations once more, last on stderr
    for dt, rec in per_dtype.items():
        log(f"[bench] C3/{dt} {n}^3: {rec['achieved']:.1f} {rec['unit']} = {rec['frac'] * 100:.1f} % of "
            f"{rec['peak']:.1f}, {rec['frac_of_sustained'] * 100:.1f} % of the {rec['sustained_peak']:.0f} the chip "
            f"sustains on random bits; {rec['ms']:.4f} ms, {rec['kernel']}")
    for tag, key in (("C1", "fp32_512"), ("C2", "int8_4096_dequant_f32"),
                     ("C4", "int8_linear_2048x11008x4096_dequant_bf16"),
                     ("C5", "skinny_bf16_M1"), ("C5", "skinny_bf16_M8"), ("C5", "skinny_bf16_M32"),
                     ("C5", "skinny_int8_M1"), ("C5", "skinny_int8_M8"), ("C5", "skinny_int8_M32")):
        if key in per_config:
            log(f"[bench] {tag} {key}: {json.dumps(compact(per_config[key]))}")
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()

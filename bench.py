#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload cfg2] [--no-cpu] [--only-headline]

A step is one pass of one workload's kernel over its synthetic input, enqueued
through the C ABI (tts_launch) on torch's current stream, on a plan compiled by
the unchanged Triton frontend.  Inputs live in HBM before the timed region; the
buffers of consecutive steps rotate over enough copies (> 600 MB) that a step
does not find its input in the 256 MB Infinity Cache left by the previous one.
Prints ONE JSON line.  The headline workload is the row softmax, fp32 [4096, 781]
(the second of the five configurations); the other four configs and two steady-state
sizes are reported in "kernels".

Per kernel: `us` = mean kernel duration from HIP events around the timed
launches; `achieved` = algorithmic bytes (or flops) / that duration; `frac` =
achieved / MI355X peak (HBM 8 TB/s, dense bf16 MFMA 2.5 PFLOP/s).  The CPU
baseline is the restatement of the reference's CPU path (oracle/cpu_path.c, one
thread as the reference launcher is single-threaded) on a bounded sample.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
BF16_PEAK_TFLOPS = 2500.0
ROTATE_BYTES = 600e6
RAMP_SECONDS = float(os.environ.get("TTS_BENCH_RAMP_SECONDS", "0.06"))  # sustained-clock warm-up, see time_workload


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="cfg2", help="headline workload: cfg1..cfg5, cfg1_2p28, cfg2_1m")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only-headline", action="store_true", help="time only the headline workload")
    ap.add_argument("--rotating-only", action="store_true",
                    help="skip the same-buffer and frontend passes, so that a kernel trace of this run holds rotating-buffer launches only")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="run a 256 MiB device-to-device copy three times and exit (the known-size kernel that scales FETCH_SIZE/WRITE_SIZE)")
    return ap.parse_args()


class Spy:
    """Records the arguments the Triton launcher hands to the C ABI, so that the
    timed loop can replay the launch without the Python JIT dispatch."""

    def __init__(self):
        from triton_shared_amd.backend import driver as drv
        self.drv = drv
        self.last = None
        orig = drv.HIPLauncher.__call__
        spy = self

        def call(launcher, gx, gy, gz, stream, function, km, lm, eh, xh, *args):
            vals = [drv._device_pointer(args[p], p) if is_ptr else args[p] for p, is_ptr in launcher.slots]
            spy.last = ((gx, gy, gz), vals)
            return orig(launcher, gx, gy, gz, stream, function, km, lm, eh, xh, *args)

        drv.HIPLauncher.__call__ = call


def make_workloads(torch, triton, K):
    """name -> dict(desc, bytes or flops, bound, dtype, make(seed)->(launch_fn, outputs), cpu(sample))"""
    dev = "cuda"
    W = {}

    def vec_add(n):
        def make():
            x, y = torch.rand(n, device=dev), torch.rand(n, device=dev)
            z = torch.empty_like(x)
            return lambda: K.vec_add[(triton.cdiv(n, 1024),)](x, y, z, n, BLOCK=1024)
        return dict(desc=f"vector add fp32 N={n}, BLOCK=1024, grid={triton.cdiv(n, 1024)}", work=12 * n, bound="hbm",
                    dtype="f32", make=make, set_bytes=12 * n)

    def softmax(rows):
        def make():
            x = torch.randn(rows, 781, device=dev)
            o = torch.empty_like(x)
            return lambda: K.row_softmax[(rows,)](o, x, x.stride(0), o.stride(0), 781, BLOCK=1024)
        return dict(desc=f"row softmax fp32 [{rows}, 781], BLOCK=1024 (-inf padded), grid={rows}", work=8 * rows * 781,
                    bound="hbm", dtype="f32", make=make, set_bytes=8 * rows * 781)

    def layernorm():
        M, N = 4096, 8192

        def make():
            x = torch.randn(M, N, device=dev).half()
            w = (1 + 0.1 * torch.randn(N, device=dev)).half()
            b = (0.1 * torch.randn(N, device=dev)).half()
            y = torch.empty_like(x)
            mean = torch.empty(M, dtype=torch.float32, device=dev)
            rstd = torch.empty_like(mean)
            return lambda: K.layer_norm_fwd[(M,)](x, y, w, b, mean, rstd, x.stride(0), N, 1e-5, BLOCK=1024)
        work = 2 * M * N * 2 + 2 * N * 2 + 2 * M * 4
        return dict(desc="LayerNorm fwd fp16 [4096, 8192], BLOCK=1024 looped, fp32 stats", work=work, bound="hbm",
                    dtype="f16", make=make, set_bytes=work)

    def gemm():
        n = 4096

        def make():
            a = (torch.randn(n, n, device=dev) * 0.02).bfloat16()
            b = (torch.randn(n, n, device=dev) * 0.02).bfloat16()
            c = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
            return lambda: K.matmul_tiles[(32 * 32,)](a, b, c, n, n, n, n, 1, n, 1, n, 1, BM=128, BN=128, BK=64, GROUP_M=8)
        return dict(desc="matmul bf16 4096x4096x4096, BM=BN=128 BK=64, fp32 acc, bf16 out", work=2 * n ** 3,
                    bound="mfma", dtype="bf16", make=make, set_bytes=3 * n * n * 2)

    def w8a16():
        M, N, Kd = 16, 28672, 8192

        def make():
            a = torch.randn(M, Kd, device=dev).half()
            w = torch.randint(-127, 128, (Kd, N), dtype=torch.int8, device=dev)
            s = (0.001 + 0.009 * torch.rand(N, device=dev)).half()
            c = torch.empty(M, N, dtype=torch.float16, device=dev)
            return lambda: K.w8a16_matmul[(1, N // 128)](a, w, s, c, M, N, Kd, Kd, 1, N, 1, N, 1, BM=16, BN=128, BK=128)
        work = Kd * N + M * Kd * 2 + N * 2 + M * N * 2
        return dict(desc="W8A16 matmul A fp16 [16, 8192] x W int8 [8192, 28672], fp16 scales, fp32 acc", work=work,
                    bound="hbm", dtype="f16", make=make, set_bytes=work)

    def fused_gelu(n):
        def make():
            x, b = torch.randn(n, device=dev), torch.randn(n, device=dev)
            y = torch.empty(n, device=dev)
            return lambda: K.gelu_tanh_bias[(triton.cdiv(n, 1024),)](x, b, y, n, BLOCK=1024)
        m = 1 << 16
        cpu = lanes((m // 1024,), [m], lambda: [np.random.rand(m).astype(np.float32), np.random.rand(m).astype(np.float32),
                                                np.zeros(m, np.float32)], m / n, f"N={m}")
        return dict(desc=f"fused map y = gelu_tanh(x + b) fp32 N={n}, BLOCK=1024 (19 elementwise ops, compiled with hipRTC)",
                    work=3 * n * 4, bound="hbm", dtype="f32", make=make, set_bytes=3 * n * 4, lanes=cpu)

    def fused_silu(n):
        def make():
            g, u = torch.randn(n, device=dev).half(), torch.randn(n, device=dev).half()
            o = torch.empty(n, dtype=torch.float16, device=dev)
            return lambda: K.silu_mul_f16[(triton.cdiv(n, 1024),)](g, u, o, n, BLOCK=1024)
        m = 1 << 16
        cpu = lanes((m // 1024,), [m], lambda: [np.random.rand(m).astype(np.float16), np.random.rand(m).astype(np.float16),
                                                np.zeros(m, np.float16)], m / n, f"N={m}")
        return dict(desc=f"fused map out = silu(g) * u fp16 N={n}, BLOCK=1024 (10 elementwise ops, compiled with hipRTC)",
                    work=3 * n * 2, bound="hbm", dtype="f16", make=make, set_bytes=3 * n * 2, lanes=cpu)

    def lanes(grid, scalars, arrays, frac, sample):
        """CPU baseline of a workload outside the five configurations: the lane-level oracle on a smaller problem
        made of the same programs.  arrays() -> numpy buffers in pointer-argument order."""
        def run(ttir):
            from oracle import ttir_lanes
            bufs = arrays()
            t0 = time.perf_counter()
            ttir_lanes.Interpreter(ttir).run(grid, [None] * len(bufs) + list(scalars), dict(enumerate(bufs)))
            return time.perf_counter() - t0, frac, sample
        return run

    import numpy as np

    def take_rows(rows, cols):
        def make():
            src = torch.randn(rows, cols, device=dev)
            idx = torch.randint(0, rows, (rows,), device=dev, dtype=torch.int32)
            dst = torch.empty_like(src)
            return lambda: K.take_rows[(triton.cdiv(rows, 4),)](src, idx, dst, rows, cols, src.stride(0), dst.stride(0), BR=4, BC=1024)
        work = 2 * rows * cols * 4 + rows * 4
        r = 256
        cpu = lanes((r // 4,), [r, cols, cols, cols],
                    lambda: [np.random.rand(r, cols).astype(np.float32).reshape(-1), np.random.randint(0, r, r).astype(np.int32),
                             np.zeros(r * cols, np.float32)], r / rows, f"{r} of {rows} rows")
        return dict(desc=f"gather of rows dst[r, :] = src[idx[r], :] fp32 [{rows}, {cols}], 4 rows per program (generic family)",
                    work=work, bound="hbm", dtype="f32", make=make, set_bytes=work, lanes=cpu)

    def row_sums(rows, cols):
        def make():
            x = torch.randn(rows, cols, device=dev)
            out = torch.empty(rows, device=dev)
            br = int(os.environ.get("TTS_BENCH_BR", "4"))
            return lambda: K.row_sums[(triton.cdiv(rows, br),)](x, out, rows, cols, x.stride(0), BR=br, BC=1024)
        work = rows * cols * 4 + rows * 4
        r = 256
        cpu = lanes((r // 4,), [r, cols, cols],
                    lambda: [np.random.rand(r, cols).astype(np.float32).reshape(-1), np.zeros(r, np.float32)], r / rows, f"{r} of {rows} rows")
        return dict(desc=f"row sums of fp32 [{rows}, {cols}], 4 rows per program (generic family, axis reduction)", work=work, bound="hbm",
                    dtype="f32", make=make, set_bytes=work, lanes=cpu)

    def block_cumsum(n):
        def make():
            x = torch.randn(n, device=dev)
            y = torch.empty_like(x)
            return lambda: K.block_cumsum[(triton.cdiv(n, 1024),)](x, y, n, BLOCK=1024)
        m = 1 << 16
        cpu = lanes((m // 1024,), [m], lambda: [np.random.rand(m).astype(np.float32), np.zeros(m, np.float32)], m / n, f"N={m}")
        return dict(desc=f"inclusive prefix sums inside blocks of 1024, fp32 N={n} (generic family, scan)", work=8 * n, bound="hbm",
                    dtype="f32", make=make, set_bytes=8 * n, lanes=cpu)

    def matmul_act(n):
        def make():
            a = (torch.randn(n, n, device=dev) * 0.02).bfloat16()
            b = (torch.randn(n, n, device=dev) * 0.02).bfloat16()
            c = torch.empty(n, n, dtype=torch.bfloat16, device=dev)
            return lambda: K.matmul_leaky_relu[(n // 128, n // 128)](a, b, c, n, n, n, n, n, n, 0.01, BM=128, BN=128, BK=64)
        return dict(desc=f"C = leaky_relu(A @ B) bf16 {n}^3, BM=BN=128 BK=64 (matmul family, the activation compiled into the kernel's epilogue)",
                    work=2 * n ** 3, bound="mfma", dtype="bf16", make=make, set_bytes=3 * n * n * 2)

    def expert_rows(tokens, kd, nd, experts):
        def make():
            a = (torch.randn(tokens, kd, device=dev) * 0.02).bfloat16()
            b = (torch.randn(experts, kd, nd, device=dev) * 0.02).bfloat16()
            c = torch.empty(tokens, nd, dtype=torch.bfloat16, device=dev)
            rows = torch.randperm(tokens, device=dev).int()
            ids = (torch.arange(tokens // 128, device=dev) % experts).int()
            return lambda: K.expert_rows_matmul[(tokens // 128, nd // 128)](a, b, c, rows, ids, tokens, kd, nd, kd, kd * nd, nd, nd, BM=128, BN=128, BK=64)
        return dict(desc=f"mixture-of-experts product bf16: {tokens} rows gathered through an index vector, x [{experts}, {kd}, {nd}] weights picked by a "
                         "loaded expert id per 128 rows (generic family: carried gather offsets, LDS-staged operands, 32x32 MFMA blocks)",
                    work=2 * tokens * kd * nd, bound="mfma", dtype="bf16", make=make, set_bytes=(tokens * kd + experts * kd * nd + tokens * nd) * 2)

    W["cfg1"] = vec_add(98432)
    W["cfg2"] = softmax(4096)
    W["cfg3"] = layernorm()
    W["cfg4"] = gemm()
    W["cfg5"] = w8a16()
    W["cfg1_2p28"] = vec_add(1 << 28)
    W["cfg2_1m"] = softmax(1 << 20)
    W["next_fused_gelu_2p26"] = fused_gelu(1 << 26)
    W["next_fused_silu_2p26"] = fused_silu(1 << 26)
    W["next_matmul_act_4096"] = matmul_act(4096)
    W["next_expert_rows_4096"] = expert_rows(4096, 2048, 2048, 8)
    W["next_take_rows_2p26"] = take_rows(1 << 16, 1024)
    W["next_row_sums_2p26"] = row_sums(1 << 16, 1024)
    W["next_block_cumsum_2p26"] = block_cumsum(1 << 26)
    return W


def time_workload(torch, spy, wl, steps, warmup, rotating_only=False):
    """Returns dict(us, kernel, sets).  Rotates over `sets` independent buffer sets."""
    sets = max(1, min(32, math.ceil(ROTATE_BYTES / wl["set_bytes"])))
    if wl["set_bytes"] > 1e9:
        sets = 1
    launches = []
    plan = None
    for _ in range(sets):
        fn = wl["make"]()
        k = fn()  # compiles on first use, launches once through the full frontend
        plan = k.function
        ttir = k.asm.get("ttir") if hasattr(k, "asm") else None
        grid, vals = spy.last
        launches.append((grid, plan.pack(vals), len(vals), fn))
    torch.cuda.synchronize()
    stream = torch.cuda.current_stream().cuda_stream
    # Warm-up: `warmup` steps at least, and on until the GPU has been busy for RAMP_SECONDS: after an idle
    # period the device takes tens of milliseconds of load to reach its sustained clocks (a 4096^3 GEMM
    # measured 125 us per launch in the first 10 ms of load and 113 us from 30 ms on).
    t_ramp, done = time.perf_counter(), 0
    while done < warmup or time.perf_counter() - t_ramp < RAMP_SECONDS:
        for i in range(max(warmup, 20)):
            g, arr, n, _ = launches[(done + i) % sets]
            plan.launch_packed(g, stream, arr, n)
        done += max(warmup, 20)
        torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for i in range(steps):
        g, arr, n, _ = launches[i % sets]
        plan.launch_packed(g, stream, arr, n)
    stop.record()
    torch.cuda.synchronize()
    wall_us = (time.perf_counter() - t0) * 1e6 / steps
    us = start.elapsed_time(stop) * 1e3 / steps
    if rotating_only:
        kernel = plan.last_kernel
        del launches
        torch.cuda.empty_cache()
        return dict(us=us, hot_us=us, wall_us=wall_us, kernel=kernel, sets=sets, frontend_us=0.0, warmup_steps_run=done, ttir=ttir)
    # same measurement on one buffer set ("hot": inputs may sit in the Infinity Cache), for information
    g, arr, n, _ = launches[0]
    for _ in range(warmup):
        plan.launch_packed(g, stream, arr, n)
    start.record()
    for _ in range(steps):
        plan.launch_packed(g, stream, arr, n)
    stop.record()
    torch.cuda.synchronize()
    hot_us = start.elapsed_time(stop) * 1e3 / steps
    # the same launch through the Triton JIT dispatch (Python overhead included), for information
    fn = launches[0][3]
    t0 = time.perf_counter()
    for _ in range(20):
        fn()
    torch.cuda.synchronize()
    frontend_us = (time.perf_counter() - t0) * 1e6 / 20
    del launches
    torch.cuda.empty_cache()
    return dict(us=us, hot_us=hot_us, wall_us=wall_us, kernel=plan.last_kernel, sets=sets, frontend_us=frontend_us, ttir=ttir,
                warmup_steps_run=done)


def measured_traffic(name):
    """HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE + WRITE_SIZE, scaled by
    a copy-kernel calibration; see profiles/hbm_traffic.json), or None if no figure is on file."""
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            return json.load(f).get(name, {}).get("hbm_bytes_per_launch")
    except (OSError, ValueError):
        return None


def roofline(wl, us, name=None):
    traffic = measured_traffic(name) if name else None
    if wl["bound"] == "hbm":
        achieved = wl["work"] / us / 1e3  # GB/s
        return dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                    frac=round(achieved / HBM_PEAK_GBS, 4), traffic=traffic)
    achieved = wl["work"] / us / 1e6  # TFLOP/s
    return dict(bound="mfma", achieved=round(achieved, 1), peak=BF16_PEAK_TFLOPS, unit="TFLOP/s",
                frac=round(achieved / BF16_PEAK_TFLOPS, 4), traffic=traffic)


def cpu_baseline(torch, name, wl, ttir=None):
    """Times the CPU restatement (1 thread) on a bounded sample of the workload."""
    from oracle import cpu
    torch.manual_seed(0)
    if "lanes" in wl:
        seconds, frac, sample = wl["lanes"](ttir)
        full_seconds = seconds / frac
        return dict(value=float(f"{wl['work'] / full_seconds / 1e9:.4g}"), unit="GB/s", cores=1, kind="port",
                    sample=sample + " (lane-level interpreter of the kernel's TTIR)", seconds_full_workload=float(f"{full_seconds:.4g}"),
                    host_cores_available=os.cpu_count())

    def timed(fn, repeats):
        ts = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return sum(ts) / len(ts), min(ts)

    if name.startswith("cfg1"):
        n = 98432 if name == "cfg1" else 1 << 24
        x, y = torch.rand(n), torch.rand(n)
        mean, best = timed(lambda: cpu.vec_add(x, y), 20)
        frac, sample = n * 12 / wl["work"], f"N={n}, 20 repeats"
    elif name.startswith("cfg2"):
        rows = 4096
        x = torch.randn(rows, 781)
        mean, best = timed(lambda: cpu.row_softmax(x), 10)
        frac, sample = rows * 781 * 8 / wl["work"], f"{rows} rows, 10 repeats"
    elif name == "cfg3":
        rows = 1024
        x = torch.randn(rows, 8192).half()
        w, b = torch.randn(8192).half(), torch.randn(8192).half()
        mean, best = timed(lambda: cpu.layer_norm_fwd(x, w, b, 1e-5), 5)
        frac, sample = rows / 4096, f"{rows} of 4096 rows, 5 repeats"
    elif name == "cfg4":
        a = (torch.randn(4096, 4096) * 0.02).bfloat16()
        b = (torch.randn(4096, 4096) * 0.02).bfloat16()
        out = torch.zeros(4096, 4096, dtype=torch.bfloat16)
        progs = 8
        mean, best = timed(lambda: cpu.matmul_tiles(a, b, pids=(0, progs), out=out), 1)
        frac, sample = progs / 1024, f"{progs} of 1024 programs (identical work each), 1 run"
    else:
        a = torch.randn(16, 8192).half()
        w = torch.randint(-127, 128, (8192, 28672), dtype=torch.int8)
        s = (0.001 + 0.009 * torch.rand(28672)).half()
        out = torch.zeros(16, 28672, dtype=torch.float16)
        ys = 16
        mean, best = timed(lambda: cpu.w8a16_matmul(a, w, s, ys=(0, ys), out=out), 1)
        frac, sample = ys / 224, f"{ys} of 224 column blocks, 1 run"
    full_seconds = mean / frac
    if wl["bound"] == "hbm":
        value, unit = wl["work"] / full_seconds / 1e9, "GB/s"
    else:
        value, unit = wl["work"] / full_seconds / 1e12, "TFLOP/s"
    return dict(value=float(f"{value:.4g}"), unit=unit, cores=1, kind="port", sample=sample,
                seconds_full_workload=float(f"{full_seconds:.4g}"), host_cores_available=os.cpu_count())


def main():
    args = parse()
    if args.gpus != 1:
        print(f"bench.py: this backend runs on one GPU; --gpus {args.gpus} is not supported (no multi-GPU path exists "
              "in this build: programs are independent, a multi-GPU version would shard the grid)", file=sys.stderr)
        sys.exit(2)
    import torch
    import triton
    import triton_shared_amd as tsa
    from triton_shared_amd.examples import kernels as K
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    if args.calibrate_copy:
        n = 256 * 1024 * 1024
        src = torch.ones(n, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration_copy_bytes": n, "copies": 3}))
        return
    tsa.activate()
    spy = Spy()
    torch.manual_seed(0)
    W = make_workloads(torch, triton, K)
    if args.workload not in W:
        print(f"unknown workload {args.workload}; choose from {sorted(W)}", file=sys.stderr)
        sys.exit(2)
    names = [args.workload] if args.only_headline else list(W)
    kernels = {}
    for name in names:
        wl = W[name]
        steps = args.steps if wl["set_bytes"] < 1e9 else max(10, args.steps // 10)
        t = time_workload(torch, spy, wl, steps, args.warmup, args.rotating_only)
        entry = dict(workload=wl["desc"], us=round(t["us"], 3), kernel=t["kernel"], steps=steps,
                     rotating_buffer_sets=t["sets"], warmup_steps_run=t["warmup_steps_run"], frontend_us_per_launch=round(t["frontend_us"], 1),
                     roofline=roofline(wl, t["us"], name), dtype=wl["dtype"], algorithmic_work=wl["work"],
                     same_buffers=dict(us=round(t["hot_us"], 3), frac=roofline(wl, t["hot_us"])["frac"]))
        if not args.no_cpu and (name == args.workload or "lanes" in wl or not name.endswith(("2p28", "1m", "2p26", "2048"))):
            entry["cpu_baseline"] = cpu_baseline(torch, name, wl, t.get("ttir"))
        kernels[name] = entry
    head = kernels[args.workload]
    wl = W[args.workload]
    unit = "GB/s" if wl["bound"] == "hbm" else "TFLOP/s"
    line = {
        "metric": "achieved HBM GB/s & bf16 TFLOP/s as % of MI355X roofline per kernel",
        "value": head["roofline"]["achieved"],
        "unit": unit,
        "n_gpus": 1,
        "steps": head["steps"],
        "warmup": args.warmup,
        "ms_per_step": round(head["us"] / 1e3, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": head["dtype"],
        "data": "synthetic (seeded torch.randn/rand/randint of the config's shapes)",
        "config": {"workload": f"{args.workload}: {wl['desc']}"},
        "roofline": head["roofline"],
        "cpu_baseline": head.get("cpu_baseline"),
        "kernels": kernels,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()

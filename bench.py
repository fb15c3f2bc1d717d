"""Benchmark of the Stream-K GEMM hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extra] [--no-cpu]
    python bench.py --case MxNxK [--dtype D] [--layout nt|nn] [--config "dict(...)"] [--data rand|zeros|ones]
                    [--reps R] [--copies C] [--time] [--vendor]       one GEMM case on its own, for a profiler

One "step" is one fp16 GEMM call through the C ABI on inputs already resident in HBM.  The headline
workload is M = N = K = 8192 (NT layout, U[-1,1) from seed 0), the compute-bound end of the
metric's sweep; `value` is whole-job TFLOP/s over exactly `steps` timed calls.  The same JSON line
carries
  roofline      the dominant kernel's achieved rate from HIP events on the launch stream,
  cpu_baseline  the oracle's fp32 host matmul timed on this box's cores on a bounded sample,
  config.metric_parts   the other two parts of the metric in short: Stream-K against the data-parallel schedule at
                M = 256 / 512 / 1024 (same tile, and the best data-parallel tile), Q4 GEMM at M = 1 / 16 as a
                fraction of HBM peak with the weights in the Infinity Cache and from HBM, fp16 with 16 / 64 rows of A
                with the weights from HBM next to the vendor GEMM, and the 16 cells M = 1 / 16 / 64 / 256 over four
                projection shapes (N, K) of a 7B / 70B decoder against `torch.matmul` in the same run,
  extra         the measurements behind them and the rest: M sweep at N = K = 8192, 1024x1024x8192 with all
                fix-ups, the large dense shapes in both layouts and types, the reference's own run shapes, one row of
                A on 16384 x 16384 and 28672 x 8192 Q4 weights from HBM
                (kernels this short are timed as graph-captured batches).
The oracle is used here as the timed CPU baseline and as a result check only.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "stream-k.tvm_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_FP16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, published
PEAK_HBM_GBS = 8000.0      # MI355X HBM3E, published


def planner_sweep(torch, streamk, time_graph):
    """Untuned plans (sk_make_plan with no configuration and no tuned-cache lookup) against the vendor GEMM that
    torch calls, M from 128 to 4096 over six (N, K) pairs, per operand type and layout.  Prints one JSON line:
    per type the mean and the worst ratio time / vendor time (below 1: faster than the vendor) and the rows."""
    schedules = {v: k for k, v in streamk._lib.SCHEDULES.items()}
    out = {}
    for dt, lay in (("float16", "nt"), ("float16", "nn"), ("bfloat16", "nt"), ("bfloat16", "nn"), ("float8_e4m3", "nt"),
                    ("int8", "nt")):
        rows = []
        for (N, K) in ((4096, 4096), (8192, 8192), (4096, 11008), (11008, 4096), (5120, 5120), (6144, 4096)):
            for M in (128, 256, 512, 768, 1024, 1536, 2048, 3000, 4096):
                g = torch.Generator().manual_seed(0)
                if dt == "int8":
                    A = torch.randint(-8, 9, (M, K), generator=g, dtype=torch.int8).cuda()
                    B = torch.randint(-8, 9, (N, K), generator=g, dtype=torch.int8).cuda()
                    C = torch.empty(M, N, dtype=torch.int32, device="cuda")
                    run = lambda p: streamk.streamk_int8(A, B, out=C, plan=p)  # noqa: E731
                    ref = lambda: torch._int_mm(A, B.T, out=C)  # noqa: E731
                elif dt == "float8_e4m3":
                    if K % 16:
                        continue
                    A = (torch.rand(M, K, generator=g) * 2 - 1).cuda().to(torch.float8_e4m3fn)
                    B = (torch.rand(N, K, generator=g) * 2 - 1).cuda().to(torch.float8_e4m3fn)
                    C = torch.empty(M, N, dtype=torch.float16, device="cuda")
                    one = torch.ones((), device="cuda")
                    run = lambda p: streamk.streamk_fp8(A, B, out=C, plan=p)  # noqa: E731
                    ref = lambda: torch._scaled_mm(A, B.T, one, one, out_dtype=torch.float16, out=C)  # noqa: E731
                else:
                    tdt = torch.float16 if dt == "float16" else torch.bfloat16
                    A = (torch.rand(M, K, generator=g) * 2 - 1).to(tdt).cuda()
                    B = (torch.rand(*((N, K) if lay == "nt" else (K, N)), generator=g) * 2 - 1).to(tdt).cuda()
                    C = torch.empty(M, N, dtype=tdt, device="cuda")
                    gemm = streamk.streamk_fp16 if dt == "float16" else streamk.streamk_bf16
                    run = lambda p: gemm(A, B, layout=lay, out=C, plan=p)  # noqa: E731
                    ref = lambda: torch.matmul(A, B.T if lay == "nt" else B, out=C)  # noqa: E731
                p = streamk.make_plan(M, N, K, dt, lay, use_tuned=False)
                try:
                    t_ref = time_graph(ref, launches=10)
                except Exception:   # no such GEMM in this torch build
                    continue
                t_sk = time_graph(lambda: run(p), launches=10)
                rows.append({"M": M, "N": N, "K": K, "us": round(t_sk * 1e3, 1), "vendor_us": round(t_ref * 1e3, 1),
                             "ratio": round(t_sk / t_ref, 3), "kernel": streamk.kernel_name(p.kernel_id),
                             "schedule": schedules.get(p.schedule, p.schedule), "grid": p.grid})
        if rows:
            out[f"{dt}_{lay}"] = {"shapes": len(rows), "mean_ratio": round(sum(r["ratio"] for r in rows) / len(rows), 3),
                                  "worst": sorted(rows, key=lambda r: -r["ratio"])[:3], "rows": rows}
    streamk.workspace_status()
    print(json.dumps({"planner_sweep": out}))


def run_case(args):
    """One GEMM case a few times, so that a profiler sees nothing else (--case).  --data chooses the operand values
    (the clock the part sustains depends on how many bits toggle); --time prints the average time of --reps launches;
    --vendor also times the vendor GEMM torch calls (hipBLASLt) on the same operands."""
    import torch
    import streamk
    M, N, K = (int(x) for x in args.case.split("x"))
    cfg = eval(args.config, {"dict": dict})  # noqa: S307 (developer option)
    g = torch.Generator(device="cpu").manual_seed(0)
    plan = streamk.make_plan(M, N, K, args.dtype, args.layout, cfg)
    vendor = None
    if args.dtype == "q4":
        A = torch.randn(M, K, generator=g).half().cuda()
        Wq = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8).cuda()
        sc = (torch.rand(N, K // 128, generator=g) * 0.015 + 0.005).half().cuda()
        Wqs, turn = [Wq] + [Wq.clone() for _ in range(args.copies - 1)], [0]

        def run():   # (--copies: the launches rotate over copies of the weights, so that each one reads HBM)
            turn[0] += 1
            streamk.streamk_q4(A, Wqs[turn[0] % len(Wqs)], sc, plan=plan)
    elif args.dtype == "int8":
        if args.data == "rand":
            A = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8).cuda()
            B = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8).cuda()
        else:
            fill = torch.zeros if args.data == "zeros" else torch.ones
            A, B = fill(M, K, dtype=torch.int8, device="cuda"), fill(N, K, dtype=torch.int8, device="cuda")
        C = torch.empty(M, N, dtype=torch.int32, device="cuda")
        run = lambda: streamk.streamk_int8(A, B, out=C, plan=plan)  # noqa: E731
        vendor = ("torch._int_mm", lambda: torch._int_mm(A, B.T))
    elif args.dtype == "float8_e4m3":
        f8 = torch.float8_e4m3fn
        if args.data == "rand":
            A = (torch.rand(M, K, generator=g) * 2 - 1).cuda().to(f8)
            B = (torch.rand(N, K, generator=g) * 2 - 1).cuda().to(f8)
        else:
            fill = torch.zeros if args.data == "zeros" else torch.ones
            A, B = fill(M, K, device="cuda").to(f8), fill(N, K, device="cuda").to(f8)
        C = torch.empty(M, N, dtype=torch.float16, device="cuda")
        one = torch.ones(1, device="cuda")
        run = lambda: streamk.streamk_fp8(A, B, out=C, plan=plan)  # noqa: E731
        vendor = ("torch._scaled_mm", lambda: torch._scaled_mm(A, B.T, scale_a=one, scale_b=one, out_dtype=torch.float16))
    else:
        dt = {"float16": torch.float16, "bfloat16": torch.bfloat16}.get(args.dtype, torch.float32)
        bshape = (N, K) if args.layout == "nt" else (K, N)
        if args.data == "rand":
            A = (torch.rand(M, K, generator=g) * 2 - 1).to(dt).cuda()
            B = (torch.rand(*bshape, generator=g) * 2 - 1).to(dt).cuda()
        else:
            fill = torch.zeros if args.data == "zeros" else torch.ones
            A, B = fill(M, K, dtype=dt, device="cuda"), fill(*bshape, dtype=dt, device="cuda")
        C = torch.empty(M, N, dtype=dt, device="cuda")
        fn = {"float16": streamk.streamk_fp16, "bfloat16": streamk.streamk_bf16}.get(args.dtype, streamk.streamk_fp32)
        Bs, turn = [B] + [B.clone() for _ in range(args.copies - 1)], [0]

        def run():   # (--copies: the launches rotate over copies of B, so that each one reads HBM)
            turn[0] += 1
            fn(A, Bs[turn[0] % len(Bs)], layout=args.layout, out=C, plan=plan)
        Bt = B.T if args.layout == "nt" else B
        vendor = ("torch.matmul", lambda: torch.matmul(A, Bt, out=C))
    for _ in range(args.reps):
        run()
    torch.cuda.synchronize()
    streamk.workspace_status()
    if args.time:
        ms = streamk.bench_ms(run, 3, args.reps)
        print(f"{args.data}: {ms * 1e3:.2f} us, {2.0 * M * N * K / ms / 1e9:.0f} TFLOP/s")
    if args.vendor and vendor is not None:
        ms = streamk.bench_ms(vendor[1], 3, args.reps)
        print(f"{args.data}: {vendor[0]} {ms * 1e3:.2f} us, {2.0 * M * N * K / ms / 1e9:.0f} TFLOP/s")
    print(f"ran {args.reps} x {args.dtype} {args.layout} {M}x{N}x{K} kernel {streamk.kernel_name(plan.kernel_id)} grid {plan.grid} "
          f"streamk_tiles {plan.streamk_tiles}")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-extra", action="store_true", help="skip the sweep / Q4 section")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--planner-sweep", action="store_true",
                    help="instead of the benchmark: time the planner's own choice (no tuned cache) against the vendor "
                         "GEMM on a grid of shapes, per operand type and layout; one JSON line")
    ap.add_argument("--case", default=None, metavar="MxNxK", help="instead of the benchmark: run this one GEMM --reps times")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16", "float32", "q4", "float8_e4m3", "int8"])
    ap.add_argument("--layout", default="nt", choices=["nt", "nn"])
    ap.add_argument("--config", default="{}", help="--case: python dict of plan options, e.g. \"dict(bm=256,bn=256,raster=8)\"")
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--copies", type=int, default=1, help="--case: rotate the launches over this many copies of the weights (fp16 / bfloat16 / q4)")
    ap.add_argument("--data", default="rand", choices=["rand", "zeros", "ones"])
    ap.add_argument("--time", action="store_true", help="--case: print the average time of the launches")
    ap.add_argument("--vendor", action="store_true", help="--case: also run (and with --time, time) the vendor GEMM")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a 1 GiB device-to-device copy (reference point for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this library runs on one GPU; --gpus must be 1 "
              "(a sharded run would split N across devices with no exchange)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch
    import streamk
    from oracle import oracle

    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    streamk.lib()
    cus = streamk.num_cus()

    def inputs(M, N, K, seed=0):
        g = torch.Generator(device="cpu").manual_seed(seed)
        A = (torch.rand(M, K, generator=g) * 2 - 1).half().cuda()
        B = (torch.rand(N, K, generator=g) * 2 - 1).half().cuda()
        return A, B

    def time_eager(fn, warmup, steps):
        """events on the launch stream (the library launches on torch's current stream)"""
        for _ in range(warmup):
            fn()
        st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        st.record()
        for _ in range(steps):
            fn()
        en.record()
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3
        return st.elapsed_time(en) / steps, wall_ms / steps

    def time_graph(fn, launches=20, **kw):
        """per-launch ms of a graph-captured batch (no host launch cost between microsecond kernels): the median
        of seven timed groups of replays over 40 ms, on the side stream whose launches are quickest (see
        streamk.timing_stream: streams differ by 1.6 us per HBM-streaming launch on this part)"""
        return streamk.graph_ms(fn, launches=launches, **kw)

    if args.planner_sweep:
        planner_sweep(torch, streamk, time_graph)
        return
    if args.case:
        run_case(args)
        return

    if args.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    # ---------------------------------------------------------------- headline: 8192^3
    M = N = K = 8192
    A, B = inputs(M, N, K)
    C = torch.empty(M, N, dtype=torch.float16, device="cuda")
    plan = streamk.make_plan(M, N, K, "float16", "nt", raster=8)
    step = lambda: streamk.streamk_fp16(A, B, out=C, plan=plan)  # noqa: E731
    # The part takes ~40 ms of matrix load to settle at its sustained clock (the first 25 launches of
    # a cold device run ~10 % slower than the 50th): bring it there before the W warm-up steps, so
    # that a small --warmup does not time the ramp.
    PREWARM = 60
    for _ in range(PREWARM):
        step()
    torch.cuda.synchronize()
    ev_ms, wall_ms = time_eager(step, args.warmup, args.steps)
    streamk.workspace_status()
    flops = 2.0 * M * N * K
    value = flops / (wall_ms * 1e-3) / 1e12
    kernel_tflops = flops / (ev_ms * 1e-3) / 1e12
    # result check on a block of rows against the oracle's fp32 host matmul
    ref = oracle.matmul_fp32(A[:64].cpu().numpy(), B.cpu().numpy(), trans_b=True)
    err = oracle.max_abs_rel(C[:64].float().cpu().numpy(), ref)
    assert err <= 1e-2, err

    # What the matrix pipes alone sustain on this box, in this process, right after the timed steps (the device
    # is at its sustained clock): a loop of nothing but 16x16x32 fp16 MFMAs on U[-1,1) register operands, ~40 ms
    # untimed, then ~40 ms timed.  The published peak assumes the maximum clock; this is the part's own ceiling.
    def mfma_only(shape):
        import ctypes
        # (bench.py's own helper, built beside the library by the same Makefile; not part of the product's C ABI)
        L = ctypes.CDLL(os.path.join(os.path.dirname(streamk._lib.LIB_PATH), "libstreamk_bench.so"))
        L.skb_mfma_only.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p,
                                    ctypes.POINTER(ctypes.c_double)]
        scratch = torch.empty(cus * 256, dtype=torch.float32, device="cuda")
        flop = ctypes.c_double(0.0)
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        iters = 4000  # ~2.5 ms per launch
        def launch():
            rc = L.skb_mfma_only(shape, iters, 0, scratch.data_ptr(), scratch.numel() * 4, stream, ctypes.byref(flop))
            assert rc == 0, rc
        for _ in range(16):
            launch()
        st, en = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        st.record()
        for _ in range(16):
            launch()
        en.record()
        torch.cuda.synchronize()
        return flop.value / (st.elapsed_time(en) / 16 * 1e-3) / 1e12
    mfma_only_tflops = mfma_only(1)
    # ... and the vendor's kernel for the same product, same operands, same moment (hipBLASLt through torch.matmul)
    vendor = lambda: torch.matmul(A, B.t(), out=C)  # noqa: E731
    for _ in range(10):
        vendor()
    torch.cuda.synchronize()
    vendor_ms, _ = time_eager(vendor, 5, max(10, args.steps // 2))
    step()  # C holds this library's result again

    # HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE (see profiles/)
    traffic = None
    tpath = os.path.join(ROOT, "profiles", f"traffic_{streamk.kernel_name(plan.kernel_id)}_8192.json")
    if os.path.exists(tpath):
        with open(tpath) as f:
            traffic = json.load(f).get("hbm_bytes_per_launch")

    out = {
        "metric": "fp16 Stream-K GEMM TFLOP/s (M=N=K=8192; Stream-K / data-parallel ratios and Q4 GB/s in config.metric_parts, sweep in extra)",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(wall_ms, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": "fp16 NT GEMM M=N=K=8192, U[-1,1) seed 0, inputs resident in HBM",
                   "tile": [plan.bm, plan.bn, plan.bk], "grid": plan.grid,
                   "streamk_tiles": plan.streamk_tiles, "dp_tiles": plan.blocking_tiles,
                   "compute_units": cus, "check_max_abs_rel": err, "prewarm_launches": PREWARM},
        "roofline": {"bound": "mfma", "achieved": round(kernel_tflops, 2), "peak": PEAK_FP16_TFLOPS,
                     "unit": "TFLOP/s", "frac": round(kernel_tflops / PEAK_FP16_TFLOPS, 4),
                     "traffic": traffic, "kernel": streamk.kernel_name(plan.kernel_id),
                     "avg_launch_ms": round(ev_ms, 5),
                     "mfma_only_tflops": round(mfma_only_tflops, 1),
                     "frac_of_mfma_only": round(kernel_tflops / mfma_only_tflops, 4),
                     "vendor_matmul_tflops": round(flops / (vendor_ms * 1e-3) / 1e12, 1)},
    }

    # ---------------------------------------------------------------- CPU baseline (oracle, bounded)
    if not args.no_cpu:
        torch.set_num_threads(os.cpu_count())
        Bh = B.float().cpu()
        rows = 256
        Ah = A[:rows].float().cpu()
        t0 = time.perf_counter()
        torch.matmul(Ah, Bh.T)
        rate = 2.0 * rows * N * K / (time.perf_counter() - t0)
        rows = int(min(M, max(256, (rate * 12.0) / (2.0 * N * K)) // 64 * 64))  # about 12 s of work
        Ah = A[:rows].float().numpy(force=True)
        Bn = Bh.numpy()
        t0 = time.perf_counter()
        oracle.matmul_fp32(Ah, Bn, trans_b=True)
        dt = time.perf_counter() - t0
        # a host that finishes the sample in well under 10 s repeats it until about 10 s have gone by
        reps = 1 if dt >= 5.0 else max(1, min(40, int(10.0 / max(dt, 1e-3))))
        if reps > 1:
            t0 = time.perf_counter()
            for _ in range(reps):
                oracle.matmul_fp32(Ah, Bn, trans_b=True)
            dt = (time.perf_counter() - t0) / reps
        # what the product actually ran on: the BLAS numpy is linked against reports its own thread count; the
        # process may be confined to fewer logical CPUs than the box has
        affinity = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else os.cpu_count()
        blas_threads, blas_name = None, None
        try:
            from threadpoolctl import threadpool_info
            for pool in threadpool_info():
                if pool.get("user_api") == "blas":
                    blas_threads, blas_name = pool.get("num_threads"), pool.get("internal_api")
        except Exception:
            pass
        cpu_model = None
        try:
            with open("/proc/cpuinfo") as f:
                cpu_model = next((ln.split(":", 1)[1].strip() for ln in f if ln.startswith("model name")), None)
        except OSError:
            pass
        out["cpu_baseline"] = {"value": round(2.0 * rows * N * K / dt / 1e12, 4), "unit": "TFLOP/s",
                               "cores": blas_threads or affinity, "kind": "port",
                               "blas": blas_name, "blas_threads": blas_threads, "cpus_in_affinity_mask": affinity,
                               "logical_cpus": os.cpu_count(), "cpu_model": cpu_model,
                               "sample": f"oracle fp32 host matmul (numpy) of the first {rows} rows of the "
                                         f"same A against all of B ({rows}x{N}x{K}), {reps} x {dt:.2f} s"}

    # ---------------------------------------------------------------- rest of the metric
    if not args.no_extra:
        extra = {"timing": "graph-captured batches of launches on the quickest of eight side streams; median of seven timed groups of replays over 40 ms"}
        sweep = []
        for m in (16, 64, 256, 512, 1024, 2048, 4096, 8192):
            a, _ = inputs(m, 8, K, seed=m)
            c = torch.empty(m, N, dtype=torch.float16, device="cuda")
            row = {"M": m}
            cands = {"auto": {}}
            tiles = {"128": (128, 128), "128x256": (128, 256), "256": (256, 256)}
            if m > 64:
                # per tile shape: the data-parallel-only schedule against the best Stream-K schedule of the same kernel
                for t, (bm, bn) in tiles.items():
                    cands["dp_" + t] = dict(bm=bm, bn=bn, bk=64, schedule="dp", raster=8)
                    for sch in ("sk2", "basic", "splitk"):
                        cands[f"{sch}_{t}"] = dict(bm=bm, bn=bn, bk=64, schedule=sch, fixup="reduce", raster=8)
            else:
                cands.update({"dp": dict(schedule="dp"), "sk": dict(schedule="sk2", grid=256)})
            # (the clock needs tens of milliseconds of load to settle after the idle time spent preparing inputs:
            # without this the first candidate of every row reads ~7 % low)
            p = streamk.make_plan(m, N, K, "float16", "nt")
            for _ in range(min(2000, max(PREWARM, int(0.05 / (2.0 * m * N * K / 1e15))))):  # about 50 ms of load
                streamk.streamk_fp16(a, B, out=c, plan=p)
            # M <= 64: one 134 MB B launched repeatedly is served by the 256 MB Infinity Cache, which is not an HBM
            # rate; these rows are timed with the launches of a batch rotating over copies of B totalling > 512 MB
            # (the figures with one B are kept beside them as `weights_in_infinity_cache`)
            copies = [B] + [B.clone() for _ in range(4)] if m <= 64 else None
            warm = {}
            for name, cfg in cands.items():
                try:
                    p = streamk.make_plan(m, N, K, "float16", "nt", **cfg)
                except streamk.StreamKError:
                    continue  # the fixed split does not divide this shape
                ms = time_graph(lambda: streamk.streamk_fp16(a, B, out=c, plan=p))
                if m > 64:
                    row[name] = round(2.0 * m * N * K / ms / 1e9, 1)
                    continue
                warm[name] = round(2.0 * m * N * K / ms / 1e9, 1)
                turn = [0]

                def rotating():
                    w = copies[turn[0] % len(copies)]
                    turn[0] += 1
                    streamk.streamk_fp16(a, w, out=c, plan=p)
                ms = time_graph(rotating)
                row[name] = round(2.0 * m * N * K / ms / 1e9, 1)
                if name == "auto":
                    row["auto_weights_from_hbm_us"] = round(ms * 1e3, 2)
            if m <= 64:
                # the vendor GEMM on the same rotation of weights
                def rotating_vendor():
                    w = copies[turn[0] % len(copies)]
                    turn[0] += 1
                    torch.matmul(a, w.T, out=c)
                turn = [0]
                row["torch_matmul_weights_from_hbm_us"] = round(time_graph(rotating_vendor) * 1e3, 2)
            copies = None
            if m > 64:
                for t in tiles:
                    sk_best = max((row.pop(f"{sch}_{t}"), sch) for sch in ("sk2", "basic", "splitk") if f"{sch}_{t}" in row)
                    row["sk_" + t], row["sk_schedule_" + t] = sk_best
                # the plan the library makes by itself: its tile, and the data-parallel-only schedule of that tile
                pa = streamk.make_plan(m, N, K, "float16", "nt")
                key = {(bm, bn): t for t, (bm, bn) in tiles.items()}.get((pa.bm, pa.bn))
                row["auto_tile"], row["auto_kernel"] = [pa.bm, pa.bn, pa.bk], streamk.kernel_name(pa.kernel_id)
                row["auto_streamk_tiles"], row["auto_grid"] = pa.streamk_tiles, pa.grid
                # (reduce16: the tuned entry exchanges its half tiles rounded to 16 bits; the sk_* rows beside it use
                # the fp32 REDUCE)
                row["auto_fixup"] = {v: k for k, v in streamk._lib.FIXUPS.items()}.get(pa.fixup, pa.fixup) if pa.streamk_tiles else "none"
                if key is None:
                    pd = streamk.make_plan(m, N, K, "float16", "nt", bm=pa.bm, bn=pa.bn, bk=pa.bk, schedule="dp", raster=8)
                    ms = time_graph(lambda: streamk.streamk_fp16(a, B, out=c, plan=pd))
                    key = f"{pa.bm}x{pa.bn}"
                    row["dp_" + key] = round(2.0 * m * N * K / ms / 1e9, 1)
                best_dp = max(v for k, v in row.items() if k.startswith("dp_"))
                # Stream-K against data-parallel on the tile the library chose, and the library's plan against the best
                # data-parallel plan of any tile measured
                row["sk_over_dp_same_tile"] = round(max(row["auto"], row.get("sk_" + key, 0.0)) / row["dp_" + key], 3)
                row["auto_over_best_dp"] = round(row["auto"] / best_dp, 3)
            best = max(v for k, v in row.items() if isinstance(v, float) and (k == "auto" or k.startswith(("dp", "sk"))) and not k.endswith("_us") and "over" not in k)
            row["best_tflops"] = best
            row["pct_fp16_peak"] = round(100 * best / PEAK_FP16_TFLOPS, 2)
            nbytes = 2.0 * (m * K + N * K + m * N)
            row["gbs"] = round(best * 1e3 * nbytes / (2.0 * m * N * K), 1)
            if m <= 64:
                row["weights_in_infinity_cache"] = warm
                row["gbs_is"] = "weights from HBM (launches rotate over 5 copies of B, 671 MB)"
                row["frac_hbm"] = round(row["gbs"] / PEAK_HBM_GBS, 4)
            else:
                row["gbs_is"] = "algorithmic bytes over time; compute-bound row, operands stay in the Infinity Cache"
            sweep.append(row)
        extra["sweep_N8192_K8192_tflops"] = sweep

        a, b = inputs(1024, 1024, 8192, seed=2)
        c = torch.empty(1024, 1024, dtype=torch.float16, device="cuda")
        cfg2 = {}
        # (atomic_c: the reference's own fix-up, partial sums rounded to fp16 and added into C with packed atomics)
        for name, cfg in {"reduce": dict(schedule="sk2", fixup="reduce"), "atomic": dict(schedule="sk2", fixup="atomic"),
                          "atomic_c": dict(schedule="sk2", fixup="atomic_c"), "dp": dict(schedule="dp")}.items():
            p = streamk.make_plan(1024, 1024, 8192, "float16", "nt", bm=128, bn=128, bk=64, grid=256, **cfg)
            ms = time_graph(lambda: streamk.streamk_fp16(a, b, out=c, plan=p))
            cfg2[name] = {"us": round(ms * 1e3, 2), "tflops": round(2.0 * 1024 * 1024 * 8192 / ms / 1e9, 1)}
        extra["cfg_1024x1024x8192_128x128"] = cfg2

        # the large dense configuration in both layouts: tuned plan against the data-parallel-only
        # schedule of the same tile, and torch.matmul (hipBLASLt) on the same operands
        dense = []
        for (m, n, k) in ((8192, 8192, 8192), (3000, 5120, 12288)):
            a, b = inputs(m, n, k, seed=5)
            bt = b.T.contiguous()
            c = torch.empty(m, n, dtype=torch.float16, device="cuda")
            for layout, bmat in (("nt", b), ("nn", bt)):
                p = streamk.make_plan(m, n, k, "float16", layout)
                pd = streamk.make_plan(m, n, k, "float16", layout, bm=p.bm, bn=p.bn, bk=p.bk, schedule="dp", raster=8)
                row = {"shape": [m, n, k], "layout": layout, "tile": [p.bm, p.bn, p.bk],
                       "kernel": streamk.kernel_name(p.kernel_id), "streamk_tiles": p.streamk_tiles}
                fns = {"tuned": lambda: streamk.streamk_fp16(a, bmat, layout=layout, out=c, plan=p),
                       "dp_only": lambda: streamk.streamk_fp16(a, bmat, layout=layout, out=c, plan=pd),
                       "torch_matmul": lambda: torch.matmul(a, bmat.T if layout == "nt" else bmat, out=c)}
                best = {}
                for _ in range(3):  # interleaved rounds: the sustained clock drifts over the first launches
                    for name, fn in fns.items():
                        best[name] = min(best.get(name, 1e9), time_eager(fn, 3, 10)[0])
                for name, ms in best.items():
                    row[name] = {"us": round(ms * 1e3, 1), "tflops": round(2.0 * m * n * k / ms / 1e9, 1)}
                dense.append(row)
            del a, b, bt, c
        extra["large_dense"] = dense

        # the same kernel structure on one-byte operands, against the 5.0 PFLOP/s (POP/s) dense fp8 / int8 peak, with
        # hipBLASLt (torch._scaled_mm / torch._int_mm) on the same operands where this torch build provides it
        for key, dt in (("fp8_e4m3_dense", "float8_e4m3"), ("int8_dense", "int8")):
            rows8 = []
            for (m, n, k) in ((8192, 8192, 8192), (1024, 8192, 8192)):
                if dt == "int8":
                    g8 = torch.Generator(device="cpu").manual_seed(6)
                    a8 = torch.randint(-128, 128, (m, k), generator=g8, dtype=torch.int8).cuda()
                    b8 = torch.randint(-128, 128, (n, k), generator=g8, dtype=torch.int8).cuda()
                    c = torch.empty(m, n, dtype=torch.int32, device="cuda")
                    ours, vendor, vname = streamk.streamk_int8, (lambda: torch._int_mm(a8, b8.T)), "torch_int_mm"
                else:
                    a, b = inputs(m, n, k, seed=6)
                    a8, b8 = a.to(torch.float8_e4m3fn), b.to(torch.float8_e4m3fn)
                    del a, b
                    c = torch.empty(m, n, dtype=torch.float16, device="cuda")
                    one = torch.ones(1, device="cuda")
                    ours, vname = streamk.streamk_fp8, "torch_scaled_mm"
                    vendor = lambda: torch._scaled_mm(a8, b8.T, scale_a=one, scale_b=one, out_dtype=torch.float16)  # noqa: E731
                p = streamk.make_plan(m, n, k, dt, "nt")
                row = {"shape": [m, n, k], "tile": [p.bm, p.bn, p.bk], "kernel": streamk.kernel_name(p.kernel_id),
                       "streamk_tiles": p.streamk_tiles}
                fns = {"tuned": lambda: ours(a8, b8, out=c, plan=p), vname: vendor}
                best = {}
                for _ in range(3):
                    for name, fn in fns.items():
                        if best.get(name, 0) is None:
                            continue
                        try:
                            best[name] = min(best.get(name, 1e9), time_eager(fn, 3, 10)[0])
                        except Exception:   # no such GEMM in this torch build
                            best[name] = None
                for name, ms in best.items():
                    row[name] = None if ms is None else {"us": round(ms * 1e3, 1), "tops": round(2.0 * m * n * k / ms / 1e9, 1),
                                                         "frac_peak": round(2.0 * m * n * k / ms / 1e9 / 5000.0, 4)}
                rows8.append(row)
                del a8, b8, c
            extra[key] = rows8

        # few rows of one-byte operands: the 64 x 128 tile kernel in two stages of 128 K-values against the same tile
        # in four stages of 64 (three loads in flight per CTA instead of one), the planner's own choice and the vendor
        # GEMM; graph-timed (these launches take 10-30 us)
        few = []
        for dt in ("float8_e4m3", "int8"):
            for (m, n, k) in ((128, 11008, 4096), (256, 5120, 5120)):
                g8 = torch.Generator(device="cpu").manual_seed(8)
                if dt == "int8":
                    a8 = torch.randint(-8, 9, (m, k), generator=g8, dtype=torch.int8).cuda()
                    b8 = torch.randint(-8, 9, (n, k), generator=g8, dtype=torch.int8).cuda()
                    c = torch.empty(m, n, dtype=torch.int32, device="cuda")
                    ours, vendor = streamk.streamk_int8, (lambda: torch._int_mm(a8, b8.T, out=c))
                else:
                    a8 = (torch.rand(m, k, generator=g8) * 2 - 1).cuda().to(torch.float8_e4m3fn)
                    b8 = (torch.rand(n, k, generator=g8) * 2 - 1).cuda().to(torch.float8_e4m3fn)
                    c = torch.empty(m, n, dtype=torch.float16, device="cuda")
                    one = torch.ones((), device="cuda")
                    ours = streamk.streamk_fp8
                    vendor = lambda: torch._scaled_mm(a8, b8.T, one, one, out_dtype=torch.float16, out=c)  # noqa: E731
                pa = streamk.make_plan(m, n, k, dt, "nt", use_tuned=False)
                p2 = streamk.make_plan(m, n, k, dt, "nt", dict(bm=64, bn=128, bk=128, schedule="dp"))
                p4 = streamk.make_plan(m, n, k, dt, "nt", dict(bm=64, bn=128, bk=64, schedule="dp"))
                row = {"dtype": dt, "shape": [m, n, k], "planner_kernel": streamk.kernel_name(pa.kernel_id), "planner_grid": pa.grid,
                       "planner_us": round(time_graph(lambda: ours(a8, b8, out=c, plan=pa), launches=10) * 1e3, 1),
                       "two_stage_64x128x128_us": round(time_graph(lambda: ours(a8, b8, out=c, plan=p2), launches=10) * 1e3, 1),
                       "four_stage_64x128x64_us": round(time_graph(lambda: ours(a8, b8, out=c, plan=p4), launches=10) * 1e3, 1)}
                try:
                    row["vendor_us"] = round(time_graph(vendor, launches=10) * 1e3, 1)
                except Exception:   # no such GEMM in this torch build
                    row["vendor_us"] = None
                few.append(row)
                del a8, b8, c
        extra["one_byte_few_rows"] = few

        q4 = []
        g = torch.Generator(device="cpu").manual_seed(4)
        Wq = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8).cuda()
        sc = (torch.rand(N, K // 128, generator=g) * 0.015 + 0.005).half().cuda()
        for m in (1, 16):
            a = torch.randn(m, K, generator=g).half().cuda()
            c = torch.empty(m, N, dtype=torch.float16, device="cuda")
            nbytes = 2 * m * K + N * K // 2 + 2 * N * (K // 128) + 2 * m * N
            row = {"M": m, "bytes": nbytes}
            for name, cfg in {"tuned": dict(),
                              "streamk_reduce": dict(schedule="sk2", fixup="reduce", grid=256),
                              "streamk_atomic": dict(schedule="sk2", fixup="atomic", grid=256),
                              "dp": dict(schedule="dp"),
                              # M = 1: `tuned` is a matrix-vector kernel, which multiplies the unrounded
                              # (q - zero) * scale; this is the fastest instance that forms the fp16-rounded
                              # weights of the dequantisation contract bit for bit (all kernels do for M > 1)
                              "rounded_weights": dict(variant=2, schedule="dp")}.items():
                if name == "rounded_weights" and m != 1:
                    continue
                p = streamk.make_plan(m, N, K, "q4", "nt", **cfg)
                ms = time_graph(lambda: streamk.streamk_q4(a, Wq, sc, out=c, plan=p))
                row[name] = {"us": round(ms * 1e3, 2), "gbs": round(nbytes / ms / 1e6, 1),
                             "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
            # the same launch with the weights coming from HBM: the 20 launches of a batch read 20
            # different copies (692 MB, against 256 MB of Infinity Cache)
            if True:
                copies = [(Wq.clone(), sc.clone()) for _ in range(20)]
                turn = [0]

                def cold():
                    w, s_ = copies[turn[0] % len(copies)]
                    turn[0] += 1
                    streamk.streamk_q4(a, w, s_, out=c, plan=p_cold)
                p_cold = streamk.make_plan(m, N, K, "q4", "nt")
                ms = time_graph(cold)
                row["tuned_weights_from_hbm"] = {"us": round(ms * 1e3, 2), "gbs": round(nbytes / ms / 1e6, 1),
                                                 "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
                if m == 1:
                    # the same measurement on eight different side streams: the streams of a process are not alike
                    per_stream = [round(time_graph(cold, stream=torch.cuda.Stream()) * 1e3, 2) for _ in range(8)]
                    row["tuned_weights_from_hbm"]["us_on_eight_other_streams"] = per_stream
            if m == 1:
                p_cold = streamk.make_plan(m, N, K, "q4", "nt", variant=2, schedule="dp")
                ms = time_graph(cold)
                row["rounded_weights_from_hbm"] = {"us": round(ms * 1e3, 2), "gbs": round(nbytes / ms / 1e6, 1),
                                                   "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
                # one zero point per scale group and row (asymmetric quantisers) instead of the scalar 8
                zp = torch.randint(0, 16, (N, K // 128), generator=g).half().cuda()
                p_zp = streamk.make_plan(m, N, K, "q4_zp", "nt")

                def cold_zp():
                    w, s_ = copies[turn[0] % len(copies)]
                    turn[0] += 1
                    streamk.streamk_q4(a, w, s_, zeros=zp, out=c, plan=p_zp)
                ms = time_graph(cold_zp)
                row["per_group_zero_points_from_hbm"] = {"us": round(ms * 1e3, 2), "kernel": streamk.kernel_name(p_zp.kernel_id)}
                # the same with the weights in the tiled layout (one contiguous KB per load instruction)
                tiles = [(streamk.tile_q4(w), s_) for (w, s_) in copies]
                del copies
                p_tiled = streamk.make_plan(m, N, K, "q4_tiled", "nt")

                def cold_tiled():
                    w, s_ = tiles[turn[0] % len(tiles)]
                    turn[0] += 1
                    streamk.streamk_q4(a, w, s_, out=c, plan=p_tiled, tiled=True)
                ms = time_graph(cold_tiled)
                row["tiled_weights_from_hbm"] = {"us": round(ms * 1e3, 2), "gbs": round(nbytes / ms / 1e6, 1),
                                                 "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
                p_zpt = streamk.make_plan(m, N, K, "q4_zp_tiled", "nt")

                def cold_zp_tiled():
                    w, s_ = tiles[turn[0] % len(tiles)]
                    turn[0] += 1
                    streamk.streamk_q4(a, w, s_, zeros=zp, out=c, plan=p_zpt, tiled=True)
                ms = time_graph(cold_zp_tiled)
                row["tiled_per_group_zero_points_from_hbm"] = {"us": round(ms * 1e3, 2),
                                                               "kernel": streamk.kernel_name(p_zpt.kernel_id)}
                del tiles
            copies = None
            q4.append(row)
        extra["q4_N8192_K8192"] = q4
        # more rows of A than the weight-streaming kernels take: the Q4 tile kernels (nibbles dequantised on their
        # way into the LDS stage), the staged path (dequantise once, fp16 tile kernels) and the fp16 product alone
        pre = []
        Wd = streamk.dequant_q4(Wq, sc)
        for m in (128, 512, 1024, 4096):
            a = torch.randn(m, K, generator=g).half().cuda()
            c = torch.empty(m, N, dtype=torch.float16, device="cuda")
            p = streamk.make_plan(m, N, K, "q4", "nt")
            fl = 2.0 * m * N * K
            t_tile = time_graph(lambda: streamk.streamk_q4(a, Wq, sc, out=c, plan=p), launches=10)
            t_auto = time_graph(lambda: streamk.streamk_q4(a, Wq, sc, out=c), launches=10)
            t_f16 = time_graph(lambda: streamk.streamk_fp16(a, Wd, out=c), launches=10)
            pre.append({"M": m, "kernel": streamk.kernel_name(p.kernel_id),
                        "q4_tile_kernel": {"us": round(t_tile * 1e3, 1), "tflops": round(fl / t_tile / 1e9, 1)},
                        "streamk_q4_default": {"us": round(t_auto * 1e3, 1), "tflops": round(fl / t_auto / 1e9, 1)},
                        "fp16_product_alone": {"us": round(t_f16 * 1e3, 1), "tflops": round(fl / t_f16 / 1e9, 1)}})
        del Wd
        extra["q4_prefill_N8192_K8192"] = pre

        # fp16 matrix-vector product at an LLM-sized weight matrix (470 MB: every launch streams it from HBM)
        nv, kv = 28672, 8192
        wv = torch.randn(nv, kv, generator=g).half().cuda()
        av = torch.randn(1, kv, generator=g).half().cuda()
        cv = torch.empty(1, nv, dtype=torch.float16, device="cuda")
        pv = streamk.make_plan(1, nv, kv, "float16", "nt")
        vbytes = 2 * (kv + nv * kv + nv)
        ms = time_graph(lambda: streamk.streamk_fp16(av, wv, out=cv, plan=pv), launches=5)
        ms_t = time_graph(lambda: torch.matmul(av, wv.T, out=cv), launches=5)
        extra["gemv_f16_M1_N28672_K8192"] = {"kernel": streamk.kernel_name(pv.kernel_id), "bytes": vbytes, "us": round(ms * 1e3, 1),
                                            "gbs": round(vbytes / ms / 1e6, 1), "frac_hbm": round(vbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                                            "torch_matmul_us": round(ms_t * 1e3, 1)}
        # the same product in bfloat16 (the twin kernel with the bfloat16 MFMA)
        wb, ab = wv.bfloat16(), av.bfloat16()
        cb = torch.empty(1, nv, dtype=torch.bfloat16, device="cuda")
        pb = streamk.make_plan(1, nv, kv, "bfloat16", "nt")
        ms = time_graph(lambda: streamk.streamk_bf16(ab, wb, out=cb, plan=pb), launches=5)
        ms_t = time_graph(lambda: torch.matmul(ab, wb.T, out=cb), launches=5)
        extra["gemv_bf16_M1_N28672_K8192"] = {"kernel": streamk.kernel_name(pb.kernel_id), "bytes": vbytes, "us": round(ms * 1e3, 1),
                                             "gbs": round(vbytes / ms / 1e6, 1), "frac_hbm": round(vbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                                             "torch_matmul_us": round(ms_t * 1e3, 1)}
        # and with one-byte weights (fp8 e4m3 -> fp16, int8 -> int32): half the bytes of the same matrix
        w8 = wv.to(torch.float8_e4m3fn)
        a8 = av.to(torch.float8_e4m3fn)
        p8 = streamk.make_plan(1, nv, kv, "float8_e4m3", "nt")
        bytes8 = kv + nv * kv + 2 * nv
        ms = time_graph(lambda: streamk.streamk_fp8(a8, w8, out=cv, plan=p8), launches=5)
        extra["gemv_fp8_M1_N28672_K8192"] = {"kernel": streamk.kernel_name(p8.kernel_id), "bytes": bytes8, "us": round(ms * 1e3, 1),
                                            "gbs": round(bytes8 / ms / 1e6, 1), "frac_hbm": round(bytes8 / ms / 1e6 / PEAK_HBM_GBS, 4)}
        wi, ai = w8.view(torch.int8), a8.view(torch.int8)
        ci = torch.empty(1, nv, dtype=torch.int32, device="cuda")
        pi = streamk.make_plan(1, nv, kv, "int8", "nt")
        bytesi = kv + nv * kv + 4 * nv
        ms = time_graph(lambda: streamk.streamk_int8(ai, wi, out=ci, plan=pi), launches=5)
        extra["gemv_int8_M1_N28672_K8192"] = {"kernel": streamk.kernel_name(pi.kernel_id), "bytes": bytesi, "us": round(ms * 1e3, 1),
                                             "gbs": round(bytesi / ms / 1e6, 1), "frac_hbm": round(bytesi / ms / 1e6 / PEAK_HBM_GBS, 4)}
        del wv, wb, w8, wi

        # offline side of the Q4 path on the same weight shape: algorithmic bytes over graph-timed launches
        Wf = (torch.randn(N, K, generator=g) * 0.05).half().cuda()
        _, _, zp = streamk.quantize_q4(Wf, asymmetric=True)
        rd, wqb, scb = N * K * 2, N * K // 2, N * (K // 128) * 2
        tools = {}
        for name, fn, nbytes in (("quantize_q4", lambda: streamk.quantize_q4(Wf), rd + wqb + scb),
                                 ("quantize_q4_asymmetric", lambda: streamk.quantize_q4(Wf, asymmetric=True), rd + wqb + 2 * scb),
                                 ("dequant_q4", lambda: streamk.dequant_q4(Wq, sc), wqb + scb + rd),
                                 ("dequant_q4_zero_points", lambda: streamk.dequant_q4(Wq, sc, zeros=zp), wqb + 2 * scb + rd),
                                 ("tile_q4", lambda: streamk.tile_q4(Wq), 2 * wqb)):
            ms = time_graph(fn, launches=5)
            tools[name] = {"us": round(ms * 1e3, 1), "gbs": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}
        extra["q4_tools_N8192_K8192"] = tools
        del Wf
        # the reference's own run shapes: fp16 NT 16 x 16384 x 8192 (streamk_fp16.py:61) and Q4 16 x 16384 x 16384
        # (streamk.fp16.breakdown/streamk_fp16_ladder_block_reduce_q4.py:73 and the autotune scripts), weights from HBM
        # (the launches of a batch rotate over copies); beside them the vendor GEMM on fp16 weights
        ref_rows = []
        m, n, k = 16, 16384, 8192
        a16 = (torch.rand(m, k, generator=g) * 2 - 1).half().cuda()
        ws16 = [(torch.rand(n, k, generator=g) * 2 - 1).half().cuda() for _ in range(3)]
        c16 = torch.empty(m, n, dtype=torch.float16, device="cuda")
        p16 = streamk.make_plan(m, n, k, "float16", "nt")
        turn = [0]

        def ref_fp16():
            turn[0] += 1
            streamk.streamk_fp16(a16, ws16[turn[0] % 3], out=c16, plan=p16)

        def ref_fp16_vendor():
            turn[0] += 1
            torch.matmul(a16, ws16[turn[0] % 3].T, out=c16)
        nbytes = 2 * (m * k + n * k + m * n)
        ms, ms_t = time_graph(ref_fp16, launches=6), time_graph(ref_fp16_vendor, launches=6)
        ref_rows.append({"shape": [m, n, k], "dtype": "float16 NT", "kernel": streamk.kernel_name(p16.kernel_id), "us": round(ms * 1e3, 1),
                         "gbs": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                         "torch_matmul_us": round(ms_t * 1e3, 1)})
        del ws16
        m, n, k = 16, 16384, 16384
        aq = torch.randn(m, k, generator=g).half().cuda()
        wqs = [(torch.randint(0, 256, (n, k // 2), generator=g, dtype=torch.uint8).cuda(),
                (torch.rand(n, k // 128, generator=g) * 0.015 + 0.005).half().cuda()) for _ in range(4)]
        cq = torch.empty(m, n, dtype=torch.float16, device="cuda")
        pq = streamk.make_plan(m, n, k, "q4", "nt")

        def ref_q4():
            turn[0] += 1
            w, s_ = wqs[turn[0] % 4]
            streamk.streamk_q4(aq, w, s_, out=cq, plan=pq)
        nbytes = 2 * m * k + n * k // 2 + 2 * n * (k // 128) + 2 * m * n
        ms = time_graph(ref_q4, launches=8)
        wd = streamk.dequant_q4(*wqs[0])   # 537 MB of fp16 weights: more than the Infinity Cache holds
        ms_t = time_graph(lambda: torch.matmul(aq, wd.T, out=cq), launches=4)
        ref_rows.append({"shape": [m, n, k], "dtype": "q4 (group 128, zero 8)", "kernel": streamk.kernel_name(pq.kernel_id),
                         "us": round(ms * 1e3, 1), "gbs": round(nbytes / ms / 1e6, 1),
                         "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4),
                         "torch_matmul_on_fp16_weights_us": round(ms_t * 1e3, 1)})
        del wd
        # one row of A on the same weights and on 28672 x 8192: the Q4 matrix-vector kernels where the planner runs
        # several 16-row tiles per CTA (the later tiles' first loads are requested while the tile before is summed)
        q4_rows = []
        for (n1, k1) in ((16384, 16384), (28672, 8192)):
            a1 = torch.randn(1, k1, generator=g).half().cuda()
            c1 = torch.empty(1, n1, dtype=torch.float16, device="cuda")
            # (the 28672 x 8192 operands are views of the same random bytes and scales)
            w1 = [(wq_.view(-1)[: n1 * k1 // 2].view(n1, k1 // 2), sc_.view(-1)[: n1 * (k1 // 128)].view(n1, k1 // 128))
                  for (wq_, sc_) in wqs]
            p1 = streamk.make_plan(1, n1, k1, "q4", "nt")

            def q4_m1():
                turn[0] += 1
                w, s_ = w1[turn[0] % 4]
                streamk.streamk_q4(a1, w, s_, out=c1, plan=p1)
            nbytes = 2 * k1 + n1 * k1 // 2 + 2 * n1 * (k1 // 128) + 2 * n1
            ms = time_graph(q4_m1, launches=8)
            q4_rows.append({"shape": [1, n1, k1], "kernel": streamk.kernel_name(p1.kernel_id), "grid": p1.grid, "us": round(ms * 1e3, 1),
                            "gbs": round(nbytes / ms / 1e6, 1), "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)})
        extra["q4_one_row_large_weights_from_hbm"] = q4_rows
        del wqs, w1
        extra["reference_run_shapes"] = ref_rows

        # the small-M sweep of the metric's third configuration: M in {1, 16, 64, 256} over four (N, K) pairs, inputs
        # normal(0, 0.02), the plan the library makes by itself (tuned cache included) next to the vendor GEMM; up to
        # 64 rows with the launches rotating over copies of the weights (> 512 MB in all), so that they come from HBM
        cells = []
        for (n3, k3) in ((4096, 4096), (11008, 4096), (4096, 11008), (28672, 8192)):
            g3 = torch.Generator(device="cpu").manual_seed(n3 + k3)
            w0 = (torch.randn(n3, k3, generator=g3) * 0.02).half().cuda()
            wc = [w0] + [w0.clone() for _ in range(int(512e6 / (n3 * k3 * 2)) + 1)]
            for m3 in (1, 16, 64, 256):
                a3 = (torch.randn(m3, k3, generator=g3) * 0.02).half().cuda()
                c3 = torch.empty(m3, n3, dtype=torch.float16, device="cuda")
                p3 = streamk.make_plan(m3, n3, k3, "float16", "nt")
                ws3 = wc if m3 <= 64 else wc[:1]
                turn = [0]

                def ours3():
                    turn[0] += 1
                    streamk.streamk_fp16(a3, ws3[turn[0] % len(ws3)], out=c3, plan=p3)

                def vendor3():
                    turn[0] += 1
                    torch.matmul(a3, ws3[turn[0] % len(ws3)].T, out=c3)
                t_o, t_v = time_graph(ours3, launches=10), time_graph(vendor3, launches=10)
                nbytes = 2.0 * (m3 * k3 + n3 * k3 + m3 * n3)
                cells.append({"M": m3, "N": n3, "K": k3, "us": round(t_o * 1e3, 2), "torch_matmul_us": round(t_v * 1e3, 2),
                              "ratio": round(t_o / t_v, 3), "gbs": round(nbytes / t_o / 1e6, 1),
                              "kernel": streamk.kernel_name(p3.kernel_id)})
            del wc, w0
        extra["small_m_sweep"] = cells

        # bfloat16 at the headline shape, both layouts, against the vendor GEMM in interleaved rounds
        bf = []
        ab, bb = A.bfloat16(), B.bfloat16()
        bbt = bb.T.contiguous()
        cb = torch.empty(M, N, dtype=torch.bfloat16, device="cuda")
        for layout, bmat in (("nt", bb), ("nn", bbt)):
            pb16 = streamk.make_plan(M, N, K, "bfloat16", layout)
            fns = {"tuned": lambda: streamk.streamk_bf16(ab, bmat, layout=layout, out=cb, plan=pb16),
                   "torch_matmul": lambda: torch.matmul(ab, bmat.T if layout == "nt" else bmat, out=cb)}
            best = {}
            for _ in range(3):
                for name, fn in fns.items():
                    best[name] = min(best.get(name, 1e9), time_eager(fn, 3, 10)[0])
            bf.append({"shape": [M, N, K], "layout": layout, "kernel": streamk.kernel_name(pb16.kernel_id),
                       **{name: {"us": round(ms * 1e3, 1), "tflops": round(flops / ms / 1e9, 1)} for name, ms in best.items()}})
        del ab, bb, bbt, cb
        extra["bf16_dense"] = bf

        extra["q4_note"] = ("34.6 MB of weights stay in the 256 MB Infinity Cache between launches of one weight "
                            "matrix; tuned_weights_from_hbm cycles through 20 copies so that every launch reads HBM")
        streamk.workspace_status()
        # the metric's other two parts in short, where the record of a run keeps them
        parts = {"streamk_vs_data_parallel_N8192_K8192": {}, "q4_gemm_N8192_K8192": {}, "few_rows_fp16_N8192_K8192": {}}
        for row in sweep:
            if row["M"] in (16, 64):   # (weights from HBM; the vendor GEMM on the same rotation of weights beside it)
                parts["few_rows_fp16_N8192_K8192"][f"M{row['M']}"] = {
                    "us_weights_from_hbm": row["auto_weights_from_hbm_us"], "frac_hbm": row["frac_hbm"],
                    "torch_matmul_us": row["torch_matmul_weights_from_hbm_us"]}
            if row["M"] in (256, 512, 1024):
                parts["streamk_vs_data_parallel_N8192_K8192"][f"M{row['M']}"] = {
                    "auto_tflops": row["auto"], "auto_tile": row["auto_tile"], "auto_fixup": row["auto_fixup"],
                    "sk_over_dp_same_tile": row["sk_over_dp_same_tile"], "auto_over_best_dp": row["auto_over_best_dp"],
                    "fp32_reduce_over_best_dp": round(max(row.get("sk_" + t, 0.0) for t in ("128", "128x256", "256")) /
                                                      max(v for k, v in row.items() if k.startswith("dp_")), 3)}
        for row in q4:
            parts["q4_gemm_N8192_K8192"][f"M{row['M']}"] = {
                "us_weights_in_infinity_cache": row["tuned"]["us"], "frac_hbm_weights_in_infinity_cache": row["tuned"]["frac_hbm"],
                "us_weights_from_hbm": row["tuned_weights_from_hbm"]["us"], "frac_hbm_weights_from_hbm": row["tuned_weights_from_hbm"]["frac_hbm"]}
        parts["small_m_sweep_16_cells"] = {
            "cells_at_or_below_torch_matmul": sum(1 for c in cells if c["ratio"] <= 1.0),
            "geomean_time_over_torch_matmul": round(float(np.exp(np.mean([np.log(c["ratio"]) for c in cells]))), 3),
            "worst": max(cells, key=lambda c: c["ratio"])}
        out["config"]["metric_parts"] = parts
        out["extra"] = extra

    print(json.dumps(out))


if __name__ == "__main__":
    main()

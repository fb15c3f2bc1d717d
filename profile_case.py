"""Runs one GEMM case a few times so that a profiler sees nothing else.

    rocprofv3 --kernel-trace --stats -- python3 profile_case.py 8192x8192x8192
    python3 profile_case.py 1x8192x8192 --dtype q4 --config "dict(grid=256)"
    python3 profile_case.py 8192x8192x8192 --data zeros --time --vendor

--data chooses the operand values (the clock the part sustains depends on how many bits toggle);
--time prints the average time of --reps launches; --vendor also times torch.matmul (hipBLASLt) on the
same operands.
"""
import argparse
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "stream-k.tvm_amd"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("shape", help="MxNxK")
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16", "float32", "q4", "float8_e4m3", "int8"])
    ap.add_argument("--layout", default="nt", choices=["nt", "nn"])
    ap.add_argument("--config", default="{}", help="python dict of plan options, e.g. \"dict(bm=256,bn=256,raster=8)\"")
    ap.add_argument("--reps", type=int, default=5)
    ap.add_argument("--data", default="rand", choices=["rand", "zeros", "ones"])
    ap.add_argument("--time", action="store_true")
    ap.add_argument("--vendor", action="store_true")
    args = ap.parse_args()
    import torch
    import streamk

    M, N, K = (int(x) for x in args.shape.split("x"))
    cfg = eval(args.config, {"dict": dict})  # noqa: S307 (developer tool)
    g = torch.Generator(device="cpu").manual_seed(0)
    plan = streamk.make_plan(M, N, K, args.dtype, args.layout, cfg)
    if args.dtype == "q4":
        A = torch.randn(M, K, generator=g).half().cuda()
        Wq = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8).cuda()
        sc = (torch.rand(N, K // 128, generator=g) * 0.015 + 0.005).half().cuda()
        run = lambda: streamk.streamk_q4(A, Wq, sc, plan=plan)  # noqa: E731
    elif args.dtype == "int8":
        if args.data == "rand":
            A = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8).cuda()
            B = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8).cuda()
        else:
            fill = torch.zeros if args.data == "zeros" else torch.ones
            A, B = fill(M, K, dtype=torch.int8, device="cuda"), fill(N, K, dtype=torch.int8, device="cuda")
        C = torch.empty(M, N, dtype=torch.int32, device="cuda")
        run = lambda: streamk.streamk_int8(A, B, out=C, plan=plan)  # noqa: E731
    elif args.dtype == "float8_e4m3":
        f8 = torch.float8_e4m3fn
        if args.data == "rand":
            A = (torch.rand(M, K, generator=g) * 2 - 1).cuda().to(f8)
            B = (torch.rand(N, K, generator=g) * 2 - 1).cuda().to(f8)
        else:
            fill = torch.zeros if args.data == "zeros" else torch.ones
            A, B = fill(M, K, device="cuda").to(f8), fill(N, K, device="cuda").to(f8)
        C = torch.empty(M, N, dtype=torch.float16, device="cuda")
        run = lambda: streamk.streamk_fp8(A, B, out=C, plan=plan)  # noqa: E731
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
        run = lambda: fn(A, B, layout=args.layout, out=C, plan=plan)  # noqa: E731
    for _ in range(args.reps):
        run()
    torch.cuda.synchronize()
    streamk.workspace_status()
    if args.time:
        ms = streamk.bench_ms(run, 3, args.reps)
        print(f"{args.data}: {ms * 1e3:.2f} us, {2.0 * M * N * K / ms / 1e9:.0f} TFLOP/s")
        if args.vendor and args.dtype == "float8_e4m3":
            one = torch.ones(1, device="cuda")
            ms = streamk.bench_ms(lambda: torch._scaled_mm(A, B.T, scale_a=one, scale_b=one, out_dtype=torch.float16), 3, args.reps)
            print(f"{args.data}: torch._scaled_mm {ms * 1e3:.2f} us, {2.0 * M * N * K / ms / 1e9:.0f} TFLOP/s")
        elif args.vendor and args.dtype == "int8":
            ms = streamk.bench_ms(lambda: torch._int_mm(A, B.T), 3, args.reps)
            print(f"{args.data}: torch._int_mm {ms * 1e3:.2f} us, {2.0 * M * N * K / ms / 1e9:.0f} TOP/s")
        elif args.vendor and args.dtype != "q4":
            Bt = B.T if args.layout == "nt" else B
            ms = streamk.bench_ms(lambda: torch.matmul(A, Bt, out=C), 3, args.reps)
            print(f"{args.data}: torch.matmul {ms * 1e3:.2f} us, {2.0 * M * N * K / ms / 1e9:.0f} TFLOP/s")
    print(f"ran {args.reps} x {args.dtype} {args.layout} {M}x{N}x{K} kernel {plan.kernel_id} grid {plan.grid} "
          f"streamk_tiles {plan.streamk_tiles}")


if __name__ == "__main__":
    main()

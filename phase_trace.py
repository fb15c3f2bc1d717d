"""Per-CTA phase timeline of a small-M kernel, from the tracing build of the library.

    make -C stream-k.tvm_amd/csrc trace
    python3 phase_trace.py 1x8192x8192 --dtype q4 --config "dict(bm=16,bn=16,bk=1024,schedule='dp')"

Thread 0 of every CTA stores the shader cycle counter at fixed points (SK_TRACE in the kernels);
the counters of different CUs are not synchronised, so every time is relative to the CTA's own
first stamp.  Prints min / median / max over the CTAs, converted with --ghz.
"""
import argparse
import ctypes
import os
import sys

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "stream-k.tvm_amd"))

NAMES = {0: "kernel entry", 10: "CTA range known", 11: "tile coordinates known", 1: "segment entered",
         2: "prologue loads issued", 3: "A staged", 4: "scales staged", 5: "barrier passed", 6: "loop entered",
         7: "loop left", 8: "before the store of C", 9: "after the store of C"}
ORDER = [0, 10, 11, 1, 2, 3, 4, 5, 6, 7, 8, 9]


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("shape", help="MxNxK")
    ap.add_argument("--dtype", default="q4", choices=["float16", "q4"])
    ap.add_argument("--config", default="{}")
    ap.add_argument("--ghz", type=float, default=2.1, help="shader clock used to convert cycles")
    args = ap.parse_args()
    import numpy as np
    import torch
    import streamk._lib as _lib
    _lib.LIB_PATH = os.path.join(os.path.dirname(_lib.LIB_PATH), "libstreamk_trace.so")
    import streamk

    M, N, K = (int(x) for x in args.shape.split("x"))
    cfg = eval(args.config, {"dict": dict})  # noqa: S307 (developer tool)
    plan = streamk.make_plan(M, N, K, args.dtype, "nt", cfg)
    g = torch.Generator(device="cpu").manual_seed(0)
    A = torch.randn(M, K, generator=g).half().cuda()
    C = torch.empty(M, N, dtype=torch.float16, device="cuda")
    if args.dtype == "q4":
        Wq = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8).cuda()
        sc = (torch.rand(N, K // 128, generator=g) * 0.015 + 0.005).half().cuda()
        run = lambda: streamk.streamk_q4(A, Wq, sc, out=C, plan=plan)  # noqa: E731
    else:
        B = torch.randn(N, K, generator=g).half().cuda()
        run = lambda: streamk.streamk_fp16(A, B, out=C, plan=plan)  # noqa: E731
    for _ in range(5):
        run()
    torch.cuda.synchronize()
    run()
    torch.cuda.synchronize()
    buf = np.zeros(2048 * 16, dtype=np.int64)
    rc = streamk.lib().sk_debug_trace_read(buf.ctypes.data_as(ctypes.c_void_p))
    assert rc == 0, rc
    t = buf.reshape(2048, 16)[:min(plan.grid, 2048)].astype(np.float64)
    t = (t - t[:, 0:1]) / (args.ghz * 1e3)  # microseconds since the CTA's own entry
    print(f"kernel {plan.kernel_id}, grid {plan.grid}, times in us at {args.ghz} GHz")
    for slot in ORDER:
        col = t[:, slot]
        if np.all(col <= 0) and slot != 0:
            continue  # a stamp this kernel family does not have
        print(f"  {NAMES[slot]:26s} min {col.min():6.2f}  median {np.median(col):6.2f}  max {col.max():6.2f}")


if __name__ == "__main__":
    main()

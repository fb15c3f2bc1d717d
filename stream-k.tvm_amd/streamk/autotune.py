"""Per-shape autotuner over tile / kernel variant / schedule / grid / fix-up.

Plays the role of the reference's `@autotune(configs=...) @jit(...)` loop
(autotune/streamk_fp16_autotune.py:38-53, 88-95, 373-386): enumerate configurations, time each,
keep the fastest and return `(best_latency, best_config, ref_latency)`.  Here no code is
generated per configuration: every candidate is a (kernel instance, partition) pair of the already
built library, so a search costs milliseconds per candidate.

Results are kept in a JSON cache keyed by (arch, dtype, layout, M, N, K); `plan.make_plan` consults
the cache when the caller gives no configuration.
"""
import itertools
import json
import os

import torch

from . import ops, plan as _plan
from ._lib import StreamKError

_HERE = os.path.dirname(os.path.abspath(__file__))
DEFAULT_CACHE = os.path.join(_HERE, "tuned", "gfx950.json")
USER_CACHE_ENV = "STREAMK_TUNE_CACHE"

_TILES_F16 = [(256, 256, 64), (128, 128, 64), (128, 256, 64), (256, 128, 64), (64, 64, 64), (128, 64, 64),
              (64, 128, 64)]
_SKINNY_F16 = [(16, 64, 128), (32, 64, 128), (64, 64, 128), (16, 16, 512), (16, 32, 256), (16, 16, 128),
               (16, 16, 1024), (16, 32, 512), (16, 16, 256), (16, 64, 256), (32, 64, 256), (64, 64, 256)]
# fp16 / bfloat16 weights streamed through LDS in contiguous loads (variant 5 of these shapes)
_STREAM_F16 = [(16, 16, 1024), (16, 32, 512), (16, 64, 256), (32, 32, 256), (32, 64, 256), (64, 32, 256), (64, 64, 256),
               (96, 32, 256)]
_SKINNY_F8 = [(16, 64, 256), (32, 64, 256), (16, 16, 1024), (16, 32, 512), (16, 32, 1024), (16, 64, 512), (32, 64, 512),
              (64, 64, 256), (64, 64, 512)]
_SKINNY_Q4 = [(16, 64, 256), (32, 64, 256), (64, 64, 256), (16, 16, 1024), (16, 32, 512), (16, 16, 256),
              (16, 32, 256), (16, 32, 1024), (16, 16, 2048), (16, 64, 512), (16, 16, 512)]


def _key(dtype, layout, M, N, K):
    return f"gfx950/{dtype}/{layout}/{M}x{N}x{K}"


def load_cache(path=None):
    path = path or os.environ.get(USER_CACHE_ENV) or DEFAULT_CACHE
    try:
        with open(path) as f:
            return json.load(f)
    except (OSError, ValueError):
        return {}


def save_cache(cache, path=None):
    path = path or os.environ.get(USER_CACHE_ENV) or DEFAULT_CACHE
    os.makedirs(os.path.dirname(path), exist_ok=True)
    with open(path, "w") as f:
        json.dump(cache, f, indent=1, sort_keys=True)


def candidate_configs(M, N, K, dtype="float16", cus=None, reduce16=True):
    """The search space.  The reference multiplies out warp/chunk/stage lists
    (autotune/streamk_fp16_autotune.py:38-53); here the axes are tile shape, kernel variant,
    schedule, grid and fix-up.  reduce16=False leaves out the candidates that exchange partial sums rounded to 16
    bits (fixup 'reduce16': within the 1e-2 every candidate is held to, but not the fp32 sums of the other fix-ups)."""
    cus = cus or _plan.num_cus()
    out = []
    f8 = dtype in ("float8_e4m3", "float8_e5m2", "int8")  # one-byte operands
    if dtype in ("q4", "q4_zp") or M <= 64:
        tiles = _SKINNY_Q4 if dtype in ("q4", "q4_zp") else (_SKINNY_F8 if f8 else _SKINNY_F16)
        for (bm, bn, bk) in tiles:
            if bm < M and not (bm == 16 and M <= 16):
                continue
            if bm >= 2 * M and bm > 16:
                continue
            out.append(dict(bm=bm, bn=bn, bk=bk, schedule="dp"))
            for grid, fixup in itertools.product((cus, 2 * cus, 4 * cus), ("reduce", "atomic")):
                out.append(dict(bm=bm, bn=bn, bk=bk, schedule="sk2", grid=grid, fixup=fixup))
            # 2 <= M <= 4: these tiles resolve to the matrix-vector form with four rows of A; the general kernel
            # of the same tile stays in the search as variant 1
            if 2 <= M <= 4 and dtype in ("float16", "bfloat16") and (bm, bn, bk) in ((16, 16, 512), (16, 32, 512), (16, 64, 256)):
                out.append(dict(bm=bm, bn=bn, bk=bk, variant=1, schedule="dp"))
                for grid in (cus, 2 * cus):
                    out.append(dict(bm=bm, bn=bn, bk=bk, variant=1, schedule="sk2", grid=grid, fixup="reduce"))
    if dtype == "q4" and M <= 16 and K % 256 == 0:
        # row-major Q4 weights streamed through LDS in contiguous loads (variant 5 of these shapes)
        for (bm, bn, bk) in ((16, 64, 512), (16, 32, 1024)):
            base = dict(bm=bm, bn=bn, bk=bk, variant=5)
            out.append(dict(base, schedule="dp"))
            for sched, fixup in (("sk2", "reduce"), ("basic", "reduce"), ("basic", "atomic")):
                out.append(dict(base, schedule=sched, grid=cus, fixup=fixup))
    if dtype in ("float16", "bfloat16") and M <= 96:
        for (bm, bn, bk) in _STREAM_F16:
            if bm < M or (bm >= 2 * M and bm > 16):
                continue
            base = dict(bm=bm, bn=bn, bk=bk, variant=5)
            out.append(dict(base, schedule="dp"))
            for sched, fixup in (("sk2", "reduce"), ("sk1", "reduce"), ("basic", "reduce"), ("basic", "atomic")):
                out.append(dict(base, schedule=sched, grid=cus, fixup=fixup))
    if dtype in ("float16", "bfloat16") and M > 16:
        for (bm, bn, bk) in _TILES_F16:
            # (variant, bk): direct-to-LDS two-stage, register-staged, direct-to-LDS four-stage, 16x16x32 form
            variants = ((2, bk), (1, bk), (4, 32)) if bm * bn > 64 * 128 else ((2, bk), (4, 32))
            variants += ((6, 32),)  # four-stage with 16x16x32 MFMAs
            if bm >= 128 and bn >= 128:
                variants += ((5, bk),)  # two-stage with 16x16x32 MFMAs
            if (bm, bn) == (256, 256):
                # 256 x 256 tiles: four waves with the K loop in assembly, or the eight-wave 16x16x32 kernel for other K
                variants = ((5, bk),) + (((8, bk),) if K % 64 == 0 else ())
            if (bm, bn) == (64, 64):
                variants += ((1, bk),)
            for (variant, vbk), raster in itertools.product(variants, (1, 8)):
                base = dict(bm=bm, bn=bn, bk=vbk, variant=variant, raster=raster)
                out.append(dict(base, schedule="dp"))
                grids = (None,) if bm * bn >= 256 * 256 else (None, cus)
                for sched, fixup, grid in itertools.product(("sk2", "sk1", "basic"), ("reduce", "atomic"), grids):
                    out.append(dict(base, schedule=sched, fixup=fixup, **({"grid": grid} if grid else {})))
                # the interleaved order of the Stream-K tiles (CTAs at the same K offset on neighbouring tiles)
                if raster == 8 and bm * bn >= 128 * 128:
                    out.extend(dict(base, schedule=sched, fixup="reduce", interleave=1) for sched in ("sk2", "basic"))
                # fixed split-K, the fallback when there are fewer tiles than CUs
                if -(-M // bm) * -(-N // bn) < cus:
                    out.extend(dict(base, schedule="splitk", fixup=fixup) for fixup in ("reduce", "atomic"))
                    out.append(dict(base, schedule="splitk", split=2, fixup="reduce"))
                    # the exchange of half tiles with the partial sums rounded to 16 bits (assembly-loop kernel)
                    if variant == 8 and reduce16:
                        out.append(dict(base, schedule="splitk", fixup="reduce16"))
                        out.append(dict(base, schedule="splitk", split=2, fixup="reduce16"))
    if dtype in ("float8_e4m3", "float8_e5m2", "int8"):
        # (bk 0: the tile's default, two stages of 128 K-values; 64: four stages of 64)
        tiles = [(256, 256, 0), (256, 128, 0), (128, 256, 0), (128, 128, 0), (64, 128, 0), (128, 128, 64), (64, 128, 64)]
        for (bm, bn, bk), raster in itertools.product(tiles, (1, 8)):
            base = dict(bm=bm, bn=bn, raster=raster, **({"bk": bk} if bk else {}))
            out.append(dict(base, schedule="dp"))
            for sched, fixup in itertools.product(("sk2", "sk1", "basic"), ("reduce", "atomic")):
                out.append(dict(base, schedule=sched, fixup=fixup))
            if raster == 8:
                out.extend(dict(base, schedule=sched, fixup="reduce", interleave=1) for sched in ("sk2", "basic"))
            if -(-M // bm) * -(-N // bn) < cus:
                out.extend(dict(base, schedule="splitk", fixup=fixup) for fixup in ("reduce", "atomic"))
                out.append(dict(base, schedule="splitk", split=2, fixup="reduce"))
    return out


_MIN_TIMED_MS = 8.0  # a candidate is timed over at least this much GPU time

_box_reference = None


def box_reference_tflops():
    """What this box sustains on one fixed launch (fp16 4096^3 NT, the eight-wave 256 x 256 data-parallel kernel,
    U[-1,1) operands), measured once per process.  Boxes of one pool differ by more than 10 % on compute-bound
    shapes; stored beside every cache entry, the figure shows on which kind of box the entry's latency was taken."""
    global _box_reference
    if _box_reference is None:
        g = torch.Generator(device="cpu").manual_seed(1)
        A = (torch.rand(4096, 4096, generator=g) * 2 - 1).half().cuda()
        C = torch.empty(4096, 4096, dtype=torch.float16, device="cuda")
        p = _plan.make_plan(4096, 4096, 4096, "float16", "nt", dict(bm=256, bn=256, bk=64, variant=5, schedule="dp", raster=8))
        ms = _time_ms(lambda: ops.streamk_fp16(A, A, out=C, plan=p), 5, 10, True, min_ms=40.0)
        _box_reference = round(2.0 * 4096 ** 3 / ms / 1e9, 1)
    return _box_reference


def _time_ms(fn, warmup, rep, graph, min_ms=None):
    """Per-launch time in ms.  The part sets its clock by the power drawn over the last milliseconds, so a burst
    of 20 launches of a compute-bound kernel runs up to 20 % faster than the same kernel sustained; a measurement
    therefore runs for at least `min_ms` (default _MIN_TIMED_MS), the first half untimed.  With `graph` (microsecond
    kernels) the launches are captured and the median of seven groups over a longer window is taken (ops.graph_ms)."""
    min_ms = _MIN_TIMED_MS if min_ms is None else min_ms
    if not graph:
        ms = ops.bench_ms(fn, warmup, rep)
        more = int(min_ms / max(ms, 1e-4)) + 1
        if more > 2 * rep:
            ms = ops.bench_ms(fn, more // 2, more // 2)
        return ms
    return ops.graph_ms(fn, launches=rep, warmup=warmup, window_ms=max(3.0 * min_ms, 24.0), groups=7)


def autotune(M, N, K, dtype="float16", layout="nt", *, configs=None, warmup=5, rep=20, check=True,
             cache=True, cache_path=None, verbose=False, weights=None, reduce16=True):
    """Searches `configs` (default: candidate_configs) for the fastest plan.

    weights="hbm" times every candidate on a rotation of copies of the weight operand (more than
    512 MB in total), so that each launch reads its weights from HBM as a layer of a model larger
    than the 256 MB Infinity Cache does; weights="warm" reuses one copy.  Default: "hbm" for
    M <= 64, where the launch is a stream over the weights, "warm" otherwise.

    Returns (best_latency_ms, best_config, ref_latency_ms); ref is torch.matmul on the same GPU, the
    reference's comparator (streamk_fp16.py:396) -- None for Q4.  Every candidate is checked against
    the first valid one (max-abs-rel 1e-2) unless check=False, mirroring `skip_check` of the
    reference's jit decorator.  reduce16=False keeps the candidates with 16-bit partial sums out of the search."""
    dev = "cuda"
    g = torch.Generator(device="cpu").manual_seed(0)
    A = (torch.rand(M, K, generator=g) * 2 - 1).half().to(dev)
    C = torch.empty(M, N, dtype=torch.float16, device=dev)
    weights = weights or ("hbm" if M <= 64 else "warm")
    wbytes = N * K // 2 if dtype in ("q4", "q4_zp") else (N * K if dtype in ("float8_e4m3", "float8_e5m2", "int8") else N * K * 2)
    copies = 1 if weights == "warm" else max(2, min(rep, -(-(512 << 20) // wbytes)))
    turn = [0]

    def rotate(items):
        turn[0] += 1
        return items[turn[0] % len(items)]
    if dtype in ("q4", "q4_zp"):
        Wq = torch.randint(0, 256, (N, K // 2), generator=g, dtype=torch.uint8).to(dev)
        sc = (torch.rand(N, K // 128, generator=g) * 0.015 + 0.005).half().to(dev)
        Ws = [(Wq, sc)] + [(Wq.clone(), sc.clone()) for _ in range(copies - 1)]
        if dtype == "q4_zp":
            zp = torch.randint(0, 16, (N, K // 128), generator=g).half().to(dev)
            run = lambda p: ops.streamk_q4(A, *rotate(Ws), zeros=zp, out=C, plan=p)  # noqa: E731
        else:
            run = lambda p: ops.streamk_q4(A, *rotate(Ws), out=C, plan=p)  # noqa: E731
        ref_ms = None
    elif dtype in ("float8_e4m3", "float8_e5m2"):
        f8 = torch.float8_e4m3fn if dtype == "float8_e4m3" else torch.float8_e5m2
        A8 = A.to(f8)
        B8 = (torch.rand(N, K, generator=g) * 2 - 1).to(dev).to(f8)
        Bs = [B8] + [B8.clone() for _ in range(copies - 1)]
        run = lambda p: ops.streamk_fp8(A8, rotate(Bs), out=C, plan=p)  # noqa: E731
        one = torch.ones(1, device=dev)
        try:   # hipBLASLt's fp8 GEMM, where this torch build has it
            ref_ms = _time_ms(lambda: torch._scaled_mm(A8, rotate(Bs).T, scale_a=one, scale_b=one, out_dtype=torch.float16),
                              warmup, rep, 2.0 * M * N * K < 5e11)
        except Exception:
            ref_ms = None
    elif dtype == "int8":
        Ai = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8).to(dev)
        Bi = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8).to(dev)
        Bs = [Bi] + [Bi.clone() for _ in range(copies - 1)]
        C = torch.empty(M, N, dtype=torch.int32, device=dev)
        run = lambda p: ops.streamk_int8(Ai, rotate(Bs), out=C, plan=p)  # noqa: E731
        try:   # the vendor's int8 GEMM, where this torch build has it
            ref_ms = _time_ms(lambda: torch._int_mm(Ai, rotate(Bs).T), warmup, rep, 2.0 * M * N * K < 5e11)
        except Exception:
            ref_ms = None
    else:
        bshape = (N, K) if layout == "nt" else (K, N)
        # (bfloat16: the twins of the fp16 kernels; candidates whose kernel has no twin are skipped below)
        tdt, gemm = (torch.bfloat16, ops.streamk_bf16) if dtype == "bfloat16" else (torch.float16, ops.streamk_fp16)
        A, C = A.to(tdt), C.to(tdt)
        B = (torch.rand(*bshape, generator=g) * 2 - 1).to(tdt).to(dev)
        Bs = [B] + [B.clone() for _ in range(copies - 1)]
        run = lambda p: gemm(A, rotate(Bs), layout=layout, out=C, plan=p)  # noqa: E731
        small = 2.0 * M * N * K < 5e11
        as_b = (lambda b: b.T) if layout == "nt" else (lambda b: b)
        ref_ms = _time_ms(lambda: torch.matmul(A, as_b(rotate(Bs)), out=C), warmup, rep, small)
    small = 2.0 * M * N * K < 5e11  # microsecond kernels: time graph-captured batches
    configs = configs if configs is not None else candidate_configs(M, N, K, dtype, reduce16=reduce16)
    best, golden, results = None, None, []
    for cfg in configs:
        try:
            p = _plan.make_plan(M, N, K, dtype, layout, cfg)
            if cfg.get("schedule", "dp") != "dp" and p.streamk_tiles == 0:
                continue  # the grid leaves no tile to split: this candidate is the data-parallel one under another name
            if cfg.get("interleave") and p.interleave <= 1:
                continue  # every CTA is at its own K offset, or all at the same one: the order changes nothing
            run(p)
            torch.cuda.synchronize()
            ops.workspace_status()
        except StreamKError as e:
            if e.status == -8:
                ops.reset_workspaces()
            continue
        if check:
            if golden is None:
                golden = C.float().clone()
            else:
                err = (C.float() - golden).abs().max().item() / max(golden.abs().max().item(), 1e-30)
                if err > 1e-2:
                    raise AssertionError(f"config {cfg} disagrees with the first candidate: {err}")
        ms = _time_ms(lambda: run(p), warmup, rep, small)
        results.append((ms, cfg))
        if verbose:
            print(f"  {ms * 1e3:9.2f} us  {cfg}")
        if best is None or ms < best[0]:
            best = (ms, cfg)
    if best is None:
        raise RuntimeError(f"no valid configuration for {M}x{N}x{K} {dtype}/{layout}")
    # Microsecond kernels: one timing of a candidate is good to a few percent, which is also what separates the
    # leaders.  The five best (and the best data-parallel one) are timed again, twice, in alternation; a candidate's
    # figure is the smaller of the two.
    if small and len(results) > 1:
        results.sort(key=lambda r: r[0])
        finalists = results[:5] + [r for r in results[5:] if r[1].get("schedule") == "dp"][:1]
        again = {id(r): [] for r in finalists}
        for _ in range(2):
            for r in finalists:
                p = _plan.make_plan(M, N, K, dtype, layout, r[1])
                again[id(r)].append(_time_ms(lambda: run(p), warmup, 2 * rep, small))
        results = [(min(again[id(r)]), r[1]) for r in finalists]
        best = min(results, key=lambda r: r[0])
        if verbose:
            for ms, cfg in sorted(results, key=lambda r: r[0]):
                print(f"  again {ms * 1e3:9.2f} us  {cfg}")
    # within the noise of the measurement prefer a data-parallel plan: no workspace, no fix-up code in the kernel
    near = [r for r in results if r[0] <= best[0] * (1.03 if small else 1.015) and r[1].get("schedule") == "dp"]
    if near and best[1].get("schedule") != "dp":
        best = min(near, key=lambda r: r[0])
    if cache:
        c = load_cache(cache_path)
        c[_key(dtype, layout, M, N, K)] = {"config": best[1], "latency_ms": best[0], "ref_latency_ms": ref_ms,
                                           "box_reference_tflops": box_reference_tflops()}
        save_cache(c, cache_path)
        _plan.invalidate_tuned_cache()
    return best[0], best[1], ref_ms

"""GPU parity tests: the HIP path, called through the C ABI, against the CPU oracle on the same
seeded inputs, against the committed fixtures, and through size-independent properties at the
full benchmark sizes.

Tolerance for fp16-out / fp32-accumulate GEMMs: max|C - ref| / max|ref| <= 1e-2 against an fp32 host
matmul (the reference asserts rtol = atol = 1e-2, streamk_fp32.py:208).  Q4 dequantisation and the
ordered-reduce fix-up are checked bit for bit.
"""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope="module")
def sk():
    import torch
    assert torch.cuda.is_available(), "these tests need the MI355X"
    import streamk
    streamk.lib()
    maps = open("/proc/self/maps").read()
    assert "libstreamk.so" in maps, "native library not loaded"
    return streamk


def _t(x):
    import torch
    return torch.from_numpy(np.ascontiguousarray(x)).cuda()


def _uniform16(shape, seed):
    # uniform [-1, 1) rounded to fp16 (streamk_fp16.py:65-67 draws rand*2-1)
    rng = np.random.default_rng(seed)
    return (rng.random(shape, dtype=np.float32) * 2 - 1).astype(np.float16)


def _rel(oracle, C, ref):
    return oracle.max_abs_rel(C.float().cpu().numpy(), ref)


# variant 1: registers -> padded LDS rows; 2: direct-to-LDS, eight (four) waves, 32x32x16 MFMAs; 4: direct-to-LDS with
# BK = 32 and four stages; 5: direct-to-LDS, 16x16x32 MFMAs; 6: as 4 with 16x16x32 MFMAs.  256 x 256 tiles exist as
# variant 5 (the eight-wave kernel for K that the assembly-loop kernel, variant 8, does not take) and variant 8.
TILE_CONFIGS = [
    dict(bm=128, bn=128, bk=64, variant=1),
    dict(bm=128, bn=256, bk=64, variant=1), dict(bm=256, bn=128, bk=64, variant=1),
    dict(bm=64, bn=64, bk=64, variant=1), dict(bm=128, bn=128, bk=32),
    dict(bm=128, bn=128, bk=64, variant=2),
    dict(bm=128, bn=256, bk=64, variant=2), dict(bm=256, bn=128, bk=64, variant=2),
    dict(bm=128, bn=128, bk=32, variant=4),
    dict(bm=128, bn=256, bk=32, variant=4), dict(bm=256, bn=128, bk=32, variant=4),
    dict(bm=64, bn=64, bk=64, variant=2), dict(bm=128, bn=64, bk=64, variant=2), dict(bm=64, bn=128, bk=64, variant=2),
    dict(bm=64, bn=64, bk=32, variant=4), dict(bm=128, bn=64, bk=32, variant=4), dict(bm=64, bn=128, bk=32, variant=4),
    dict(bm=128, bn=128, bk=64, variant=5), dict(bm=256, bn=256, bk=64, variant=5),
    dict(bm=128, bn=256, bk=64, variant=5), dict(bm=256, bn=128, bk=64, variant=5),
    dict(bm=128, bn=128, bk=32, variant=6),
    dict(bm=128, bn=256, bk=32, variant=6), dict(bm=256, bn=128, bk=32, variant=6),
    dict(bm=64, bn=64, bk=32, variant=6), dict(bm=128, bn=64, bk=32, variant=6), dict(bm=64, bn=128, bk=32, variant=6),
]
SKINNY_CONFIGS = [
    dict(bm=16, bn=64, bk=128), dict(bm=32, bn=64, bk=128), dict(bm=64, bn=64, bk=128),
    dict(bm=16, bn=16, bk=512), dict(bm=16, bn=32, bk=256),
    dict(bm=16, bn=32, bk=512, variant=1), dict(bm=16, bn=64, bk=256), dict(bm=32, bn=64, bk=256), dict(bm=64, bn=64, bk=256),
]
# variant 5 of the small-M shapes: the weights stream through LDS in contiguous loads
STREAM_CONFIGS = [
    dict(bm=16, bn=64, bk=256, variant=5), dict(bm=32, bn=64, bk=256, variant=5), dict(bm=16, bn=32, bk=512, variant=5),
    dict(bm=64, bn=32, bk=256, variant=5), dict(bm=32, bn=32, bk=256, variant=5), dict(bm=64, bn=64, bk=256, variant=5),
    dict(bm=16, bn=16, bk=1024, variant=5), dict(bm=96, bn=32, bk=256, variant=5),
]


@pytest.mark.parametrize("cfg", TILE_CONFIGS + SKINNY_CONFIGS + STREAM_CONFIGS, ids=lambda c: f"{c['bm']}x{c['bn']}x{c['bk']}v{c.get('variant', 0)}")
@pytest.mark.parametrize("sched,fixup,grid", [("dp", "reduce", 8), ("basic", "reduce", 8),
                                             ("basic", "atomic", 8), ("sk2", "reduce", 3),
                                             ("sk2", "atomic", 5)])
def test_fixture_ragged_f16(sk, oracle, golden_dir, cfg, sched, fixup, grid):
    """200 x 136 x 328 (ragged in M, N and K for every tile shape) against the committed fixture;
    small grids force tiles to be split over several CTAs."""
    g = np.load(os.path.join(golden_dir, "gemm_f16_nt_200x136x328.npz"))
    A, B, ref = g["A"], g["B"], g["C"]
    if cfg["bm"] <= 96 and cfg["bn"] <= 64 and cfg["bk"] != 64:  # small-M kernels take M <= bm
        A, ref = A[:cfg["bm"] - 3], ref[:cfg["bm"] - 3]
    C = sk.streamk_fp16(_t(A), _t(B), schedule=sched, fixup=fixup, grid=grid, **cfg)
    sk.workspace_status()
    assert _rel(oracle, C, ref) <= 2e-3 <= TOL


@pytest.mark.parametrize("fixup", ["atomic", "reduce"])
@pytest.mark.parametrize("cfg", [dict(bm=128, bn=128, bk=64, grid=256), dict(bm=128, bn=128, bk=32, grid=256),
                                 dict(bm=256, bn=256, bk=64)],
                         ids=["128x128x64", "128x128x32", "256x256x64"])
def test_cfg2_streamk_both_fixups(sk, oracle, cfg, fixup):
    """M = N = 1024, K = 8192, NT, U[-1,1) seed 0: 64 tiles of 128x128 on 256 CUs, every tile split
    along K over 4 CTAs; both fix-ups against the oracle's fp32 host matmul."""
    A, B = _uniform16((1024, 8192), 0), _uniform16((1024, 8192), 1)
    ref = oracle.matmul_fp32(A, B, trans_b=True)
    plan = sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="sk2", fixup=fixup, **cfg)
    assert plan.streamk_tiles == plan.total_tiles and plan.blocking_tiles == 0
    C = sk.streamk_fp16(_t(A), _t(B), plan=plan)
    sk.workspace_status()
    assert _rel(oracle, C, ref) <= 1e-3 <= TOL


def test_four_equal_segments_two_round_exchange(sk, oracle):
    """Every Stream-K tile cut into four equal segments (fixed split 4, or `basic` on four CTAs per tile) with the
    ordered fix-up: the four CTAs exchange halves in two rounds and two of them finish half of C each.  Against the
    fp32 host product, exact on integer data, bitwise repeatable, equal between `splitk` and `basic` on the same grid,
    with ragged edges, a bias, data-parallel tiles beside the split ones, fp16 / bfloat16 / int8 / fp8, and after an
    ATOMIC launch on the same workspace."""
    import torch
    rng = np.random.default_rng(59)
    ran = 0
    for (M, N, K) in [(512, 512, 1024), (300, 700, 2048), (1000, 264, 512)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Ai, Bi = rng.integers(-1, 2, (M, K)).astype(np.float16), rng.integers(-1, 2, (N, K)).astype(np.float16)
        bias = (rng.random(N, dtype=np.float32) - 0.5).astype(np.float16)
        ref = oracle.matmul_fp32(A, B, trans_b=True)
        exact = Ai.astype(np.int32) @ Bi.astype(np.int32).T
        for layout in ("nt", "nn"):
            if layout == "nn" and N % 8:
                continue
            dB = _t(np.ascontiguousarray(B.T) if layout == "nn" else B)
            dBi = _t(np.ascontiguousarray(Bi.T) if layout == "nn" else Bi)
            for tile in (dict(bm=256, bn=256, bk=64, variant=8), dict(bm=256, bn=256, bk=64, variant=5), dict(bm=128, bn=128, bk=64, variant=5),
                         dict(bm=128, bn=256, bk=64, variant=5)):
                try:
                    plan = sk.make_plan(M, N, K, "float16", layout, dict(tile, schedule="splitk", split=4, fixup="reduce"))
                except sk.StreamKError:
                    continue
                assert plan.streamk_tiles == plan.total_tiles and 4 * plan.streamk_full_tiles == plan.iters_per_tile
                C = sk.streamk_fp16(_t(A), dB, layout=layout, plan=plan)
                assert _rel(oracle, C, ref) <= 1e-3 <= TOL, (M, N, K, layout, tile)
                assert torch.equal(C, sk.streamk_fp16(_t(A), dB, layout=layout, plan=plan))
                basic = sk.make_plan(M, N, K, "float16", layout, dict(tile, schedule="basic", grid=plan.grid, fixup="reduce"))
                assert torch.equal(C, sk.streamk_fp16(_t(A), dB, layout=layout, plan=basic))
                assert np.array_equal(sk.streamk_fp16(_t(Ai), dBi, layout=layout, plan=plan).cpu().numpy().astype(np.int32), exact)
                # an ATOMIC launch in between leaves the workspace fit for the next ordered launch
                atomic = sk.make_plan(M, N, K, "float16", layout, dict(tile, schedule="splitk", split=4, fixup="atomic"))
                assert _rel(oracle, sk.streamk_fp16(_t(A), dB, layout=layout, plan=atomic), ref) <= 1e-3
                assert torch.equal(C, sk.streamk_fp16(_t(A), dB, layout=layout, plan=plan))
                if layout == "nt":
                    Cb = sk.streamk_fp16(_t(A), dB, plan=plan, bias=_t(bias))
                    assert _rel(oracle, Cb, ref + bias.astype(np.float32)[None, :]) <= 1e-3
                ran += 1
    assert ran >= 14, ran
    # split tiles beside data-parallel ones: sk2 on a grid that gives every split tile four CTAs
    M, N, K = 1280, 1024, 2048   # 5 x 4 = 20 tiles of 256 x 256; grid 16: 4 Stream-K tiles over 16 CTAs, 16 data-parallel
    A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    plan = sk.make_plan(M, N, K, "float16", "nt", dict(bm=256, bn=256, bk=64, variant=8, schedule="sk1", grid=16, fixup="reduce"))
    assert plan.streamk_tiles == 4 and plan.blocking_tiles == 16 and 4 * plan.streamk_full_tiles == plan.iters_per_tile
    C = sk.streamk_fp16(_t(A), _t(B), plan=plan)
    assert _rel(oracle, C, oracle.matmul_fp32(A, B, trans_b=True)) <= 1e-3
    assert torch.equal(C, sk.streamk_fp16(_t(A), _t(B), plan=plan))
    # one-byte operands and bfloat16
    M, N, K = 512, 512, 2048
    Ai8, Bi8 = rng.integers(-128, 128, (M, K)).astype(np.int8), rng.integers(-128, 128, (N, K)).astype(np.int8)
    for bm in (256, 128):
        p8 = sk.make_plan(M, N, K, "int8", "nt", dict(bm=bm, bn=bm, schedule="splitk", split=4, fixup="reduce"))
        assert np.array_equal(sk.streamk_int8(_t(Ai8), _t(Bi8), plan=p8).cpu().numpy(), Ai8.astype(np.int32) @ Bi8.astype(np.int32).T)
    f8 = torch.float8_e4m3fn
    Af, Bf = torch.randn(M, K).to(f8), torch.randn(N, K).to(f8)
    pf = sk.make_plan(M, N, K, "float8_e4m3", "nt", dict(bm=256, bn=256, schedule="splitk", split=4, fixup="reduce"))
    Cf = sk.streamk_fp8(Af.cuda(), Bf.cuda(), plan=pf)
    assert _rel(oracle, Cf, oracle.f8_gemm_ref(Af.view(torch.uint8).numpy(), Bf.view(torch.uint8).numpy())) <= 2e-3
    assert torch.equal(Cf, sk.streamk_fp8(Af.cuda(), Bf.cuda(), plan=pf))
    Ab, Bb = torch.randn(M, K).bfloat16(), torch.randn(N, K).bfloat16()
    pb = sk.make_plan(M, N, K, "bfloat16", "nt", dict(bm=256, bn=256, bk=64, variant=8, schedule="splitk", split=4, fixup="reduce"))
    Cb = sk.streamk_bf16(Ab.cuda(), Bb.cuda(), plan=pb)
    assert _rel(oracle, Cb, oracle.matmul_fp32(Ab.float().numpy(), Bb.float().numpy(), trans_b=True)) <= 4e-3
    sk.workspace_status()


def test_whole_tile_ranges_need_no_workspace(sk, oracle):
    """A Stream-K schedule whose CTA ranges are whole tiles (`basic` on a tile count that is a multiple of the grid)
    only changes which tiles a CTA takes: the plan asks for no workspace and the result equals the data-parallel
    one bit for bit."""
    import torch
    rng = np.random.default_rng(53)
    M, N, K = 2048, 1024, 512
    A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    for tile in (dict(bm=256, bn=256, bk=64, variant=8), dict(bm=128, bn=128, bk=64, variant=5)):
        tiles = (M // tile["bm"]) * (N // tile["bn"])
        for fixup in ("reduce", "atomic"):
            plan = sk.make_plan(M, N, K, "float16", "nt", dict(tile, schedule="basic", fixup=fixup, grid=tiles // 4, raster=1))
            assert plan.streamk_tiles == tiles and plan.workspace_bytes == 0
            dp = sk.make_plan(M, N, K, "float16", "nt", dict(tile, schedule="dp"))
            C = sk.streamk_fp16(_t(A), _t(B), plan=plan)
            assert torch.equal(C, sk.streamk_fp16(_t(A), _t(B), plan=dp))
            assert _rel(oracle, C, oracle.matmul_fp32(A, B, trans_b=True)) <= 1e-3
    Ai, Bi = rng.integers(-8, 9, (M, K)).astype(np.int8), rng.integers(-8, 9, (N, K)).astype(np.int8)
    plan = sk.make_plan(M, N, K, "int8", "nt", dict(bm=256, bn=256, schedule="basic", fixup="reduce", grid=8))
    assert plan.workspace_bytes == 0
    assert np.array_equal(sk.streamk_int8(_t(Ai), _t(Bi), plan=plan).cpu().numpy(), Ai.astype(np.int32) @ Bi.astype(np.int32).T)
    sk.workspace_status()


def test_untuned_plans_on_ragged_shapes(sk, oracle):
    """The planner's own choice (no configuration, no tuned cache: cost model, aligned split, admitted Stream-K in
    raster and in interleaved tile order) on shapes that exercise each of its branches, ragged edges included: fp16 NT / NN and bfloat16 against the
    fp32 host product (1e-3 / 4e-3), int8 exactly."""
    import torch
    rng = np.random.default_rng(47)
    kinds, interleaved = set(), 0
    for (M, N, K) in [(65, 136, 328), (200, 1000, 1032), (384, 4096, 1024), (520, 2048, 4096), (768, 4096, 2048), (1000, 1096, 8192),
                      (1536, 11008, 1024), (2100, 4000, 512), (3000, 5120, 1024), (3000, 8192, 4096), (4096, 4096, 64), (1536, 11008, 4096),
                      (1024, 8192, 512), (512, 8192, 1024), (2990, 6104, 4096)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.matmul_fp32(A, B, trans_b=True)
        for layout in ("nt", "nn"):
            dB = _t(np.ascontiguousarray(B.T) if layout == "nn" else B)
            plan = sk.make_plan(M, N, K, "float16", layout, use_tuned=False)
            kinds.add((plan.schedule, plan.streamk_tiles > 0))
            interleaved += plan.interleave > 1
            C = sk.streamk_fp16(_t(A), dB, layout=layout, plan=plan)
            assert _rel(oracle, C, ref) <= 1e-3 <= TOL, (M, N, K, layout, sk.kernel_name(plan.kernel_id), plan.as_dict())
            if M * N * K > 5e9:   # (the host reference of the large shapes is computed once, for fp16)
                continue
            pb = sk.make_plan(M, N, K, "bfloat16", layout, use_tuned=False)
            Ab, Bb = torch.from_numpy(A).bfloat16(), torch.from_numpy(np.ascontiguousarray(B.T) if layout == "nn" else B).bfloat16()
            refb = oracle.matmul_fp32(Ab.float().numpy(), Bb.float().numpy(), trans_b=layout == "nt")
            Cb = sk.streamk_bf16(Ab.cuda(), Bb.cuda(), layout=layout, plan=pb)
            assert _rel(oracle, Cb, refb) <= 4e-3 <= TOL, (M, N, K, layout, sk.kernel_name(pb.kernel_id))
        if K % 16 == 0 and M * N * K <= 5e9:
            Ai, Bi = rng.integers(-8, 9, (M, K)).astype(np.int8), rng.integers(-8, 9, (N, K)).astype(np.int8)
            pi = sk.make_plan(M, N, K, "int8", "nt", use_tuned=False)
            kinds.add((pi.schedule, pi.streamk_tiles > 0))
            assert np.array_equal(sk.streamk_int8(_t(Ai), _t(Bi), plan=pi).cpu().numpy(), Ai.astype(np.int32) @ Bi.astype(np.int32).T), (M, N, K)
    S = sk._lib.SCHEDULES
    assert (S["dp"], False) in kinds and (S["splitk"], True) in kinds and ((S["basic"], True) in kinds or (S["sk2"], True) in kinds), kinds
    assert interleaved >= 2   # 288 tiles of 64 iterations on 256 CUs: nine offsets, 32 CTAs at each (both layouts)
    sk.workspace_status()


def test_interleaved_streamk_tile_order(sk, oracle):
    """The interleaved order of the Stream-K tiles only changes which tile of C a tile id stands for: every
    kernel family and fix-up gives the product within the usual bound on ragged shapes; with exact (integer) data the
    result equals that of the plain order bit for bit."""
    import torch
    rng = np.random.default_rng(31)
    ran = 0
    for (M, N, K, grid) in [(1100, 1400, 1024, 40), (3000, 1300, 512, 56), (640, 2000, 2048, 48)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Ai, Bi = rng.integers(-1, 2, (M, K)).astype(np.float16), rng.integers(-1, 2, (N, K)).astype(np.float16)
        ref = oracle.matmul_fp32(A, B, trans_b=True)
        dA, dB, dAi, dBi = _t(A), _t(B), _t(Ai), _t(Bi)
        for tile in (dict(bm=256, bn=256, bk=64, variant=8), dict(bm=256, bn=256, bk=64, variant=5), dict(bm=128, bn=128, bk=64, variant=5),
                     dict(bm=128, bn=256, bk=32, variant=6), dict(bm=128, bn=128, bk=64, variant=2)):
            for sch in (dict(schedule="basic", fixup="reduce"), dict(schedule="basic", fixup="atomic"),
                        dict(schedule="sk2", fixup="reduce"), dict(schedule="basic", fixup="atomic_c")):
                for raster in (1, 4):
                    cfg = dict(tile, grid=grid, raster=raster, **sch)
                    try:
                        plan = sk.make_plan(M, N, K, "float16", "nt", dict(cfg, interleave=1))
                        plain = sk.make_plan(M, N, K, "float16", "nt", cfg)
                    except sk.StreamKError:
                        continue
                    if plan.interleave <= 1:
                        continue
                    assert plan.streamk_tiles % plan.interleave == 0
                    C = sk.streamk_fp16(dA, dB, plan=plan)
                    assert _rel(oracle, C, ref) <= (1e-2 if sch["fixup"] == "atomic_c" else 1e-3) <= TOL, (M, N, K, cfg)
                    assert torch.equal(sk.streamk_fp16(dAi, dBi, plan=plan), sk.streamk_fp16(dAi, dBi, plan=plain)), (M, N, K, cfg)
                    ran += 1
    assert ran >= 40, ran
    # one-byte operands (assembly-loop and eight-wave kernels) and the small-M kernels share the tile mapping
    M, N, K = 1100, 1400, 1024
    Ai8, Bi8 = rng.integers(-8, 9, (M, K)).astype(np.int8), rng.integers(-8, 9, (N, K)).astype(np.int8)
    exact = Ai8.astype(np.int32) @ Bi8.astype(np.int32).T
    for bm, grid in ((256, 40), (128, 44)):   # 30 and 99 tiles
        plan = sk.make_plan(M, N, K, "int8", "nt", dict(bm=bm, bn=bm, grid=grid, schedule="basic", fixup="reduce", raster=4, interleave=1))
        assert plan.interleave > 1
        assert np.array_equal(sk.streamk_int8(_t(Ai8), _t(Bi8), plan=plan).cpu().numpy(), exact)
    M, N, K = 16, 2000, 4096
    A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    B = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    plan = sk.make_plan(M, N, K, "float16", "nt", dict(bm=16, bn=64, bk=256, grid=24, schedule="basic", fixup="reduce", interleave=1))
    assert plan.interleave > 1
    assert _rel(oracle, sk.streamk_fp16(_t(A), _t(B), plan=plan), oracle.matmul_fp32(A, B, trans_b=True)) <= 1e-3
    sk.workspace_status()


def test_reference_fixup_packed_atomics_into_c(sk, oracle):
    """The reference's own fix-up (streamk_fp16.py:248-255): every segment of a split tile rounds its partial to
    C's type and adds it into C with packed 16-bit atomics, no workspace, C zero-filled by the library (handed
    over full of garbage here).  Exact on integer data (every partial and every sum is an integer below 2048);
    within 1e-2 of the fp32 host product on U[-1,1) data (each of the few partials is rounded once); fp16 and
    bfloat16, NT and NN, the eight-wave 16x16x32 kernels and the assembly-loop kernel, ragged M and N (N even);
    refused for other kernels, an odd N, a bias."""
    import torch
    rng = np.random.default_rng(29)
    ran = 0
    for (M, N, K) in [(1024, 1024, 8192), (200, 136, 320), (1000, 1096, 2048), (520, 266, 448)]:
        Ai = rng.integers(-1, 2, (M, K)).astype(np.float16)
        Bi = rng.integers(-1, 2, (N, K)).astype(np.float16)
        Ai[:, 1500:] = 0
        exact = Ai.astype(np.int32) @ Bi.astype(np.int32).T
        assert np.abs(exact).max() < 2048
        Ar = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Br = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.matmul_fp32(Ar, Br, trans_b=True)
        for layout in ("nt", "nn"):
            if layout == "nn" and N % 8:
                continue
            dAi, dAr = _t(Ai), _t(Ar)
            dBi = _t(np.ascontiguousarray(Bi.T) if layout == "nn" else Bi)
            dBr = _t(np.ascontiguousarray(Br.T) if layout == "nn" else Br)
            for tile in (dict(bm=128, bn=128, bk=64, variant=5), dict(bm=256, bn=256, bk=64, variant=5), dict(bm=256, bn=256, bk=64, variant=8),
                         dict(bm=128, bn=256, bk=64, variant=5)):
                if layout == "nn" and tile["bm"] != tile["bn"]:
                    continue
                for sch in (dict(schedule="sk2"), dict(schedule="basic", grid=24), dict(schedule="splitk", split=2)):
                    try:
                        plan = sk.make_plan(M, N, K, "float16", layout, dict(tile, fixup="atomic_c", **sch))
                    except sk.StreamKError:
                        assert tile.get("variant") == 8 and K % 64 or sch["schedule"] == "splitk"
                        continue
                    assert plan.workspace_bytes == 0
                    out = torch.full((M, N), 777.0, dtype=torch.float16, device="cuda")
                    C = sk.streamk_fp16(dAi, dBi, plan=plan, layout=layout, out=out)
                    assert np.array_equal(C.cpu().numpy().astype(np.int32), exact), (M, N, K, layout, tile, sch)
                    C = sk.streamk_fp16(dAr, dBr, plan=plan, layout=layout, out=out)
                    assert _rel(oracle, C, ref) <= 4e-3 <= TOL, (M, N, K, layout, tile, sch)
                    if tile == dict(bm=256, bn=256, bk=64, variant=8) and layout == "nt":
                        pb = sk.make_plan(M, N, K, "bfloat16", layout, dict(tile, fixup="atomic_c", **sch))
                        Cb = sk.streamk_bf16(dAi.bfloat16(), dBi.bfloat16(), plan=pb, out=torch.full((M, N), -3.0, dtype=torch.bfloat16, device="cuda"))
                        # (partials and sums are rounded to bfloat16's eight bits: integers are exact only below 256)
                        assert _rel(oracle, Cb, exact.astype(np.float32)) <= 2e-2, (M, N, K, tile, sch)
                    ran += 1
    assert ran >= 40
    # not for the 32x32 accumulator kernels, the small-M kernels, an odd N or a bias
    with pytest.raises(sk.StreamKError):
        sk.make_plan(1024, 1024, 8192, "float16", "nt", dict(bm=128, bn=128, bk=64, variant=2, schedule="sk2", fixup="atomic_c"))
    with pytest.raises(sk.StreamKError):
        sk.make_plan(16, 1024, 8192, "float16", "nt", dict(schedule="sk2", fixup="atomic_c"))
    with pytest.raises(sk.StreamKError):
        sk.make_plan(1024, 1023, 8192, "float16", "nt", dict(bm=128, bn=128, bk=64, variant=5, schedule="sk2", fixup="atomic_c"))
    A, B = _t(_uniform16((512, 1024), 3)), _t(_uniform16((512, 1024), 4))
    with pytest.raises(sk.StreamKError):
        sk.streamk_fp16(A, B, bm=128, bn=128, bk=64, variant=5, schedule="sk2", fixup="atomic_c", bias=torch.zeros(512, dtype=torch.float16, device="cuda"))
    sk.workspace_status()


def test_assembly_loop_tile_kernels(sk, oracle, golden_dir):
    """The four-wave 256 x 256 x 64 kernels whose K loop is hand-scheduled assembly (accumulators in the
    accumulation registers): fp16 and bfloat16, NT and NN, ragged M and N, K any multiple of 64 (odd and even iteration
    counts, a single iteration), every schedule and both fix-ups including the halves exchange -- exact on
    integer data, bit-identical to the eight-wave 16x16x32 kernel on random data (same instruction, same order
    of the K-steps), within tolerance of the oracle; a K that is no multiple of 64 falls back to the eight-wave
    kernel; bias and activation epilogue."""
    import torch
    rng = np.random.default_rng(91)
    assert sk.kernel_name(sk.make_plan(8192, 8192, 8192, "float16", "nt", use_tuned=False).kernel_id) == "tile_f16_nt_asm_256x256x64"
    assert sk.kernel_name(sk.make_plan(2048, 2048, 2048, "bfloat16", "nt", dict(bm=256, bn=256)).kernel_id) == "tile_bf16_nt_asm_256x256x64"
    assert "asm" not in sk.kernel_name(sk.make_plan(2048, 2048, 2056, "float16", "nt", dict(bm=256, bn=256)).kernel_id)
    assert sk.kernel_name(sk.make_plan(2048, 2048, 2048, "float16", "nn", dict(bm=256, bn=256)).kernel_id) == "tile_f16_nn_asm_256x256x64"
    assert "asm" not in sk.kernel_name(sk.make_plan(2048, 2048, 2056, "float16", "nn", dict(bm=256, bn=256)).kernel_id)
    with pytest.raises(sk.StreamKError):
        sk.make_plan(2048, 2048, 2056, "float16", "nt", dict(bm=256, bn=256, variant=8))
    ran = 0
    for (M, N, K) in [(256, 256, 64), (256, 256, 192), (200, 136, 320), (1000, 1096, 4096), (520, 264, 448), (512, 1024, 2048)]:
        Ai = rng.integers(-2, 3, (M, K)).astype(np.float16)
        Bi = rng.integers(-2, 3, (N, K)).astype(np.float16)
        exact = torch.from_numpy((Ai.astype(np.int32) @ Bi.astype(np.int32).T).astype(np.float32)).cuda()
        Ar = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Br = (rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.matmul_fp32(Ar, Br, trans_b=True)
        dAi, dBi, dAr, dBr = _t(Ai), _t(Bi), _t(Ar), _t(Br)
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7), dict(schedule="basic", fixup="atomic", grid=5),
                    dict(schedule="sk2", fixup="reduce", grid=3), dict(schedule="splitk", split=2, fixup="reduce"),
                    dict(schedule="splitk", split=2, fixup="atomic"), dict(schedule="sk1", fixup="reduce", grid=2, raster=2)):
            try:
                plan = sk.make_plan(M, N, K, "float16", "nt", dict(bm=256, bn=256, bk=64, variant=8, **sch))
            except sk.StreamKError:
                assert sch["schedule"] == "splitk"      # the split does not divide this K
                continue
            assert sk.kernel_name(plan.kernel_id) == "tile_f16_nt_asm_256x256x64"
            assert torch.equal(sk.streamk_fp16(dAi, dBi, plan=plan).float(), exact), (M, N, K, sch)
            C = sk.streamk_fp16(dAr, dBr, plan=plan)
            assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, sch)
            if sch["schedule"] == "dp" or sch.get("fixup") == "reduce":
                twin = sk.streamk_fp16(dAr, dBr, **dict(sch, bm=256, bn=256, bk=64, variant=5))
                assert torch.equal(C, twin), (M, N, K, sch)
            # bfloat16 twin of the loop
            pb = sk.make_plan(M, N, K, "bfloat16", "nt", dict(bm=256, bn=256, bk=64, variant=8, **sch))
            # (the exact integer sums, rounded once to bfloat16's eight bits)
            assert torch.equal(sk.streamk_bf16(dAi.bfloat16(), dBi.bfloat16(), plan=pb), exact.bfloat16()), (M, N, K, sch)
            ran += 1
    assert ran >= 30
    # the NN form of the loop (B is [K, N]: 512-byte K-rows in LDS, transposing fragment reads): the same checks
    # against the eight-wave NN kernel; N ragged in multiples of 8
    ran = 0
    for (M, N, K) in [(256, 256, 64), (256, 256, 192), (200, 136, 320), (1000, 1096, 1024), (520, 264, 448)]:
        Ai = rng.integers(-2, 3, (M, K)).astype(np.float16)
        Bi = rng.integers(-2, 3, (K, N)).astype(np.float16)
        exact = torch.from_numpy((Ai.astype(np.int32) @ Bi.astype(np.int32)).astype(np.float32)).cuda()
        Ar = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Br = (rng.random((K, N), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.matmul_fp32(Ar, Br, trans_b=False)
        dAi, dBi, dAr, dBr = _t(Ai), _t(Bi), _t(Ar), _t(Br)
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7), dict(schedule="basic", fixup="atomic", grid=5),
                    dict(schedule="splitk", split=2, fixup="reduce"), dict(schedule="sk1", fixup="reduce", grid=2, raster=2)):
            try:
                plan = sk.make_plan(M, N, K, "float16", "nn", dict(bm=256, bn=256, bk=64, variant=8, **sch))
            except sk.StreamKError:
                assert sch["schedule"] == "splitk"
                continue
            assert sk.kernel_name(plan.kernel_id) == "tile_f16_nn_asm_256x256x64"
            assert torch.equal(sk.streamk_fp16(dAi, dBi, plan=plan, layout="nn").float(), exact), (M, N, K, sch)
            C = sk.streamk_fp16(dAr, dBr, plan=plan, layout="nn")
            assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, sch)
            if sch["schedule"] == "dp" or sch.get("fixup") == "reduce":
                twin = sk.streamk_fp16(dAr, dBr, layout="nn", **dict(sch, bm=256, bn=256, bk=64, variant=5))
                assert torch.equal(C, twin), (M, N, K, sch)
            pb = sk.make_plan(M, N, K, "bfloat16", "nn", dict(bm=256, bn=256, bk=64, variant=8, **sch))
            assert sk.kernel_name(pb.kernel_id) == "tile_bf16_nn_asm_256x256x64"
            assert torch.equal(sk.streamk_bf16(dAi.bfloat16(), dBi.bfloat16(), plan=pb, layout="nn"), exact.bfloat16()), (M, N, K, sch)
            ran += 1
    assert ran >= 20
    # epilogue: integer bias + relu exact; silu within tolerance
    M, N, K = 520, 264, 448
    Ai = rng.integers(-1, 2, (M, K)).astype(np.float16)
    Bi = rng.integers(-1, 2, (N, K)).astype(np.float16)
    bias = rng.integers(-3, 4, N).astype(np.float16)
    want = np.maximum(Ai.astype(np.int32) @ Bi.astype(np.int32).T + bias.astype(np.int32), 0)
    for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7), dict(schedule="splitk", split=1)):
        C = sk.streamk_fp16(_t(Ai), _t(Bi), bm=256, bn=256, bk=64, variant=8, bias=_t(bias), activation="relu", **sch)
        assert np.array_equal(C.cpu().numpy().astype(np.int32), want), sch
    x = Ai.astype(np.float64) @ Bi.astype(np.float64).T * 0.125 + bias.astype(np.float64)
    C = sk.streamk_fp16(_t((Ai * np.float16(0.125)).astype(np.float16)), _t(Bi), bm=256, bn=256, bk=64, variant=8, bias=_t(bias), activation="silu")
    assert oracle.max_abs_rel(C.float().cpu().numpy(), oracle.activation_ref(x, "silu")) <= 2e-3
    sk.workspace_status()


def test_fixed_split_k(sk, oracle):
    """Fixed split-K (the reference's data-parallel comparator with splitk_factor,
    thread_level_gemm_with_macro_ladder_atomic_reduce.py:129-199) on tile and small-M kernels, both
    fix-ups; with the ordered reduce it is the same partition as basic Stream-K on tiles * split CTAs,
    so the two agree bit for bit."""
    import torch
    A, B = _uniform16((1024, 8192), 0), _uniform16((1024, 8192), 1)
    ref = oracle.matmul_fp32(A, B, trans_b=True)
    dA, dB = _t(A), _t(B)
    for cfg in (dict(bm=128, bn=128, bk=64, split=4), dict(bm=128, bn=128, bk=32, variant=4, split=8),
                dict(bm=256, bn=256, bk=64, split=16), dict(bm=64, bn=64, bk=64, split=2), dict(bm=128, bn=128, bk=64)):
        for fixup in ("atomic", "reduce"):
            plan = sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="splitk", fixup=fixup, **cfg)
            assert plan.grid == plan.total_tiles * cfg.get("split", 8)
            C = sk.streamk_fp16(dA, dB, plan=plan)
            assert _rel(oracle, C, ref) <= 1e-3 <= TOL, (cfg, fixup)
        same = dict(cfg)
        same.pop("split", None)
        basic = sk.streamk_fp16(dA, dB, schedule="basic", fixup="reduce", grid=plan.grid, **same)
        assert torch.equal(C, basic), cfg
    # small-M kernels: 16 x 4096 x 11008 with 16 x 64 x 128 tiles, 86 K-iterations = 2 * 43
    A, B = _uniform16((16, 11008), 2), _uniform16((4096, 11008), 3)
    ref = oracle.matmul_fp32(A, B, trans_b=True)
    for fixup in ("atomic", "reduce"):
        plan = sk.make_plan(16, 4096, 11008, "float16", "nt", bm=16, bn=64, bk=128, schedule="splitk", split=2, fixup=fixup)
        assert plan.grid == 128 and plan.iters_per_tile == 86
        assert _rel(oracle, sk.streamk_fp16(_t(A), _t(B), plan=plan), ref) <= 1e-3
    sk.workspace_status()


def test_reduce_fixup_with_16_bit_partials(sk, oracle):
    """SK_FIXUP_REDUCE16: the halves of a split tile travel rounded to C's 16-bit type and are added in fp32 by the CTA
    that finishes them.  Tiles cut in two and in four, fp16 and bfloat16, ragged shapes: within 2e-3 (bfloat16: 8e-3)
    of the fp32 host product, the same bits on every launch, exact on small-integer data (every partial sum is
    representable in 16 bits), equal to the fp32 REDUCE wherever no partial sum needs rounding; refused for any plan
    that is not an equal split in two or four on the 256 x 256 assembly-loop kernel."""
    import torch
    g = torch.Generator(device="cpu").manual_seed(7)
    for (M, N, K, split) in [(1024, 8192, 8192, 2), (512, 8192, 8192, 4), (256, 512, 1024, 2), (200, 500, 2048, 4), (300, 1000, 512, 2)]:
        for name, dt, fn, tol in (("float16", torch.float16, sk.streamk_fp16, 2e-3), ("bfloat16", torch.bfloat16, sk.streamk_bf16, 8e-3)):
            A = (torch.rand(M, K, generator=g) * 2 - 1).to(dt)
            B = (torch.rand(N, K, generator=g) * 2 - 1).to(dt)
            Ai = torch.randint(-1, 2, (M, K), generator=g).to(dt)
            Bi = torch.randint(-1, 2, (N, K), generator=g).to(dt)
            Ai[:, 150:] = 0   # |sums| <= 150: exact in fp16 and in bfloat16's eight bits
            ref = oracle.matmul_fp32(A.float().numpy(), B.float().numpy(), trans_b=True)
            exact = (Ai.double() @ Bi.double().T).numpy()
            cfg = dict(bm=256, bn=256, bk=64, variant=8, schedule="splitk", split=split)
            p16 = sk.make_plan(M, N, K, name, "nt", dict(cfg, fixup="reduce16"))
            p32 = sk.make_plan(M, N, K, name, "nt", dict(cfg, fixup="reduce"))
            assert p16.workspace_bytes == p32.workspace_bytes and p16.grid == p32.grid
            C = fn(A.cuda(), B.cuda(), plan=p16)
            assert _rel(oracle, C, ref) <= tol <= TOL, (M, N, K, split, name)
            assert torch.equal(C, fn(A.cuda(), B.cuda(), plan=p16)), (M, N, K, split, name)
            Ci = fn(Ai.cuda(), Bi.cuda(), plan=p16)
            assert np.array_equal(Ci.double().cpu().numpy(), exact), (M, N, K, split, name)
            assert torch.equal(Ci, fn(Ai.cuda(), Bi.cuda(), plan=p32)), (M, N, K, split, name)
    # `basic` / `sk2` with two CTAs per tile are the same equal split; with bias and activation
    M, N, K = 512, 1024, 4096
    Ai = torch.randint(-1, 2, (M, K), generator=g).half()
    Bi = torch.randint(-1, 2, (N, K), generator=g).half()
    Ai[:, 150:] = 0
    bias = torch.randint(-3, 4, (N,), generator=g).half()
    want = np.maximum((Ai.double() @ Bi.double().T).numpy() + bias.double().numpy(), 0)
    for sch in (dict(schedule="basic", grid=16), dict(schedule="sk2", grid=16), dict(schedule="basic", grid=32)):
        C = sk.streamk_fp16(Ai.cuda(), Bi.cuda(), bias=bias.cuda(), activation="relu", bm=256, bn=256, bk=64, variant=8,
                            fixup="reduce16", **sch)
        assert np.array_equal(C.double().cpu().numpy(), want), sch
    for cfg in (dict(bm=128, bn=128, bk=64, schedule="splitk", split=2), dict(bm=256, bn=256, bk=64, variant=5, schedule="splitk", split=2),
                dict(bm=256, bn=256, bk=64, variant=8, schedule="dp"), dict(bm=256, bn=256, bk=64, variant=8, schedule="basic", grid=24),
                dict(bm=256, bn=256, bk=64, variant=8, schedule="splitk", split=8)):
        with pytest.raises(sk.StreamKError):
            sk.make_plan(M, N, K, "float16", "nt", dict(cfg, fixup="reduce16"))
    with pytest.raises(sk.StreamKError):
        sk.make_plan(M, N, K, "int8", "nt", dict(bm=256, bn=256, schedule="splitk", split=2, fixup="reduce16"))
    sk.workspace_status()


@pytest.mark.gpu
def test_reduce_fixup_is_bitwise_reproducible(sk):
    """The ordered reduce must give identical bits run to run (10 runs, two shapes); the schedule
    splits every tile."""
    import torch
    for (M, N, K, cfg) in [(1024, 1024, 8192, dict(bm=128, bn=128, bk=64, grid=256)),
                           (16, 4096, 11008, dict()), (300, 1000, 4096, dict(bm=64, bn=64, bk=64, grid=200))]:
        A, B = _t(_uniform16((M, K), 2)), _t(_uniform16((N, K), 3))
        first = sk.streamk_fp16(A, B, schedule="basic", fixup="reduce", **cfg).clone()
        for _ in range(9):
            again = sk.streamk_fp16(A, B, schedule="basic", fixup="reduce", **cfg)
            assert torch.equal(first, again)
    sk.workspace_status()


@pytest.mark.parametrize("NK", [(4096, 4096), (11008, 4096), (4096, 11008), (28672, 8192)],
                         ids=lambda nk: f"N{nk[0]}_K{nk[1]}")
@pytest.mark.parametrize("M", [1, 16, 64, 256])
def test_cfg3_small_m_sweep(sk, oracle, M, NK):
    """Small-M sweep, inputs normal(0, 0.02); heuristic plan (weight-streaming kernels for M <= 64,
    LDS-tiled kernel for M = 256)."""
    N, K = NK
    rng = np.random.default_rng(M * 7 + N)
    A = (rng.standard_normal((M, K), dtype=np.float32) * 0.02).astype(np.float16)
    B = (rng.standard_normal((N, K), dtype=np.float32) * 0.02).astype(np.float16)
    ref = oracle.matmul_fp32(A, B, trans_b=True)
    for fixup in ("reduce", "atomic"):
        C = sk.streamk_fp16(_t(A), _t(B), fixup=fixup)
        assert _rel(oracle, C, ref) <= 2e-3 <= TOL, fixup
    sk.workspace_status()


def test_q4_dequant_bit_exact(sk, oracle, golden_dir):
    g = np.load(os.path.join(golden_dir, "q4_16x256.npz"))
    W = sk.dequant_q4(_t(g["Wq"]), _t(g["scales"])).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), g["W"].view(np.uint16))
    # every nibble x 4096 scales spread over all of fp16 (incl. subnormal results), zero points 0/8/15
    bits = np.arange(0, 65536, 16, dtype=np.uint16)
    sc = bits.view(np.float16)
    sc = sc[np.isfinite(sc.astype(np.float32))].reshape(-1, 1)
    nib = (np.arange(128) % 16).astype(np.uint8)
    Wq = np.broadcast_to((nib[0::2] | (nib[1::2] << 4)).astype(np.uint8), (sc.shape[0], 64)).copy()
    for zero in (8, 0, 15):
        got = sk.dequant_q4(_t(Wq), _t(sc), zero=zero).cpu().numpy().view(np.uint16)
        assert np.array_equal(got, oracle.dequant_q4(Wq, sc, 128, zero).view(np.uint16)), zero


def test_q4_gemm_fixture(sk, oracle, golden_dir):
    g = np.load(os.path.join(golden_dir, "q4_16x256.npz"))
    for cfg in (dict(), dict(schedule="basic", grid=2), dict(schedule="basic", grid=2, fixup="atomic")):
        C = sk.streamk_q4(_t(g["A"]), _t(g["Wq"]), _t(g["scales"]), **cfg)
        assert _rel(oracle, C, g["C"]) <= 2e-3 <= TOL


@pytest.mark.parametrize("M", [1, 16])
def test_cfg4_q4_gemm(sk, oracle, M):
    """Q4 weight-only GEMM at N = K = 8192: A normal(0,1), nibbles uniform 0..15, zero-point 8,
    scales U[0.005, 0.02] per (row, 128-wide group); Stream-K with the ordered reduce (and atomic),
    every kernel variant."""
    N = K = 8192
    rng = np.random.default_rng(40 + M)
    A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    ref = oracle.q4_gemm_ref(A, Wq, sc, 128, 8)
    dA, dW, dS = _t(A), _t(Wq), _t(sc)
    # the GEMM consumes exactly the weights the standalone dequant produces: check those first
    W = sk.dequant_q4(dW, dS).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), oracle.dequant_q4(Wq, sc, 128, 8).view(np.uint16))
    for cfg in (dict(fixup="reduce"), dict(fixup="atomic"), dict(schedule="dp"),
                dict(bm=16, bn=16, bk=1024), dict(bm=16, bn=32, bk=512), dict(schedule="basic", grid=256)):
        C = sk.streamk_q4(dA, dW, dS, **cfg)
        assert _rel(oracle, C, ref) <= 2e-3 <= TOL, cfg
    sk.workspace_status()


Q4_TILES = [(16, 64, 256), (16, 32, 512), (16, 16, 1024), (16, 128, 256), (16, 64, 512), (16, 32, 256),
            (16, 16, 512), (16, 16, 256), (32, 64, 256), (64, 64, 256), (16, 32, 1024)]


@pytest.mark.parametrize("variant", [1, 2, 3], ids=["general", "row1", "gemv"])
def test_q4_ragged_shapes_every_kernel(sk, oracle, variant):
    """Every Q4 kernel instance (general small-M, single-row, matrix-vector) on ragged shapes: N not
    a multiple of the tile, K a multiple of 128 only (a scale row shorter than one 16-byte piece, a
    last iteration hanging over K), zero points 0 / 5 / 8 / 15, all three schedules.  The
    matrix-vector kernels accumulate unrounded (q - zero) * scale products in fp32, the others
    multiply fp16-rounded weights; both stay within 2e-3 of the fp32 host product of the
    dequantised weights."""
    rng = np.random.default_rng(50 + variant)
    shapes = [(1, 1000, 1152, 8), (1, 520, 384, 15), (1, 72, 4096, 0), (1, 2048, 16384, 5), (1, 264, 28672, 8)]
    if variant == 1:
        shapes += [(5, 1000, 1152, 8), (16, 520, 384, 15), (33, 200, 640, 8), (64, 136, 2048, 3)]
    ran = 0
    for (M, N, K, zero) in shapes:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        ref = oracle.q4_gemm_ref(A, Wq, sc, 128, zero)
        dA, dW, dS = _t(A), _t(Wq), _t(sc)
        for (bm, bn, bk) in Q4_TILES:
            # (data-parallel on five CTAs: every CTA takes several tiles one after the other, and the matrix-vector
            # kernels keep the row of A in LDS from the first one on)
            for sch in (dict(schedule="dp"), dict(schedule="dp", grid=5), dict(schedule="sk2", fixup="reduce", grid=48),
                        dict(schedule="sk2", fixup="atomic", grid=40)):
                try:
                    plan = sk.make_plan(M, N, K, "q4", "nt", dict(bm=bm, bn=bn, bk=bk, variant=variant, **sch))
                except sk.StreamKError:
                    continue  # no such instance of this variant, or it does not take this M / K
                C = sk.streamk_q4(dA, dW, dS, zero=zero, plan=plan)
                assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, zero, bm, bn, bk, sch, plan.kernel_id)
                ran += 1
    assert ran >= 50
    sk.workspace_status()


def test_q4_weights_streamed_through_lds(sk, oracle):
    """Up to 16 rows of A on the kernels that stream row-major Q4 weights through LDS in contiguous loads (64 and 32
    weight rows per tile): ragged M and N, K a multiple of 256 only (a last iteration hanging over K), zero points
    0 / 5 / 8 / 15, all schedules and both fix-ups.  Exact on integer data with power-of-two scales (any wrong nibble,
    K order, scale row or rotation shows), within 2e-3 of the oracle on random data (these kernels multiply the
    unrounded (q - zero) * scale, the oracle the fp16-rounded weights); K that is not a multiple of 256 is refused."""
    import torch
    rng = np.random.default_rng(58)
    ran = 0
    for (M, N, K, zero) in [(16, 1000, 2304, 8), (9, 520, 256, 15), (1, 72, 4096, 0), (13, 2048, 16384, 5), (5, 264, 28672, 8),
                            (16, 8192, 8192, 8), (2, 4099, 11008, 3)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        Ai = rng.integers(-2, 3, (M, K)).astype(np.float16)
        sci = (2.0 ** rng.integers(-3, 1, (N, K // 128))).astype(np.float16)
        full = N * K <= 1 << 24   # (the host product of the large cases is taken on a slice of the weight rows)
        rows = slice(None) if full else slice(N - 520, N)
        ref = oracle.q4_gemm_ref(A, Wq[rows], sc[rows], 128, zero)
        exact = oracle.q4_gemm_ref(Ai, Wq[rows], sci[rows], 128, zero)
        assert np.abs(exact).max() < 2 ** 20 and np.array_equal(exact, np.rint(exact * 8) / 8)   # (exact in fp32)
        dA, dAi, dW, dS, dSi = _t(A), _t(Ai), _t(Wq), _t(sc), _t(sci)
        for (bn, bk) in ((64, 512), (32, 1024)):
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48),
                        dict(schedule="sk2", fixup="atomic", grid=40), dict(schedule="basic", fixup="reduce", grid=56)):
                plan = sk.make_plan(M, N, K, "q4", "nt", dict(bm=16, bn=bn, bk=bk, variant=5, **sch))
                assert sk.kernel_name(plan.kernel_id).startswith("stream_q4_")
                C = sk.streamk_q4(dA, dW, dS, zero=zero, plan=plan)
                assert _rel(oracle, C[:, rows], ref) <= 2e-3 <= TOL, (M, N, K, zero, bn, bk, sch)
                C = sk.streamk_q4(dAi, dW, dSi, zero=zero, plan=plan)
                assert np.array_equal(C[:, rows].float().cpu().numpy(), exact.astype(np.float16).astype(np.float32)), (M, N, K, zero, bn, bk, sch)
                ran += 1
    assert ran >= 56
    with pytest.raises(sk.StreamKError):
        sk.make_plan(16, 1000, 1152, "q4", "nt", dict(bm=16, bn=64, bk=512, variant=5))
    with pytest.raises(sk.StreamKError):
        sk.make_plan(17, 1000, 1024, "q4", "nt", dict(bm=16, bn=64, bk=512, variant=5))
    # what the library picks by itself for 2..16 rows and 16 MB of weights or more
    assert sk.kernel_name(sk.make_plan(16, 8192, 8192, "q4", "nt", use_tuned=False).kernel_id).startswith("stream_q4_")
    assert sk.kernel_name(sk.make_plan(16, 4096, 4096, "q4", "nt", use_tuned=False).kernel_id).startswith("stream_q4_")
    assert not sk.kernel_name(sk.make_plan(16, 2048, 4096, "q4", "nt", use_tuned=False).kernel_id).startswith("stream_q4_")
    sk.workspace_status()


@pytest.mark.gpu
def test_q4_tile_kernels_more_than_64_rows(sk, oracle):
    """Q4 weights with more rows of A than the weight-streaming kernels take: the tile kernels that dequantise B
    in registers on its way into the LDS stage (the reference dequantises right before the MMA,
    streamk_fp16_ladder_block_reduce_q4.py:283-294).  Every tile shape, schedule and fix-up on ragged shapes and
    zero points 0 / 5 / 8 / 15: exact on integer data with unit scales (any wrong nibble, K order or scale row
    shows), within 2e-3 of the oracle on random data; the weights the kernel multiplies are the bit-exact ones
    (it must equal the fp16 kernel of the same tile on sk_dequant_q4's output bit for bit)."""
    import torch
    rng = np.random.default_rng(53)
    ran = 0
    for (M, N, K, zero) in [(128, 128, 128, 8), (200, 136, 384, 5), (300, 520, 1152, 0), (1000, 1096, 4096, 8), (65, 72, 128, 15)]:
        Ai = rng.integers(-1, 2, (M, K)).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        exact = Ai.astype(np.int64) @ (oracle.unpack_q4_np(Wq).astype(np.int64) - zero).T
        ones = torch.ones(N, K // 128, dtype=torch.float16, device="cuda")
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        Ar = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.q4_gemm_ref(Ar, Wq, sc, 128, zero)
        dAi, dAr, dW, dS = _t(Ai), _t(Ar), _t(Wq), _t(sc)
        W16 = sk.dequant_q4(dW, dS, zero=zero)
        for (bm, bn) in ((128, 128), (256, 128)):
            for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7),
                        dict(schedule="basic", fixup="atomic", grid=5), dict(schedule="sk2", fixup="reduce", grid=3)):
                plan = sk.make_plan(M, N, K, "q4", "nt", dict(bm=bm, bn=bn, **sch))
                assert sk.kernel_name(plan.kernel_id) == f"tile_q4_nt_dma16_{bm}x{bn}x64"
                C = sk.streamk_q4(dAi, dW, ones, zero=zero, plan=plan)
                assert np.array_equal(C.cpu().numpy().astype(np.int64), exact), (M, N, K, zero, bm, bn, sch)
                C = sk.streamk_q4(dAr, dW, dS, zero=zero, plan=plan)
                assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, zero, bm, bn, sch)
                if sch.get("fixup") != "atomic":
                    twin = sk.streamk_fp16(dAr, W16, **dict(sch, bm=bm, bn=bn, bk=64, variant=5))
                    assert torch.equal(C, twin), (M, N, K, zero, bm, bn, sch)
                ran += 1
    assert ran == 40
    # the planner's own choice, bias and activation in the epilogue
    M, N, K = 300, 520, 1152
    A = rng.integers(-1, 2, (M, K)).astype(np.float16)
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    bias = rng.integers(-3, 4, N).astype(np.float16)
    want = np.maximum(A.astype(np.int64) @ (oracle.unpack_q4_np(Wq).astype(np.int64) - 8).T + bias.astype(np.int64), 0)
    C = sk.streamk_q4(_t(A), _t(Wq), torch.ones(N, K // 128, dtype=torch.float16, device="cuda"), bias=_t(bias), activation="relu")
    assert np.array_equal(C.cpu().numpy().astype(np.int64), want)
    sk.workspace_status()


def test_q4_prefill_sizes_at_full_width(sk, oracle):
    """N = K = 8192, M = 128 / 512 / 4096 (the fused tile kernels up to 1024 rows, beyond that one dequantisation
    pass into a per-stream staging buffer and the fp16 tile kernels): a sample of rows within 2e-3 of the oracle,
    exact integer checksums, and no allocation once the first call of a size has run."""
    import torch
    N = K = 8192
    rng = np.random.default_rng(54)
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    W = oracle.dequant_q4(Wq, sc, 128, 8).astype(np.float32)
    q8 = oracle.unpack_q4_np(Wq).astype(np.int64) - 8
    dW, dS = _t(Wq), _t(sc)
    ones = torch.ones(N, K // 128, dtype=torch.float16, device="cuda")
    for M in (128, 512, 4096):
        A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
        dA = _t(A)
        C = sk.streamk_q4(dA, dW, dS)
        rows = np.sort(rng.choice(M, 48, replace=False))
        ref = A[rows].astype(np.float32) @ W.T
        assert oracle.max_abs_rel(C[torch.from_numpy(rows).cuda()].float().cpu().numpy(), ref) <= 2e-3 <= TOL, M
        torch.cuda.synchronize()
        before = torch.cuda.memory_allocated()
        out = torch.empty_like(C)
        after_out = torch.cuda.memory_allocated()
        sk.streamk_q4(dA, dW, dS, out=out)
        torch.cuda.synchronize()
        assert torch.cuda.memory_allocated() == after_out and torch.equal(out, C), M   # nothing allocated inside the call
        del out
        Ai = rng.integers(-1, 2, (M, K)).astype(np.int8)
        Ci = sk.streamk_q4(_t(Ai.astype(np.float16)), dW, ones).double()
        assert np.array_equal(Ci.sum(dim=1).cpu().numpy().astype(np.int64), Ai.astype(np.int64) @ q8.sum(axis=0)), M
        assert np.array_equal(Ci.sum(dim=0).cpu().numpy().astype(np.int64), Ai.astype(np.int64).sum(axis=0) @ q8.T), M
    sk.workspace_status()


def test_q4_per_group_zero_points(sk, oracle):
    """Q4 with one zero point per scale group and row: device dequantisation bit for bit against the
    oracle; the GEMM on every kernel instance, ragged shapes, all schedules, within 2e-3 of the fp32 host
    product of the dequantised weights; with a constant zero point the result equals the scalar-zero
    kernel's bit for bit; more than 64 rows through the split / dequantise paths; device quantiser equal to
    the host one."""
    import torch
    rng = np.random.default_rng(77)
    tiles = [(16, 64, 256), (32, 64, 256), (64, 64, 256), (16, 32, 1024), (16, 64, 512), (16, 16, 1024), (16, 32, 512)]
    ran = 0
    for (M, N, K) in [(1, 1000, 1152), (5, 520, 384), (16, 264, 4096), (33, 200, 640), (64, 136, 2048), (1, 72, 16384)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        zp = rng.integers(0, 16, (N, K // 128)).astype(np.float16)
        dA, dW, dS, dZ = _t(A), _t(Wq), _t(sc), _t(zp)
        W = sk.dequant_q4(dW, dS, zeros=dZ)
        assert np.array_equal(W.cpu().numpy().view(np.uint16), oracle.dequant_q4_zp_np(Wq, sc, zp).view(np.uint16))
        ref = oracle.q4_zp_gemm_ref(A, Wq, sc, zp)
        z7 = torch.full_like(dZ, 7.0)
        for (bm, bn, bk) in tiles:
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48),
                        dict(schedule="sk2", fixup="atomic", grid=40)):
                try:
                    plan = sk.make_plan(M, N, K, "q4_zp", "nt", dict(bm=bm, bn=bn, bk=bk, **sch))
                except sk.StreamKError:
                    continue  # the instance does not take this M / K
                C = sk.streamk_q4(dA, dW, dS, zeros=dZ, plan=plan)
                assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, bm, bn, bk, sch, plan.kernel_id)
                gemv = sk.kernel_name(plan.kernel_id).startswith("gemv_q4zp")
                assert gemv == (M == 1 and (bm, bn, bk) in ((16, 32, 512), (16, 64, 256), (16, 16, 1024))), (M, bm, bn, bk)
                if sch.get("fixup") != "atomic" and not gemv:
                    same = sk.make_plan(M, N, K, "q4", "nt", dict(bm=bm, bn=bn, bk=bk, variant=1, **sch))
                    Cz, Cs = sk.streamk_q4(dA, dW, dS, zeros=z7, plan=plan), sk.streamk_q4(dA, dW, dS, zero=7, plan=same)
                    if bm > 16:
                        assert torch.equal(Cz, Cs)
                    else:  # up to 16 rows the scalar-zero kernels multiply the nibbles undecoded and scale fp32 group sums
                        assert _rel(oracle, Cz, Cs.double().cpu().numpy()) <= 1e-3
                if gemv and (bm, bn, bk) != (16, 32, 512):   # the general kernel of the tile (bit-exact rounded weights) stays selectable
                    general = sk.make_plan(M, N, K, "q4_zp", "nt", dict(bm=bm, bn=bn, bk=bk, variant=1, **sch))
                    assert sk.kernel_name(general.kernel_id).startswith("skinny_q4zp")
                    assert _rel(oracle, sk.streamk_q4(dA, dW, dS, zeros=dZ, plan=general), ref) <= 2e-3
                ran += 1
        C = sk.streamk_q4(dA, dW, dS, zeros=_t(zp.astype(np.uint8)))      # heuristic plan; integer zero points are converted
        assert _rel(oracle, C, ref) <= 2e-3
    assert ran >= 60
    # more rows than one launch takes: blocks of 64 rows, then dequantise + fp16 GEMM
    N, K = 520, 1024
    Wf = torch.randn(N, K, device="cuda").half() * 0.05 + 0.02
    Wq, sc, zp = sk.quantize_q4(Wf, asymmetric=True)
    hq, hs, hz = sk.quantize_q4(Wf.cpu(), asymmetric=True)
    assert torch.equal(Wq.cpu(), hq) and torch.equal(sc.cpu(), hs) and torch.equal(zp.cpu(), hz)
    for M in (150, 300):
        A = torch.randn(M, K, device="cuda").half()
        ref = oracle.q4_zp_gemm_ref(A.cpu().numpy(), hq.numpy(), hs.numpy(), hz.numpy())
        assert _rel(oracle, sk.streamk_q4(A, Wq, sc, zeros=zp), ref) <= 2e-3
    # quantisation error of the asymmetric rule on shifted weights is below the symmetric rule's
    back_a = sk.dequant_q4(Wq, sc, zeros=zp).float()
    sq, ss = sk.quantize_q4(Wf)
    back_s = sk.dequant_q4(sq, ss).float()
    assert (back_a - Wf.float()).abs().mean() < (back_s - Wf.float()).abs().mean()
    with pytest.raises(ValueError):
        sk.streamk_q4(A, Wq, sc, zeros=zp[:, :4])
    # as a layer: asymmetric weights, plans per M, state round trip
    lin = torch.nn.Linear(K, N, bias=True).cuda().half()
    with torch.no_grad():
        lin.weight.add_(0.03)
    layer = sk.StreamKLinear.from_linear(lin, weight_format="q4_zp")
    assert set(layer.state_dict()) == {"qweight", "scales", "zeros", "bias"}
    for shape in ((1, K), (2, 8, K), (150, K)):
        x = torch.randn(*shape, device="cuda").half()
        W = oracle.dequant_q4_zp_np(layer.qweight.cpu().numpy(), layer.scales.cpu().numpy(), layer.zeros.cpu().numpy())
        ref = x.float().cpu().numpy().reshape(-1, K) @ W.astype(np.float32).T + lin.bias.detach().float().cpu().numpy()
        assert oracle.max_abs_rel(layer(x).float().cpu().numpy().reshape(-1, N), ref) <= 2e-3
    sk.workspace_status()


def test_q4_tiled_weights_give_identical_results(sk, oracle):
    """The tiled weight layout (16-row x 64-byte tiles) hands every lane the bytes it gets from the
    row-major array, so each tiled kernel must reproduce its row-major twin bit for bit (ordered
    reduce and data-parallel schedules); the device tiler must write what the host one writes."""
    import torch
    rng = np.random.default_rng(91)
    ran = 0
    for (M, N, K, zero) in [(1, 1000, 1152, 8), (1, 264, 28672, 8), (1, 2048, 4096, 5), (5, 1000, 1152, 8),
                            (16, 520, 384, 15), (33, 200, 640, 8), (64, 136, 2048, 3), (16, 4096, 4096, 8)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        dA, dW, dS = _t(A), _t(Wq), _t(sc)
        dT = sk.tile_q4(dW)
        assert torch.equal(dT.cpu(), sk.tile_q4(torch.from_numpy(Wq)))
        ref = oracle.q4_gemm_ref(A, Wq, sc, 128, zero)
        C = sk.streamk_q4(dA, dT, dS, zero=zero, tiled=True)           # heuristic plan
        assert _rel(oracle, C, ref) <= 2e-3 <= TOL
        for (bm, bn, bk) in Q4_TILES:
            for variant in (1, 3):
                for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48)):
                    cfg = dict(bm=bm, bn=bn, bk=bk, variant=variant, **sch)
                    try:
                        pt = sk.make_plan(M, N, K, "q4_tiled", "nt", cfg)
                        pr = sk.make_plan(M, N, K, "q4", "nt", cfg)
                    except sk.StreamKError:
                        continue
                    Ct = sk.streamk_q4(dA, dT, dS, zero=zero, plan=pt, tiled=True)
                    Cr = sk.streamk_q4(dA, dW, dS, zero=zero, plan=pr)
                    assert torch.equal(Ct, Cr), (M, N, K, cfg)
                    ran += 1
    assert ran >= 40
    with pytest.raises(ValueError):
        sk.streamk_q4(dA, dW, dS, plan=pt)  # a tiled plan with row-major weights
    sk.workspace_status()


def test_q4_tiled_weights_with_per_group_zero_points(sk, oracle):
    """Per-group zero points with the weights in the tiled layout (scales and zero points stay row-major): every
    kernel instance reproduces its row-major twin bit for bit (data-parallel and ordered-reduce schedules) and
    stays within 2e-3 of the fp32 host product of the dequantised weights; ragged N, M from 1 to 64, more than 64
    rows through the blocks of 64."""
    import torch
    rng = np.random.default_rng(93)
    tiles = [(16, 64, 256), (32, 64, 256), (64, 64, 256), (16, 32, 1024), (16, 64, 512), (16, 16, 1024), (16, 32, 512)]
    ran, gemv_ran = 0, 0
    for (M, N, K) in [(1, 1000, 1152), (1, 2048, 4096), (1, 72, 28672), (5, 520, 384), (16, 264, 4096), (33, 200, 640),
                      (64, 136, 2048)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        zp = rng.integers(0, 16, (N, K // 128)).astype(np.float16)
        dA, dW, dS, dZ = _t(A), _t(Wq), _t(sc), _t(zp)
        dT = sk.tile_q4(dW)
        ref = oracle.q4_zp_gemm_ref(A, Wq, sc, zp)
        C = sk.streamk_q4(dA, dT, dS, zeros=dZ, tiled=True)            # heuristic plan
        assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K)
        assert torch.equal(C, sk.streamk_q4(dA, dW, dS, zeros=dZ)), (M, N, K)
        for (bm, bn, bk) in tiles:
            for variant in (0, 1):
                for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48)):
                    cfg = dict(bm=bm, bn=bn, bk=bk, **sch)
                    if variant:
                        cfg["variant"] = variant
                    try:
                        pt = sk.make_plan(M, N, K, "q4_zp_tiled", "nt", cfg)
                        pr = sk.make_plan(M, N, K, "q4_zp", "nt", cfg)
                    except sk.StreamKError:
                        continue
                    name_t, name_r = sk.kernel_name(pt.kernel_id), sk.kernel_name(pr.kernel_id)
                    assert name_t.replace("q4zpt", "q4zp") == name_r, (name_t, name_r)
                    Ct = sk.streamk_q4(dA, dT, dS, zeros=dZ, plan=pt, tiled=True)
                    assert torch.equal(Ct, sk.streamk_q4(dA, dW, dS, zeros=dZ, plan=pr)), (M, N, K, cfg, name_t)
                    assert _rel(oracle, Ct, ref) <= 2e-3, (M, N, K, cfg, name_t)
                    ran += 1
                    gemv_ran += name_t.startswith("gemv_q4zpt")
    assert ran >= 60 and gemv_ran >= 8, (ran, gemv_ran)
    with pytest.raises(ValueError):
        sk.streamk_q4(dA, dW, dS, zeros=dZ, plan=pt)   # a tiled plan with row-major weights
    with pytest.raises(ValueError):
        sk.streamk_q4(dA, dT, dS, plan=pt, tiled=True)  # a zero-point plan without zero points
    # more rows than one launch takes: blocks of 64 rows
    A = (rng.random((150, K), dtype=np.float32) * 2 - 1).astype(np.float16)
    C = sk.streamk_q4(_t(A), dT, dS, zeros=dZ, tiled=True)
    assert _rel(oracle, C, oracle.q4_zp_gemm_ref(A, Wq, sc, zp)) <= 2e-3
    sk.workspace_status()


def test_q4_matrix_vector_exact_on_integer_data(sk):
    """M = 1, N = K = 8192, A in {-1, 0, 1}, scales 1 (and 0.5): every group sum is an integer
    below 2^24, so the fp32 arithmetic of the matrix-vector kernels is exact and C must equal the
    integer product bit for bit, for every kernel instance, schedule and fix-up."""
    import torch
    N = K = 8192
    rng = np.random.default_rng(61)
    A = rng.integers(-1, 2, (1, K)).astype(np.int64)
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    q = np.empty((N, K), dtype=np.int64)
    q[:, 0::2], q[:, 1::2] = Wq & 15, Wq >> 4
    exact = (q - 8) @ A[0]
    assert np.abs(exact).max() < 2048
    dA, dW = _t(A.astype(np.float16)), _t(Wq)
    ones = torch.ones(N, K // 128, dtype=torch.float16, device="cuda")
    for (bm, bn, bk) in Q4_TILES[:8]:
        for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce"), dict(schedule="sk2", fixup="atomic"),
                    dict(schedule="basic", fixup="reduce", grid=1000)):
            try:
                plan = sk.make_plan(1, N, K, "q4", "nt", dict(bm=bm, bn=bn, bk=bk, variant=3, **sch))
            except sk.StreamKError:
                assert "grid" in sch  # more CTAs than this instance keeps resident
                continue
            C = sk.streamk_q4(dA, dW, ones, zero=8, plan=plan)
            assert np.array_equal(C.cpu().numpy()[0].astype(np.int64), exact), (bm, bn, bk, sch)
            C = sk.streamk_q4(dA, dW, ones * 0.5, zero=8, plan=plan)
            assert np.array_equal((C.double() * 2).cpu().numpy()[0].astype(np.int64), exact), (bm, bn, bk, sch)
    sk.workspace_status()


def test_q4_matrix_vector_tiles_chained_in_one_cta(sk, oracle):
    """Data-parallel launches of the Q4 matrix-vector kernels with fewer CTAs than tiles: a CTA requests the first
    loads and scales of its next tile during the last round of the tile before.  Whatever the grid, every element
    of C must equal, bit for bit, what the launch with one tile per CTA gives -- on a ragged N (last tile partial),
    K with a tail iteration, K shorter than the prefetch depth, with a bias, with per-group zero points and with
    tiled weights -- and the oracle's product."""
    import torch
    rng = np.random.default_rng(73)
    ran = 0
    for (N, K) in [(1000, 1152), (264, 28672), (2056, 4096), (520, 384), (4096, 8192)]:
        A = (rng.random((1, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        zp = rng.integers(0, 16, (N, K // 128)).astype(np.float16)
        bias = (rng.random(N, dtype=np.float32) * 2 - 1).astype(np.float16)
        dA, dW, dS, dZ, dB = _t(A), _t(Wq), _t(sc), _t(zp), _t(bias)
        dT = sk.tile_q4(dW)
        ref = oracle.q4_gemm_ref(A, Wq, sc, 128, 8)
        refz = oracle.q4_zp_gemm_ref(A, Wq, sc, zp)
        for (bm, bn, bk) in Q4_TILES + [(16, 16, 2048)]:
            for name, kw in (("q4", dict()), ("q4_zp", dict(zeros=dZ)), ("q4_tiled", dict(tiled=True)),
                             ("q4_zp_tiled", dict(zeros=dZ, tiled=True))):
                cfg = dict(bm=bm, bn=bn, bk=bk, variant=3, schedule="dp")
                try:
                    one = sk.make_plan(1, N, K, name, "nt", cfg)
                except sk.StreamKError:
                    continue  # no such instance for this format, or K beyond what it stages
                if not sk.kernel_name(one.kernel_id).startswith("gemv_q4"):
                    continue
                w = dT if "tiled" in name else dW
                want = sk.streamk_q4(dA, w, dS, plan=one, **kw)
                assert _rel(oracle, want, refz if "zp" in name else ref) <= 2e-3, (N, K, name, cfg)
                want_b = sk.streamk_q4(dA, w, dS, plan=one, bias=dB, **kw)
                for grid in (1, 3, 7, 64):
                    if grid >= one.grid:
                        continue
                    plan = sk.make_plan(1, N, K, name, "nt", dict(cfg, grid=grid))
                    assert plan.grid == grid and plan.kernel_id == one.kernel_id
                    C = torch.full_like(want, float("nan"))
                    sk.streamk_q4(dA, w, dS, out=C, plan=plan, **kw)
                    assert torch.equal(C, want), (N, K, name, cfg, grid)
                    assert torch.equal(sk.streamk_q4(dA, w, dS, plan=plan, bias=dB, **kw), want_b), (N, K, name, cfg, grid, "bias")
                    ran += 1
    assert ran >= 150, ran
    # the planner's own choice for more 16-row tiles than CTAs stay resident: every CTA walks the same number of tiles
    plan = sk.make_plan(1, 28672, 8192, "q4", "nt", use_tuned=False)
    assert sk.kernel_name(plan.kernel_id) == "gemv_q4_nb1_wn1_rk8_k16384" and plan.grid == 256
    plan = sk.make_plan(1, 32000, 4096, "q4", "nt", use_tuned=False)
    assert sk.kernel_name(plan.kernel_id) == "gemv_q4_nb1_wn1_rk2_k16384" and plan.grid == 1000
    # such plans against the oracle, N ragged (the host product is taken on the first and the last rows of the weights)
    for (N, K) in [(20010, 4096), (28672 + 8, 8192), (16400, 1536)]:
        A = (rng.random((1, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
        plan = sk.make_plan(1, N, K, "q4", "nt", use_tuned=False)
        assert plan.grid < plan.total_tiles and sk.kernel_name(plan.kernel_id).startswith("gemv_q4"), (N, K, plan.grid)
        C = torch.full((1, N), float("nan"), dtype=torch.float16, device="cuda")
        sk.streamk_q4(_t(A), _t(Wq), _t(sc), out=C, plan=plan)
        assert not bool(torch.isnan(C).any())
        for rows in (slice(0, 600), slice(N // 2 - 300, N // 2 + 300), slice(N - 600, N)):
            assert _rel(oracle, C[:, rows], oracle.q4_gemm_ref(A, Wq[rows], sc[rows], 128, 8)) <= 2e-3, (N, K, rows)
    sk.workspace_status()


def test_q4_matrix_vector_deviation_from_rounded_weights_is_bounded(sk, oracle):
    """The M = 1 matrix-vector kernels and the 16-row kernels with a scalar zero point multiply the unrounded
    (q - zero) * scale instead of the fp16-rounded weights the other kernels (and sk_dequant_q4) form.  Per output that moves the result by at most
    sum_k |a_k| |w_exact - w_rounded| <= 2^-11 sum_k |a_k w_k|, plus the rounding of C to fp16 (2^-11 |c|) and fp32
    accumulation noise; and the result is the fp16 rounding of the exact (unrounded-weight) product up to that
    noise.  Checked at N = K = 8192 on the benchmark's data for every matrix-vector instance, beside the
    instances that form the rounded weights bit for bit (which meet the rounded-weight product itself)."""
    N = K = 8192
    rng = np.random.default_rng(41)
    A = rng.standard_normal((1, K), dtype=np.float32).astype(np.float16)
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    a64 = A[0].astype(np.float64)
    w_rounded = oracle.dequant_q4(Wq, sc, 128, 8).astype(np.float64)
    w_exact = (oracle.unpack_q4_np(Wq).astype(np.float64) - 8.0) * np.repeat(sc.astype(np.float64), 128, axis=1)
    assert np.abs(w_exact - w_rounded).max() <= 2.0 ** -11 * np.abs(w_exact).max()   # per-weight premise
    y_rounded, y_exact = w_rounded @ a64, w_exact @ a64
    mass = np.abs(w_exact) @ np.abs(a64)          # sum_k |a_k w_k| per output
    noise = 2e-5 * mass                           # fp32 accumulation over 8192 terms (25 times below the 2^-11 term)
    dA, dW, dS = _t(A), _t(Wq), _t(sc)
    ran = 0
    for (bm, bn, bk) in Q4_TILES[:8]:
        # (the single-row instances form the rounded weights; the 16-row instances multiply the nibbles undecoded
        # like the matrix-vector kernels)
        for variant, rounded in ((3, False), (2, True), (1, (bm, bn, bk) == (16, 64, 256))):  # (that one instance decodes)
            try:
                plan = sk.make_plan(1, N, K, "q4", "nt", dict(bm=bm, bn=bn, bk=bk, variant=variant, schedule="dp"))
            except sk.StreamKError:
                continue
            y = sk.streamk_q4(dA, dW, dS, plan=plan).double().cpu().numpy()[0]
            assert np.all(np.abs(y - y_rounded) <= 2.0 ** -11 * mass + 2.0 ** -11 * np.abs(y_rounded) + noise), (bm, bn, bk, variant)
            target = y_rounded if rounded else y_exact
            assert np.all(np.abs(y - target) <= 2.0 ** -11 * np.abs(target) + 2.0 ** -24 + noise), (bm, bn, bk, variant)
            ran += 1
    assert ran >= 12
    # sixteen rows of A on the 16-row kernels (general and streamed through LDS): every row meets the same bounds
    A16 = rng.standard_normal((16, K), dtype=np.float32).astype(np.float16)
    a16 = A16.astype(np.float64)
    y_rounded16, y_exact16 = a16 @ w_rounded.T, a16 @ w_exact.T
    mass16 = np.abs(a16) @ np.abs(w_exact).T
    for cfg in (dict(bm=16, bn=64, bk=512, variant=1), dict(bm=16, bn=32, bk=1024, variant=1), dict(bm=16, bn=16, bk=1024, variant=1),
                dict(bm=16, bn=64, bk=512, variant=5), dict(bm=16, bn=32, bk=1024, variant=5)):
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=200)):
            plan = sk.make_plan(16, N, K, "q4", "nt", dict(cfg, **sch))
            y = sk.streamk_q4(_t(A16), dW, dS, plan=plan).double().cpu().numpy()
            assert np.all(np.abs(y - y_rounded16) <= 2.0 ** -11 * mass16 + 2.0 ** -11 * np.abs(y_rounded16) + 2e-5 * mass16), (cfg, sch)
            assert np.all(np.abs(y - y_exact16) <= 2.0 ** -11 * np.abs(y_exact16) + 2.0 ** -24 + 2e-5 * mass16), (cfg, sch)
    # the same bound for the matrix-vector kernels with one zero point per group and row
    zp = rng.integers(0, 16, (N, K // 128)).astype(np.float16)
    w_rounded = oracle.dequant_q4_zp_np(Wq, sc, zp).astype(np.float64)
    w_exact = (oracle.unpack_q4_np(Wq).astype(np.float64) - np.repeat(zp.astype(np.float64), 128, axis=1)) * \
        np.repeat(sc.astype(np.float64), 128, axis=1)
    assert np.abs(w_exact - w_rounded).max() <= 2.0 ** -11 * np.abs(w_exact).max()
    y_rounded, y_exact = w_rounded @ a64, w_exact @ a64
    mass = np.abs(w_exact) @ np.abs(a64)
    noise = 2e-5 * mass
    dZ = _t(zp)
    ran = 0
    for (bm, bn, bk) in ((16, 16, 1024), (16, 32, 512), (16, 64, 256)):
        for variant, rounded in ((3, False), (1, True)):
            if rounded and (bm, bn, bk) == (16, 32, 512):
                continue   # this tile exists as a matrix-vector kernel only
            plan = sk.make_plan(1, N, K, "q4_zp", "nt", dict(bm=bm, bn=bn, bk=bk, variant=variant, schedule="dp"))
            assert sk.kernel_name(plan.kernel_id).startswith("skinny_q4zp" if rounded else "gemv_q4zp")
            y = sk.streamk_q4(dA, dW, dS, zeros=dZ, plan=plan).double().cpu().numpy()[0]
            assert np.all(np.abs(y - y_rounded) <= 2.0 ** -11 * mass + 2.0 ** -11 * np.abs(y_rounded) + noise), (bm, bn, bk, variant)
            target = y_rounded if rounded else y_exact
            assert np.all(np.abs(y - target) <= 2.0 ** -11 * np.abs(target) + 2.0 ** -24 + noise), (bm, bn, bk, variant)
            ran += 1
    assert ran == 5
    assert sk.kernel_name(sk.make_plan(1, N, K, "q4_zp", "nt", use_tuned=False).kernel_id) == "gemv_q4zp_nb1_wn1_rk4_k16384"
    sk.workspace_status()


F16_GEMV_TILES = [(16, 16, 512), (16, 16, 1024), (16, 32, 512), (16, 64, 128), (16, 32, 256), (16, 16, 256)]


def test_f16_matrix_vector_every_kernel(sk, oracle):
    """Every fp16 matrix-vector instance (M = 1, NT) on ragged shapes: N not a multiple of 16, K a
    multiple of 8 only, a strided W, K beyond 8192 (the instances that keep a longer A in LDS), all
    schedules and both fix-ups, against the fp32 host product.  On integer data (|sums| < 2048) the
    result must be exact."""
    import torch
    rng = np.random.default_rng(71)
    ran = 0
    for (N, K, pad) in [(1000, 1160, 0), (520, 392, 8), (72, 4096, 0), (2048, 8192, 64), (264, 28672, 0), (4099, 11008, 0)]:
        A = (rng.random((1, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        W = (rng.random((N, K + pad), dtype=np.float32) * 2 - 1).astype(np.float16)
        Ai = rng.integers(-1, 2, (1, K)).astype(np.float16)
        Wi = rng.integers(-2, 3, (N, K + pad)).astype(np.float16)
        ref = oracle.matmul_fp32(A, W[:, :K], trans_b=True)
        exact = Wi[:, :K].astype(np.int64) @ Ai[0].astype(np.int64)
        assert np.abs(exact).max() < 2048
        dA, dW, dAi, dWi = _t(A), _t(W)[:, :K], _t(Ai), _t(Wi)[:, :K]
        for (bm, bn, bk) in F16_GEMV_TILES:
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48),
                        dict(schedule="sk2", fixup="atomic", grid=40), dict(schedule="basic", fixup="reduce", grid=56)):
                try:
                    plan = sk.make_plan(1, N, K, "float16", "nt", dict(bm=bm, bn=bn, bk=bk, variant=3, **sch))
                except sk.StreamKError:
                    assert K > 8192  # only some instances take a long K
                    continue
                C = sk.streamk_fp16(dA, dW, plan=plan)
                assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (N, K, bm, bn, bk, sch, plan.kernel_id)
                C = sk.streamk_fp16(dAi, dWi, plan=plan)
                assert np.array_equal(C.cpu().numpy()[0].astype(np.int64), exact), (N, K, bm, bn, bk, sch)
                ran += 1
    assert ran >= 100
    # the heuristic plan for M = 1 is one of these kernels
    plan = sk.make_plan(1, 4096, 4096, "float16", "nt", {})
    assert (plan.bm, plan.bn, plan.bk) == (16, 16, 512) and 160 <= plan.kernel_id < 168
    sk.workspace_status()


def test_f16_few_rows_in_the_matrix_vector_form(sk, oracle):
    """2 <= M <= 4 on the kernels that stream the weights as the matrix-vector kernels do and multiply them with
    four rows of A: ragged N, K a multiple of 8 only, strided A and W, K beyond the 8192 values of A that stay in
    LDS at a time (several windows), all schedules and both fix-ups, fp16 and bfloat16, bias and activation;
    exact on integer data, within 2e-3 of the fp32 host product otherwise; 5 rows fall to the general kernel."""
    import torch
    rng = np.random.default_rng(73)
    ran = 0
    for (M, N, K, pad) in [(2, 1000, 1160, 0), (3, 520, 392, 8), (4, 72, 4096, 0), (4, 2048, 8192, 64), (3, 264, 28672, 0), (2, 4099, 11008, 0)]:
        A = (rng.random((M, K + pad), dtype=np.float32) * 2 - 1).astype(np.float16)
        W = (rng.random((N, K + pad), dtype=np.float32) * 2 - 1).astype(np.float16)
        Ai = rng.integers(-1, 2, (M, K + pad)).astype(np.float16)
        Wi = rng.integers(-2, 3, (N, K + pad)).astype(np.float16)
        ref = oracle.matmul_fp32(A[:, :K], W[:, :K], trans_b=True)
        exact = Ai[:, :K].astype(np.int64) @ Wi[:, :K].astype(np.int64).T
        assert np.abs(exact).max() < 2048
        dA, dW, dAi, dWi = _t(A)[:, :K], _t(W)[:, :K], _t(Ai)[:, :K], _t(Wi)[:, :K]
        for (bn, bk) in ((16, 512), (32, 512), (64, 256)):
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48),
                        dict(schedule="sk2", fixup="atomic", grid=40), dict(schedule="basic", fixup="reduce", grid=56)):
                plan = sk.make_plan(M, N, K, "float16", "nt", dict(bm=16, bn=bn, bk=bk, variant=4, **sch))
                assert sk.kernel_name(plan.kernel_id).startswith("gemv_rows_f16_m4")
                C = sk.streamk_fp16(dA, dW, plan=plan)
                assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, bn, bk, sch)
                C = sk.streamk_fp16(dAi, dWi, plan=plan)
                assert np.array_equal(C.cpu().numpy().astype(np.int64), exact), (M, N, K, bn, bk, sch)
                if bn != 64:   # bfloat16 twins of the first two
                    pb = sk.make_plan(M, N, K, "bfloat16", "nt", dict(bm=16, bn=bn, bk=bk, variant=4, **sch))
                    assert sk.kernel_name(pb.kernel_id).startswith("gemv_rows_bf16_m4")
                    C = sk.streamk_bf16(dAi.bfloat16(), dWi.bfloat16(), plan=pb)
                    # (the exact sums, rounded once to bfloat16's eight bits)
                    assert torch.equal(C.cpu(), torch.from_numpy(exact).float().bfloat16()), (M, N, K, bn, bk, sch)
                ran += 1
    assert ran >= 70
    # heuristic plans, bias and activation, an output with a row stride
    M, N, K = 3, 1000, 2048
    Ai = rng.integers(-1, 2, (M, K)).astype(np.float16)
    Wi = rng.integers(-1, 2, (N, K)).astype(np.float16)
    bias = rng.integers(-3, 4, N).astype(np.float16)
    want = np.maximum(Ai.astype(np.int64) @ Wi.astype(np.int64).T + bias.astype(np.int64), 0)
    # (the planner itself takes the kernels that stream the weights through LDS from two rows on; this form stays an
    # explicit choice)
    assert sk.kernel_name(sk.make_plan(M, N, K, "float16", "nt", use_tuned=False).kernel_id).startswith("stream_f16_")
    rows = dict(bm=16, bn=16, bk=512, variant=4)
    assert sk.kernel_name(sk.make_plan(M, N, K, "float16", "nt", rows).kernel_id) == "gemv_rows_f16_m4_wn1_rk4"
    for sch in (dict(), rows, dict(rows, schedule="sk2", fixup="reduce", grid=64), dict(rows, schedule="sk2", fixup="atomic", grid=64)):
        out = torch.zeros(M, N + 24, dtype=torch.float16, device="cuda")[:, 8:8 + N]
        C = sk.streamk_fp16(_t(Ai), _t(Wi), out=out, bias=_t(bias), activation="relu", **sch)
        assert np.array_equal(C.cpu().numpy().astype(np.int64), want), sch
    assert not sk.kernel_name(sk.make_plan(5, N, K, "float16", "nt", use_tuned=False).kernel_id).startswith("gemv_rows")
    with pytest.raises(sk.StreamKError):
        sk.make_plan(5, N, K, "float16", "nt", dict(bm=16, bn=16, bk=512, variant=4))
    sk.workspace_status()


def test_f16_weights_streamed_through_lds(sk, oracle):
    """Up to 96 rows of A on the kernels that stream the weights through LDS in contiguous loads (eight tile
    shapes, fp16 and bfloat16): ragged M and N, K a multiple of 8 only and shorter than one iteration, strided A
    and W, all schedules and both fix-ups, bias and activation, an output with a row stride; exact on integer data
    (every tile adds its K-iterations up from a different start), within 2e-3 of the fp32 host product otherwise."""
    import torch
    rng = np.random.default_rng(74)
    ran = 0
    shapes = {16: (16, 64, 256), 32: (32, 64, 256), 17: (16, 32, 512), 64: (64, 32, 256), 33: (32, 32, 256), 65: (64, 64, 256),
              18: (16, 16, 1024), 96: (96, 32, 256)}
    for (M, N, K, pad) in [(16, 1000, 1160, 0), (9, 520, 392, 8), (1, 72, 8, 0), (13, 2048, 8192, 64), (5, 264, 28672, 0),
                           (64, 4099, 4104, 0), (50, 328, 776, 8), (32, 200, 1032, 0), (27, 8192, 4096, 0), (96, 1000, 1160, 8),
                           (81, 8192, 2048, 0)]:
        A = (rng.random((M, K + pad), dtype=np.float32) * 2 - 1).astype(np.float16)
        W = (rng.random((N, K + pad), dtype=np.float32) * 2 - 1).astype(np.float16)
        Ai = rng.integers(-1, 2, (M, K + pad)).astype(np.float16)
        Wi = rng.integers(-2, 3, (N, K + pad)).astype(np.float16)
        ref = oracle.matmul_fp32(A[:, :K], W[:, :K], trans_b=True)
        exact = Ai[:, :K].astype(np.int64) @ Wi[:, :K].astype(np.int64).T
        assert np.abs(exact).max() < 2048
        dA, dW, dAi, dWi = _t(A)[:, :K], _t(W)[:, :K], _t(Ai)[:, :K], _t(Wi)[:, :K]
        for (bm, bn, bk) in shapes.values():
            if M > bm:
                with pytest.raises(sk.StreamKError):
                    sk.make_plan(M, N, K, "float16", "nt", dict(bm=bm, bn=bn, bk=bk, variant=5))
                continue
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48),
                        dict(schedule="sk2", fixup="atomic", grid=40), dict(schedule="basic", fixup="reduce", grid=56)):
                plan = sk.make_plan(M, N, K, "float16", "nt", dict(bm=bm, bn=bn, bk=bk, variant=5, **sch))
                assert sk.kernel_name(plan.kernel_id).startswith("stream_f16_")
                C = sk.streamk_fp16(dA, dW, plan=plan)
                assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, bm, bn, bk, sch)
                C = sk.streamk_fp16(dAi, dWi, plan=plan)
                assert np.array_equal(C.cpu().numpy().astype(np.int64), exact), (M, N, K, bm, bn, bk, sch)
                pb = sk.make_plan(M, N, K, "bfloat16", "nt", dict(bm=bm, bn=bn, bk=bk, variant=5, **sch))
                assert sk.kernel_name(pb.kernel_id).startswith("stream_bf16_")
                C = sk.streamk_bf16(dAi.bfloat16(), dWi.bfloat16(), plan=pb)
                # (the exact sums, rounded once to bfloat16's eight bits)
                assert torch.equal(C.cpu(), torch.from_numpy(exact).float().bfloat16()), (M, N, K, bm, bn, bk, sch)
                ran += 1
    assert ran >= 100
    # bias and activation, an output with a row stride
    M, N, K = 48, 1000, 2048
    Ai = rng.integers(-1, 2, (M, K)).astype(np.float16)
    Wi = rng.integers(-1, 2, (N, K)).astype(np.float16)
    bias = rng.integers(-3, 4, N).astype(np.float16)
    want = np.maximum(Ai.astype(np.int64) @ Wi.astype(np.int64).T + bias.astype(np.int64), 0)
    for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=64), dict(schedule="sk2", fixup="atomic", grid=64)):
        out = torch.zeros(M, N + 24, dtype=torch.float16, device="cuda")[:, 8:8 + N]
        C = sk.streamk_fp16(_t(Ai), _t(Wi), out=out, bias=_t(bias), activation="relu", bm=64, bn=32, bk=256, variant=5, **sch)
        assert np.array_equal(C.cpu().numpy().astype(np.int64), want), sch
    sk.workspace_status()


@pytest.mark.gpu
def test_device_quantiser_matches_host_and_feeds_the_gemm(sk, oracle):
    """sk_q4_quantize on the device writes the bytes sk_q4_quantize_host and the numpy restatement
    write (special groups included), and a Q4 GEMM on the result agrees with the fp32 product of
    the dequantised weights; against the unquantised weights the error is that of 4-bit rounding."""
    import torch
    rng = np.random.default_rng(81)
    for zero in (8, 0, 5, 15):
        N, K, pad = 1000, 4096, 8
        W = (rng.standard_normal((N, K + pad), dtype=np.float32) * 0.02).astype(np.float16)
        W[0, :128] = 0
        W[1, :128] = np.float16(6e-8) * rng.integers(-3, 4, 128)
        W[2, :128] = 65504 * rng.choice([-1, 1], 128)
        W[3, :128] = rng.integers(-40, 41, 128) * 0.25
        dW = _t(W)[:, :K]
        Wq, sc = sk.quantize_q4(dW, zero=zero)
        hWq, hsc = sk.quantize_q4(torch.from_numpy(W)[:, :K], zero=zero)
        nWq, nsc = oracle.quantize_q4_np(W[:, :K], zero=zero)
        assert torch.equal(Wq.cpu(), hWq) and np.array_equal(hWq.numpy(), nWq)
        assert torch.equal(sc.cpu().view(torch.int16), hsc.view(torch.int16))
        assert np.array_equal(hsc.numpy().view(np.uint16), nsc.view(np.uint16))
    W = (rng.standard_normal((2048, 4096), dtype=np.float32) * 0.02).astype(np.float16)
    Wq, sc = sk.quantize_q4(_t(W))
    for M in (1, 16):
        A = rng.standard_normal((M, 4096), dtype=np.float32).astype(np.float16)
        C = sk.streamk_q4(_t(A), Wq, sc)
        ref_q = oracle.q4_gemm_ref(A, Wq.cpu().numpy(), sc.cpu().numpy())
        assert _rel(oracle, C, ref_q) <= 2e-3 <= TOL
        ref = oracle.matmul_fp32(A, W, trans_b=True)
        assert _rel(oracle, C, ref) <= 0.12  # 4-bit weights: ~7 % rms per weight at 7 levels
    sk.workspace_status()


def test_linear_module_matches_functional_linear(sk, oracle):
    """StreamKLinear (fp16 and Q4 weights, with bias) against the fp32 host product for the shapes
    a model sends: one token, a decode batch, a [batch, tokens, K] prefill, an unaligned slice."""
    import torch
    torch.manual_seed(5)
    lin = torch.nn.Linear(1024, 1536, bias=True).half().cuda()
    lin.weight.data.mul_(2.0)
    fp = sk.StreamKLinear.from_linear(lin)
    q4 = sk.StreamKLinear.from_linear(lin, weight_format="q4")
    Wd = oracle.dequant_q4(q4.qweight.cpu().numpy(), q4.scales.cpu().numpy()).astype(np.float32)
    Wf, b = lin.weight.detach().float().cpu().numpy(), lin.bias.detach().float().cpu().numpy()
    big = torch.randn(40, 1032, device="cuda").half()
    for x in (torch.randn(1, 1024, device="cuda").half(), torch.randn(16, 1024, device="cuda").half(),
              torch.randn(3, 50, 1024, device="cuda").half(), big[:, 1:1025], torch.randn(1024, device="cuda").half(),
              torch.randn(2, 300, 1024, device="cuda").half()):
        xf = x.float().cpu().numpy().reshape(-1, 1024)
        for mod, W in ((fp, Wf), (q4, Wd)):
            y = mod(x)
            assert y.shape == x.shape[:-1] + (1536,) and y.dtype == torch.float16
            ref = xf @ W.T + b
            assert oracle.max_abs_rel(y.float().cpu().numpy().reshape(-1, 1536), ref) <= 2e-3 <= TOL
    # the operators keep one plan per (M, N, K, type, layout) they have been called with
    import sys
    cache = sys.modules["streamk.ops"]._plan_cache
    assert {k[0] for k in cache if k[1:5] == (1536, 1024, "float16", "nt")} >= {1, 16, 150, 40, 600}
    assert {k[0] for k in cache if k[1:5] == (1536, 1024, "q4", "nt")} >= {1, 16, 40}
    assert set(q4.state_dict()) == {"qweight", "scales", "bias"}
    # state round trip into a freshly constructed module
    fresh = sk.StreamKLinear(1024, 1536, bias=True, weight_format="q4", device="cuda")
    fresh.load_state_dict(q4.state_dict())
    x = torch.randn(4, 1024, device="cuda").half()
    assert torch.equal(fresh(x), q4(x))
    with pytest.raises(ValueError):
        fp(torch.randn(4, 1000, device="cuda").half())
    sk.workspace_status()


def test_bf16_tile_kernels(sk, oracle):
    """bfloat16 instances of the tile kernels, NT and NN: ragged shapes, every instance, all schedules
    and both fix-ups against the fp32 host product of the same (bfloat16-valued) operands; tolerance
    1e-2 (bfloat16 rounds C to 8 bits: 2^-9 relative).  On {-1, 0, 1} data with |sums| <= 256 the
    result must be exact, and the ordered reduce bitwise repeatable."""
    import torch
    torch.manual_seed(7)
    tiles = {"nt": [(256, 256, 64), (128, 128, 64), (128, 128, 32), (64, 64, 32), (128, 256, 64), (256, 128, 64), (64, 128, 32)],
             "nn": [(256, 256, 64), (128, 128, 64), (128, 256, 64), (256, 128, 64)]}
    for (M, N, K) in [(200, 136, 328), (1000, 1096, 1032), (520, 264, 64), (64, 512, 2048)]:
        A = (torch.rand(M, K) * 2 - 1).bfloat16()
        Ai = torch.randint(-1, 2, (M, K)).bfloat16()
        for layout in ("nt", "nn"):
            B = (torch.rand(*((N, K) if layout == "nt" else (K, N))) * 2 - 1).bfloat16()
            Bi = torch.randint(-1, 2, tuple(B.shape)).bfloat16()
            ref = oracle.matmul_fp32(A.float().numpy(), B.float().numpy(), trans_b=layout == "nt")
            exact = (Ai.double() @ (Bi.double().T if layout == "nt" else Bi.double())).numpy()
            dA, dB, dAi, dBi = A.cuda(), B.cuda(), Ai.cuda(), Bi.cuda()
            for (bm, bn, bk) in tiles[layout]:
                for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=24),
                            dict(schedule="sk2", fixup="atomic", grid=16)):
                    plan = sk.make_plan(M, N, K, "bfloat16", layout, dict(bm=bm, bn=bn, bk=bk, **sch))
                    C = sk.streamk_bf16(dA, dB, layout=layout, plan=plan)
                    assert C.dtype == torch.bfloat16 and _rel(oracle, C, ref) <= 4e-3 <= TOL, (M, N, K, layout, bm, bn, bk, sch)
                    Ci = sk.streamk_bf16(dAi, dBi, layout=layout, plan=plan)
                    if np.abs(exact).max() <= 256:
                        assert np.array_equal(Ci.double().cpu().numpy(), exact), (M, N, K, layout, bm, bn, bk, sch)
                    if sch.get("fixup") == "reduce":
                        assert torch.equal(C, sk.streamk_bf16(dA, dB, layout=layout, plan=plan))
    # heuristic plans, from one row to a large tile count; a float16 tensor is refused
    for (M, N, K) in [(1, 512, 1024), (16, 4096, 4096), (2048, 2048, 2048)]:
        A, B = (torch.rand(M, K) * 2 - 1).bfloat16(), (torch.rand(N, K) * 2 - 1).bfloat16()
        ref = oracle.matmul_fp32(A.float().numpy(), B.float().numpy(), trans_b=True)
        assert _rel(oracle, sk.streamk_bf16(A.cuda(), B.cuda()), ref) <= 4e-3
    with pytest.raises(TypeError):
        sk.streamk_bf16(torch.zeros(8, 64, dtype=torch.float16, device="cuda"), torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda"))
    sk.workspace_status()


def test_bf16_small_m_kernels(sk, oracle):
    """bfloat16 instances of the weight-streaming small-M kernels (M <= 64) and of the matrix-vector kernels: every instance, ragged N, K tails,
    data-parallel, Stream-K with both fix-ups and fixed split-K; {-1,0,1} operands must come out exact (|sums| <= 256)
    and random ones within 4e-3 of the fp32 host product (bfloat16 rounds C to 8 bits); the bias and activation
    epilogue in bfloat16; the plans the library picks by itself for 1..32 rows are these kernels."""
    import torch
    torch.manual_seed(17)
    cfgs = SKINNY_CONFIGS + [dict(bm=16, bn=16, bk=128, variant=2), dict(bm=16, bn=64, bk=128, variant=2)]
    # the matrix-vector instances (one row of A, 4x4x4 MFMAs)
    cfgs += [dict(bm=16, bn=16, bk=512, variant=3), dict(bm=16, bn=16, bk=1024, variant=3), dict(bm=16, bn=32, bk=512, variant=3),
             dict(bm=16, bn=64, bk=128, variant=3), dict(bm=16, bn=32, bk=256, variant=3), dict(bm=16, bn=16, bk=256, variant=3)]
    N, K = 1000, 1032
    B = (torch.rand(N, K) * 2 - 1).bfloat16()
    Bi = torch.randint(-1, 2, (N, K)).bfloat16()
    bias = torch.randint(-20, 20, (N,)).bfloat16()
    for cfg in cfgs:
        row1 = cfg.get("variant") in (2, 3)
        for M in ((1,) if row1 else (cfg["bm"], cfg["bm"] - 3, 1)):
            A = (torch.rand(M, K) * 2 - 1).bfloat16()
            Ai = torch.randint(-1, 2, (M, K)).bfloat16()
            Ai[:, 200:] = 0  # keeps the sums within bfloat16's exact integers
            ref = oracle.matmul_fp32(A.float().numpy(), B.float().numpy(), trans_b=True)
            exact = (Ai.double() @ Bi.double().T).numpy()
            assert np.abs(exact).max() <= 256
            schedules = [dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=24),
                         dict(schedule="sk2", fixup="atomic", grid=20)]
            if -(-K // cfg["bk"]) % 3 == 0:  # fixed split-K takes a factor of the K-iteration count
                schedules.append(dict(schedule="splitk", split=3, fixup="reduce"))
            for sch in schedules:
                plan = sk.make_plan(M, N, K, "bfloat16", "nt", dict(cfg, **sch))
                # (without a variant, one row takes the matrix-vector instance of the same tile where there is one)
                assert (241 if cfg.get("variant") == 3 else 230) <= plan.kernel_id <= (240 if M > 1 else 248), (cfg, plan.kernel_id)
                C = sk.streamk_bf16(A.cuda(), B.cuda(), plan=plan)
                assert C.dtype == torch.bfloat16 and _rel(oracle, C, ref) <= 4e-3 <= TOL, (cfg, M, sch)
                Ci = sk.streamk_bf16(Ai.cuda(), Bi.cuda(), plan=plan)
                assert np.array_equal(Ci.double().cpu().numpy(), exact), (cfg, M, sch)
                Cb = sk.streamk_bf16(Ai.cuda(), Bi.cuda(), plan=plan, bias=bias.cuda(), activation="relu")
                assert np.array_equal(Cb.double().cpu().numpy(), np.maximum(exact + bias.double().numpy(), 0)), (cfg, M, sch)
                if sch.get("fixup") == "reduce":
                    assert torch.equal(C, sk.streamk_bf16(A.cuda(), B.cuda(), plan=plan))
    for M in (1, 2, 16, 32):
        plan = sk.make_plan(M, 4096, 4096, "bfloat16", "nt")
        # (one row of 4096 x 4096: matrix-vector kernels; more rows: the general kernels or the ones that stream the
        # weights through LDS)
        assert (241 <= plan.kernel_id <= 248) if M == 1 else (230 <= plan.kernel_id <= 240 or
                                                               plan.kernel_id in (282, 283, 285, 287, 289, 293, 297)), (M, plan.kernel_id)
        A, W = (torch.rand(M, 4096) * 2 - 1).bfloat16(), (torch.rand(4096, 4096) * 2 - 1).bfloat16()
        ref = oracle.matmul_fp32(A.float().numpy(), W.float().numpy(), trans_b=True)
        assert _rel(oracle, sk.streamk_bf16(A.cuda(), W.cuda()), ref) <= 4e-3, M
    # a shape tuned for fp16 only: the bfloat16 plan takes that entry where its kernel has a bfloat16 twin
    for shape in ((256, 4096, 4096), (16, 4096, 4096), (2048, 8192, 8192)):
        cfg = sk.tuned_config(*shape, "float16")
        if sk.tuned_config(*shape, "bfloat16") is None and cfg:
            try:
                want = sk.make_plan(*shape, "bfloat16", "nt", cfg)
            except sk.StreamKError:
                continue  # no bfloat16 instance of that kernel: the heuristic plans the shape
            got = sk.make_plan(*shape, "bfloat16")
            assert (got.kernel_id, got.grid, got.schedule) == (want.kernel_id, want.grid, want.schedule), shape
    sk.workspace_status()


def test_fp8_tile_kernels(sk, oracle):
    """fp8 (OCP e4m3) operands, fp16 C: every instance, ragged shapes, K tails (K a multiple of 16 but not
    of the 128-value iteration), all schedules and both fix-ups against the float64 host product of the
    decoded bytes; tolerance 1e-2 (measured <= 1e-3: fp16 rounding of C).  On {-1, 0, 1} data with
    |sums| <= 2048 the result must equal the host product exactly -- any mispairing of A and B bytes along
    K would show -- and the ordered reduce must be bitwise repeatable."""
    import torch
    torch.manual_seed(11)
    f8 = torch.float8_e4m3fn
    # (bm, bn, bk): two stages of 128 K-values (the default of a tile shape), four stages of 64
    tiles = [(256, 256, 128), (128, 128, 128), (128, 256, 128), (256, 128, 128), (64, 128, 128), (128, 128, 64), (64, 128, 64)]
    for (M, N, K) in [(200, 136, 336), (1000, 1096, 1040), (520, 264, 128), (64, 512, 2048), (300, 300, 16)]:
        A, B = torch.randn(M, K).to(f8), torch.randn(N, K).to(f8)
        Ai, Bi = torch.randint(-1, 2, (M, K)).float().to(f8), torch.randint(-1, 2, (N, K)).float().to(f8)
        ref = oracle.f8_gemm_ref(A.view(torch.uint8).numpy(), B.view(torch.uint8).numpy())
        exact = oracle.f8_gemm_ref(Ai.view(torch.uint8).numpy(), Bi.view(torch.uint8).numpy())
        assert np.abs(exact).max() <= 2048
        dA, dB, dAi, dBi = A.cuda(), B.cuda(), Ai.cuda(), Bi.cuda()
        for (bm, bn, bk) in tiles:
            for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=24),
                        dict(schedule="sk2", fixup="atomic", grid=16), dict(schedule="sk1", fixup="reduce", grid=7)):
                plan = sk.make_plan(M, N, K, "float8_e4m3", "nt", dict(bm=bm, bn=bn, **(dict(bk=64) if bk == 64 else {}), **sch))
                assert plan.bk == bk and plan.iters_per_tile == -(-K // bk)
                assert sk.kernel_name(plan.kernel_id) == (f"tile_f8e4m3_nt_dma_{bm}x{bn}x{bk}" if (bm, bn) != (256, 256) or K % 128 else "tile_f8e4m3_nt_asm_256x256x128")
                C = sk.streamk_fp8(dA, dB, plan=plan)
                assert C.dtype == torch.float16 and _rel(oracle, C, ref) <= 1e-3 <= TOL, (M, N, K, bm, bn, bk, sch)
                Ci = sk.streamk_fp8(dAi.view(torch.uint8), dBi.view(torch.uint8), plan=plan)   # raw bytes are accepted too
                assert np.array_equal(Ci.double().cpu().numpy(), exact), (M, N, K, bm, bn, bk, sch)
                if sch.get("fixup") == "reduce":
                    assert torch.equal(C, sk.streamk_fp8(dA, dB, plan=plan))
                if bk == 64:   # the e5m2 twin of the four-stage kernels, on exact data
                    p5 = sk.make_plan(M, N, K, "float8_e5m2", "nt", dict(bm=bm, bn=bn, bk=64, **sch))
                    assert sk.kernel_name(p5.kernel_id) == f"tile_f8e5m2_nt_dma_{bm}x{bn}x64"
                    C5 = sk.streamk_fp8(Ai.to(torch.float8_e5m2).cuda(), Bi.to(torch.float8_e5m2).cuda(), plan=p5)
                    assert np.array_equal(C5.double().cpu().numpy(), exact), (M, N, K, bm, bn, sch)
    # the four-wave kernels whose K loop is assembly (K a multiple of 128; one 16x16x128 MFMA per accumulator block
    # and iteration): both formats, every schedule and fix-up incl. the halves exchange, alpha, bias and activation;
    # same bits as the eight-wave 32x32x64 kernel (the K-values are summed in the same groups of 128)
    assert sk.kernel_name(sk.make_plan(4096, 4096, 4096, "float8_e4m3", "nt", use_tuned=False).kernel_id) == "tile_f8e4m3_nt_asm_256x256x128"
    assert "asm" not in sk.kernel_name(sk.make_plan(4096, 4096, 4112, "float8_e4m3", "nt", use_tuned=False).kernel_id)
    ran = 0
    for (M, N, K) in [(256, 256, 128), (200, 136, 384), (1000, 1096, 2048), (520, 264, 896)]:
        for fmt, name, dec in ((f8, "float8_e4m3", oracle.f8_gemm_ref), (torch.float8_e5m2, "float8_e5m2", None)):
            A, B = torch.randn(M, K).to(fmt), torch.randn(N, K).to(fmt)
            Ai, Bi = torch.randint(-1, 2, (M, K)).float().to(fmt), torch.randint(-1, 2, (N, K)).float().to(fmt)
            ref = (A.double() @ B.double().T).numpy() * 0.25
            exact = (Ai.double() @ Bi.double().T).numpy()
            if dec is not None:
                assert np.array_equal(dec(Ai.view(torch.uint8).numpy(), Bi.view(torch.uint8).numpy()), exact)
            dA, dB, dAi, dBi = A.cuda(), B.cuda(), Ai.cuda(), Bi.cuda()
            for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7), dict(schedule="basic", fixup="atomic", grid=5),
                        dict(schedule="splitk", split=2, fixup="reduce"), dict(schedule="sk1", fixup="reduce", grid=2, raster=2)):
                try:
                    plan = sk.make_plan(M, N, K, name, "nt", dict(bm=256, bn=256, variant=8, **sch))
                except sk.StreamKError:
                    assert sch["schedule"] == "splitk"
                    continue
                assert sk.kernel_name(plan.kernel_id) == f"tile_f8{'e4m3' if fmt is f8 else 'e5m2'}_nt_asm_256x256x128"
                assert np.array_equal(sk.streamk_fp8(dAi, dBi, plan=plan).double().cpu().numpy(), exact), (M, N, K, name, sch)
                C = sk.streamk_fp8(dA, dB, alpha=0.25, plan=plan)
                assert _rel(oracle, C, ref) <= 1e-3 <= TOL, (M, N, K, name, sch)
                if sch["schedule"] == "dp" or sch.get("fixup") == "reduce":
                    twin = sk.streamk_fp8(dA, dB, alpha=0.25, **dict(sch, bm=256, bn=256, variant=7))
                    assert torch.equal(C, twin), (M, N, K, name, sch)
                ran += 1
    assert ran >= 30
    M, N, K = 520, 264, 896
    Ai, Bi = torch.randint(-1, 2, (M, K)).float().to(f8).cuda(), torch.randint(-1, 2, (N, K)).float().to(f8).cuda()
    bias = torch.randint(-3, 4, (N,)).half().cuda()
    want = torch.relu((Ai.float() @ Bi.float().T) * 2.0 + bias.float())
    for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7)):
        C = sk.streamk_fp8(Ai, Bi, alpha=2.0, bias=bias, activation="relu", bm=256, bn=256, variant=8, **sch)
        assert torch.equal(C.float(), want), sch
    # heuristic plans from one row to many tiles; strided operands (leading dimension a multiple of 16)
    for (M, N, K) in [(1, 512, 1024), (16, 4096, 4096), (2048, 2048, 2048), (1024, 8192, 8192)]:
        A, B = torch.randn(M, K).to(f8), torch.randn(N, K).to(f8)
        rows = np.random.RandomState(M).choice(M, size=min(M, 64), replace=False)
        ref = oracle.f8_gemm_ref(A.view(torch.uint8).numpy()[rows], B.view(torch.uint8).numpy())
        C = sk.streamk_fp8(A.cuda(), B.cuda())
        assert oracle.max_abs_rel(C.float().cpu().numpy()[rows], ref) <= 1e-3
    big = torch.randn(300, 1024).to(f8).cuda()
    A, B = big[:200, 16:16 + 640], big[40:, 256:256 + 640]
    ref = oracle.f8_gemm_ref(A.cpu().view(torch.uint8).numpy(), B.cpu().view(torch.uint8).numpy())
    assert _rel(oracle, sk.streamk_fp8(A, B), ref) <= 1e-3
    # every byte value except the NaN patterns (subnormals, +-0, +-448), against partners 0 and +-2^-6
    allv = torch.tensor([b for b in range(256) if b & 127 != 127], dtype=torch.uint8)
    A = torch.stack([allv.repeat(4)[torch.randperm(1016)[:1008]] for _ in range(40)])
    B = torch.tensor([0x00, 0x08, 0x88], dtype=torch.uint8)[torch.randint(0, 3, (24, 1008))]
    ref = oracle.f8_gemm_ref(A.numpy(), B.numpy())
    assert _rel(oracle, sk.streamk_fp8(A.cuda(), B.cuda()), ref) <= 1e-3
    # alpha scales the fp32 sums before the rounding to fp16: operands near the top of the range, whose plain
    # product overflows fp16 (448 * 448 * K), come back finite and accurate with alpha = 2^-14
    A = (torch.rand(130, 512) * 200 + 200).to(f8)
    B = (torch.rand(70, 512) * 200 + 200).to(f8)
    ref = oracle.f8_gemm_ref(A.view(torch.uint8).numpy(), B.view(torch.uint8).numpy())
    assert torch.isinf(sk.streamk_fp8(A.cuda(), B.cuda())).all() and ref.min() > 65504
    for cfg in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=8), dict(schedule="basic", fixup="atomic", grid=8)):
        C = sk.streamk_fp8(A.cuda(), B.cuda(), alpha=2.0 ** -14, bm=128, bn=128, **cfg)
        assert _rel(oracle, C, ref * 2.0 ** -14) <= 1e-3, cfg
    Cp = sk.streamk_fp8(A.cuda(), B.cuda(), alpha=2.0 ** -14, bm=128, bn=128, schedule="dp")
    Cn = sk.streamk_fp8(A.cuda(), B.cuda(), alpha=-2.0 ** -15, bm=128, bn=128, schedule="dp")
    assert torch.equal(Cn * -2, Cp)     # sign and power of two: exact
    with pytest.raises(sk.StreamKError):
        sk.streamk_fp8(A.cuda(), B.cuda(), alpha=float("nan"))
    with pytest.raises(TypeError):
        sk.streamk_fp8(torch.zeros(8, 64, dtype=torch.float16, device="cuda"), torch.zeros(8, 64, dtype=torch.uint8, device="cuda"))
    with pytest.raises(sk.StreamKError):
        sk.streamk_fp8(torch.zeros(8, 72, dtype=torch.uint8, device="cuda"), torch.zeros(8, 72, dtype=torch.uint8, device="cuda"))
    with pytest.raises(sk.StreamKError):
        sk.make_plan(64, 64, 128, "float8_e4m3", "nn")
    sk.workspace_status()


def test_fp8_small_m_kernels(sk, oracle):
    """Weight-streaming fp8 kernels (M <= 64; e4m3 and e5m2): every instance, ragged N, a K tail (K a multiple of 16
    only), data-parallel and Stream-K with both fix-ups, against the float64 host product of the decoded bytes
    (1e-3: fp16 rounding of C); {-1,0,1} data must come out exact -- a lane's 16 bytes are split over two MFMAs, so
    any mispairing of A and weight bytes along K would show; alpha, bias and activation in the epilogue; the plans
    the library picks for 1..64 rows are these kernels."""
    import torch
    torch.manual_seed(23)
    cfgs = [dict(bm=16, bn=64, bk=256), dict(bm=32, bn=64, bk=256), dict(bm=16, bn=16, bk=1024), dict(bm=16, bn=32, bk=512),
            dict(bm=16, bn=32, bk=1024), dict(bm=16, bn=64, bk=512), dict(bm=32, bn=64, bk=512), dict(bm=16, bn=64, bk=256, variant=2),
            dict(bm=64, bn=64, bk=256), dict(bm=64, bn=64, bk=512)]
    N, K = 1000, 2064
    bias = torch.randint(-20, 20, (N,)).half()
    for fmt, dt in (("e4m3", torch.float8_e4m3fn), ("e5m2", torch.float8_e5m2)):
        first, last = (250, 259) if fmt == "e4m3" else (260, 269)
        B = torch.randn(N, K).to(dt)
        Bi = torch.randint(-1, 2, (N, K)).float().to(dt)
        for cfg in cfgs:
            for M in ((1,) if cfg.get("variant") == 2 else (cfg["bm"], cfg["bm"] - 3, 1)):
                A = torch.randn(M, K).to(dt)
                Ai = torch.randint(-1, 2, (M, K)).float().to(dt)
                ref = oracle.f8_gemm_ref(A.view(torch.uint8).numpy(), B.view(torch.uint8).numpy(), fmt)
                exact = oracle.f8_gemm_ref(Ai.view(torch.uint8).numpy(), Bi.view(torch.uint8).numpy(), fmt)
                assert np.abs(exact).max() <= 2048
                for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=24), dict(schedule="sk2", fixup="atomic", grid=20)):
                    plan = sk.make_plan(M, N, K, "float8_" + fmt, "nt", dict(cfg, **sch))
                    assert first <= plan.kernel_id <= last and plan.iters_per_tile == -(-K // cfg["bk"]), (fmt, cfg, plan.kernel_id)
                    C = sk.streamk_fp8(A.cuda(), B.cuda(), plan=plan)
                    assert C.dtype == torch.float16 and _rel(oracle, C, ref) <= 1e-3 <= TOL, (fmt, cfg, M, sch)
                    Ci = sk.streamk_fp8(Ai.cuda(), Bi.cuda(), plan=plan)
                    assert np.array_equal(Ci.double().cpu().numpy(), exact), (fmt, cfg, M, sch)
                    Cb = sk.streamk_fp8(Ai.cuda(), Bi.cuda(), plan=plan, alpha=0.5, bias=bias.cuda(), activation="relu")
                    assert np.array_equal(Cb.double().cpu().numpy(), np.maximum(0.5 * exact + bias.double().numpy(), 0)), (fmt, cfg, M, sch)
                    if sch.get("fixup") == "reduce":
                        assert torch.equal(C, sk.streamk_fp8(A.cuda(), B.cuda(), plan=plan))
        for M in (1, 7, 16, 32, 64):
            plan = sk.make_plan(M, 4096, 4096, "float8_" + fmt, "nt")
            assert first <= plan.kernel_id <= last, (fmt, M, plan.kernel_id)
            A, W = torch.randn(M, 4096).to(dt), torch.randn(4096, 4096).to(dt)
            ref = oracle.f8_gemm_ref(A.view(torch.uint8).numpy(), W.view(torch.uint8).numpy(), fmt)
            assert _rel(oracle, sk.streamk_fp8(A.cuda(), W.cuda()), ref) <= 1e-3, (fmt, M)
    # an e5m2 shape without a tuned entry of its own takes the e4m3 entry (twin kernels)
    if sk.tuned_config(1, 8192, 8192, "float8_e5m2") is None and sk.tuned_config(1, 8192, 8192, "float8_e4m3"):
        want, got = sk.make_plan(1, 8192, 8192, "float8_e4m3"), sk.make_plan(1, 8192, 8192, "float8_e5m2")
        assert (got.bm, got.bn, got.bk, got.grid, got.schedule) == (want.bm, want.bn, want.bk, want.grid, want.schedule)
        assert got.kernel_id == want.kernel_id + 10
    # strided operands (leading dimensions a multiple of 16 bytes)
    big = torch.randn(300, 4096).to(torch.float8_e4m3fn).cuda()
    A, W = big[:9, 16:16 + 2048], big[40:, 1024:1024 + 2048]
    ref = oracle.f8_gemm_ref(A.cpu().view(torch.uint8).numpy(), W.cpu().view(torch.uint8).numpy())
    assert _rel(oracle, sk.streamk_fp8(A, W), ref) <= 1e-3
    sk.workspace_status()


def test_int8_small_m_kernels(sk, oracle):
    """Weight-streaming int8 kernels (M <= 64, int32 C): every instance, ragged N, a K tail, data-parallel and
    Stream-K with both fix-ups and the K split over waves -- all must equal the host product in int64 exactly, on
    the full int8 range (-128 included); strided operands; the plans the library picks for 1..64 rows."""
    import torch
    g = torch.Generator().manual_seed(29)
    cfgs = [dict(bm=16, bn=64, bk=256), dict(bm=32, bn=64, bk=256), dict(bm=16, bn=16, bk=1024), dict(bm=16, bn=32, bk=512),
            dict(bm=16, bn=32, bk=1024), dict(bm=16, bn=64, bk=512), dict(bm=32, bn=64, bk=512), dict(bm=16, bn=64, bk=256, variant=2),
            dict(bm=64, bn=64, bk=256), dict(bm=64, bn=64, bk=512)]
    N, K = 1000, 2064
    B = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    for cfg in cfgs:
        for M in ((1,) if cfg.get("variant") == 2 else (cfg["bm"], cfg["bm"] - 3, 1)):
            A = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
            ref = oracle.i8_gemm_ref(A.numpy(), B.numpy())
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=24), dict(schedule="sk2", fixup="atomic", grid=20)):
                plan = sk.make_plan(M, N, K, "int8", "nt", dict(cfg, **sch))
                assert 270 <= plan.kernel_id <= 279 and plan.iters_per_tile == -(-K // cfg["bk"]), (cfg, plan.kernel_id)
                C = sk.streamk_int8(A.cuda(), B.cuda(), plan=plan)
                assert C.dtype == torch.int32 and np.array_equal(C.cpu().numpy(), ref), (cfg, M, sch)
    for M in (1, 7, 16, 32, 64):
        plan = sk.make_plan(M, 4096, 4096, "int8", "nt")
        assert 270 <= plan.kernel_id <= 279, (M, plan.kernel_id)
        A = torch.randint(-128, 128, (M, 4096), generator=g, dtype=torch.int8)
        W = torch.randint(-128, 128, (4096, 4096), generator=g, dtype=torch.int8)
        assert np.array_equal(sk.streamk_int8(A.cuda(), W.cuda()).cpu().numpy(), oracle.i8_gemm_ref(A.numpy(), W.numpy())), M
    big = torch.randint(-128, 128, (300, 4096), generator=g, dtype=torch.int8).cuda()
    A, W = big[:9, 16:16 + 2048], big[40:, 1024:1024 + 2048]
    out = torch.full((9, 264), 7, dtype=torch.int32, device="cuda")   # a strided C: columns beyond N stay untouched
    sk.streamk_int8(A, W, out=out[:, :260])
    assert np.array_equal(out[:, :260].cpu().numpy(), oracle.i8_gemm_ref(A.cpu().numpy(), W.cpu().numpy()))
    assert bool((out[:, 260:] == 7).all())
    sk.workspace_status()


def test_fp8_e5m2_tile_kernels(sk, oracle):
    """The e5m2 instances of the fp8 kernels: same checks as for e4m3 on fewer shapes (the two differ in one
    immediate operand of the MFMA): host product of the decoded bytes within 1e-3, {-1,0,1} data exact, every
    finite byte value, mixed formats refused."""
    import torch
    torch.manual_seed(13)
    f8 = torch.float8_e5m2
    for (M, N, K) in [(200, 136, 336), (520, 264, 1040)]:
        A, B = torch.randn(M, K).to(f8), torch.randn(N, K).to(f8)
        Ai, Bi = torch.randint(-1, 2, (M, K)).float().to(f8), torch.randint(-1, 2, (N, K)).float().to(f8)
        ref = oracle.f8_gemm_ref(A.view(torch.uint8).numpy(), B.view(torch.uint8).numpy(), "e5m2")
        exact = oracle.f8_gemm_ref(Ai.view(torch.uint8).numpy(), Bi.view(torch.uint8).numpy(), "e5m2")
        for (bm, bn) in [(256, 256), (128, 128), (128, 256), (256, 128), (64, 128)]:
            for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=24), dict(schedule="sk2", fixup="atomic", grid=16)):
                plan = sk.make_plan(M, N, K, "float8_e5m2", "nt", dict(bm=bm, bn=bn, **sch))
                assert "e5m2" in sk.kernel_name(plan.kernel_id)
                C = sk.streamk_fp8(A.cuda(), B.cuda(), plan=plan)
                assert _rel(oracle, C, ref) <= 1e-3 <= TOL, (M, N, K, bm, bn, sch)
                Ci = sk.streamk_fp8(Ai.cuda().view(torch.uint8), Bi.cuda().view(torch.uint8), fmt="e5m2", plan=plan)
                assert np.array_equal(Ci.double().cpu().numpy(), exact), (M, N, K, bm, bn, sch)
    # every finite byte value against partners 0 and +-2^-14 (57344 * 2^-14 = 3.5)
    allv = torch.tensor([b for b in range(256) if b & 127 < 0x7C], dtype=torch.uint8)
    A = torch.stack([allv.repeat(5)[torch.randperm(1240)[:1008]] for _ in range(40)])
    B = torch.tensor([0x00, 0x04, 0x84], dtype=torch.uint8)[torch.randint(0, 3, (24, 1008))]
    ref = oracle.f8_gemm_ref(A.numpy(), B.numpy(), "e5m2")
    assert _rel(oracle, sk.streamk_fp8(A.cuda(), B.cuda(), fmt="e5m2"), ref) <= 1e-3
    with pytest.raises(TypeError):
        sk.streamk_fp8(torch.zeros(8, 64, device="cuda").to(f8), torch.zeros(8, 64, device="cuda").to(torch.float8_e4m3fn))
    with pytest.raises(ValueError):
        sk.streamk_fp8(torch.zeros(8, 64, device="cuda").to(f8), torch.zeros(8, 64, device="cuda").to(f8),
                       plan=sk.make_plan(8, 8, 64, "float8_e4m3", "nt"))
    sk.workspace_status()


def test_int8_tile_kernels(sk, oracle):
    """int8 operands, int32 C: integer arithmetic, so every instance, schedule and fix-up (the atomic one
    included) must return the host's exact product, on the full range -128..127, ragged shapes, K tails,
    strided operands and an output whose rows are not 16-byte aligned."""
    import torch
    torch.manual_seed(12)
    # (bm, bn, bk): two stages of 128 K-values (the default of a tile shape), four stages of 64
    tiles = [(256, 256, 128), (128, 128, 128), (128, 256, 128), (256, 128, 128), (64, 128, 128), (128, 128, 64), (64, 128, 64)]
    for (M, N, K) in [(200, 136, 336), (1000, 1096, 1040), (520, 264, 128), (64, 512, 2048), (300, 300, 16)]:
        A = torch.randint(-128, 128, (M, K), dtype=torch.int8)
        B = torch.randint(-128, 128, (N, K), dtype=torch.int8)
        ref = torch.from_numpy(oracle.i8_gemm_ref(A.numpy(), B.numpy()))
        dA, dB = A.cuda(), B.cuda()
        for (bm, bn, bk) in tiles:
            for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=24),
                        dict(schedule="sk2", fixup="atomic", grid=16), dict(schedule="sk1", fixup="reduce", grid=7),
                        dict(schedule="basic", fixup="atomic", grid=40, raster=1)):
                plan = sk.make_plan(M, N, K, "int8", "nt", dict(bm=bm, bn=bn, **(dict(bk=64) if bk == 64 else {}), **sch))
                assert plan.bk == bk and plan.iters_per_tile == -(-K // bk)
                assert sk.kernel_name(plan.kernel_id).endswith(f"_{bm}x{bn}x{bk}")
                C = sk.streamk_int8(dA, dB, plan=plan)
                assert C.dtype == torch.int32 and torch.equal(C.cpu().long(), ref), (M, N, K, bm, bn, bk, sch)
    # the four-wave kernel with the K loop in assembly (K a multiple of 128): every schedule, both fix-ups, the
    # halves exchange of a tile split in two
    assert sk.kernel_name(sk.make_plan(4096, 4096, 4096, "int8", "nt", use_tuned=False).kernel_id) == "tile_i8_nt_asm_256x256x128"
    assert "asm" not in sk.kernel_name(sk.make_plan(4096, 4096, 4112, "int8", "nt", use_tuned=False).kernel_id)
    for (M, N, K) in [(256, 256, 128), (200, 136, 384), (1000, 1096, 2048), (520, 264, 896)]:
        A = torch.randint(-128, 128, (M, K), dtype=torch.int8)
        B = torch.randint(-128, 128, (N, K), dtype=torch.int8)
        ref = torch.from_numpy(oracle.i8_gemm_ref(A.numpy(), B.numpy()))
        dA, dB = A.cuda(), B.cuda()
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=7), dict(schedule="basic", fixup="atomic", grid=5),
                    dict(schedule="sk2", fixup="reduce", grid=3), dict(schedule="splitk", split=2, fixup="reduce"),
                    dict(schedule="splitk", split=2, fixup="atomic"), dict(schedule="sk1", fixup="reduce", grid=2, raster=2)):
            try:
                plan = sk.make_plan(M, N, K, "int8", "nt", dict(bm=256, bn=256, variant=8, **sch))
            except sk.StreamKError:
                assert sch["schedule"] == "splitk"
                continue
            assert sk.kernel_name(plan.kernel_id) == "tile_i8_nt_asm_256x256x128"
            C = sk.streamk_int8(dA, dB, plan=plan)
            assert torch.equal(C.cpu().long(), ref), (M, N, K, sch)
    # heuristic plans; extreme values (K * 128 * 128 stays below 2^31)
    for (M, N, K) in [(1, 512, 1024), (16, 4096, 4096), (2048, 2048, 2048), (1024, 8192, 8192)]:
        A = torch.randint(-128, 128, (M, K), dtype=torch.int8)
        B = torch.randint(-128, 128, (N, K), dtype=torch.int8)
        rows = np.random.RandomState(M).choice(M, size=min(M, 64), replace=False)
        ref = torch.from_numpy(oracle.i8_gemm_ref(A.numpy()[rows], B.numpy()))
        assert torch.equal(sk.streamk_int8(A.cuda(), B.cuda()).cpu().long()[rows], ref)
    A = torch.full((130, 4096), -128, dtype=torch.int8)
    B = torch.full((70, 4096), -128, dtype=torch.int8)
    B[::2] = 127
    assert torch.equal(sk.streamk_int8(A.cuda(), B.cuda()).cpu().long(), torch.from_numpy(oracle.i8_gemm_ref(A.numpy(), B.numpy())))
    big = torch.randint(-128, 128, (300, 1024), dtype=torch.int8).cuda()
    A, B = big[:200, 16:16 + 640], big[40:, 256:256 + 640]
    ref = torch.from_numpy(oracle.i8_gemm_ref(A.cpu().numpy(), B.cpu().numpy()))
    out = torch.zeros(200, 263, dtype=torch.int32, device="cuda")[:, 1:261]     # ldc 263, first column misaligned
    assert torch.equal(sk.streamk_int8(A, B, out=out).cpu().long(), ref)
    with pytest.raises(TypeError):
        sk.streamk_int8(torch.zeros(8, 64, dtype=torch.uint8, device="cuda"), torch.zeros(8, 64, dtype=torch.int8, device="cuda"))
    with pytest.raises(sk.StreamKError):
        sk.streamk_int8(torch.zeros(8, 72, dtype=torch.int8, device="cuda"), torch.zeros(8, 72, dtype=torch.int8, device="cuda"))
    with pytest.raises(sk.StreamKError):
        sk.make_plan(64, 64, 128, "int8", "nn")
    sk.workspace_status()


def test_fused_bias_epilogue(sk, oracle):
    """bias (one value per column, C's type) added in fp32 before the rounding: every kernel family (LDS-tiled
    with both accumulator layouts and the register-staged variant, NN, bfloat16, small-M, matrix-vector, Q4 in
    all formats), data-parallel and both fix-ups, ragged N; {-1,0,1} operands with an integer bias must come out
    exact, which also shows that the bias is added once per tile however many CTAs share it."""
    import torch
    rng = np.random.default_rng(91)
    cases = [  # (M, N, K, layout, config)
        (200, 1000, 328, "nt", dict(bm=256, bn=256, bk=64, variant=5)), (200, 1000, 328, "nt", dict(bm=128, bn=128, bk=64, variant=2)),
        (200, 1000, 328, "nt", dict(bm=128, bn=128, bk=64, variant=1)), (200, 1000, 328, "nt", dict(bm=64, bn=64, bk=32, variant=6)),
        (200, 1000, 328, "nn", dict(bm=128, bn=128, bk=64, variant=5)), (200, 1000, 328, "nn", dict(bm=256, bn=128, bk=64, variant=2)),
        (40, 1000, 1024, "nt", dict(bm=64, bn=64, bk=128)), (9, 1000, 1024, "nt", dict(bm=16, bn=32, bk=512)),
        (1, 1000, 1024, "nt", dict(bm=16, bn=16, bk=512, variant=3)), (1, 1000, 1024, "nt", dict(bm=16, bn=64, bk=128, variant=2)),
    ]
    for (M, N, K, layout, cfg) in cases:
        A = rng.integers(-1, 2, (M, K)).astype(np.float16)
        B = rng.integers(-1, 2, (N, K) if layout == "nt" else (K, N)).astype(np.float16)
        bias = rng.integers(-300, 300, N).astype(np.float16)
        want = (A.astype(np.float64) @ (B.T if layout == "nt" else B).astype(np.float64)) + bias.astype(np.float64)
        Af = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        bf = (rng.random(N, dtype=np.float32) * 20 - 10).astype(np.float16)
        reff = oracle.matmul_fp32(Af, B, trans_b=layout == "nt") + bf.astype(np.float32)
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=12), dict(schedule="sk2", fixup="atomic", grid=10)):
            plan = sk.make_plan(M, N, K, "float16", layout, dict(cfg, **sch))
            C = sk.streamk_fp16(_t(A), _t(B), layout=layout, plan=plan, bias=_t(bias))
            assert np.array_equal(C.double().cpu().numpy(), want), (M, N, K, layout, cfg, sch)
            C = sk.streamk_fp16(_t(Af), _t(B), layout=layout, plan=plan, bias=_t(bf))
            assert _rel(oracle, C, reff) <= 1e-3, (M, N, K, layout, cfg, sch)
    # bfloat16: the bias vector is bfloat16 too
    A, B = torch.randint(-1, 2, (200, 328)).bfloat16(), torch.randint(-1, 2, (1000, 328)).bfloat16()
    bias = torch.randint(-100, 100, (1000,)).bfloat16()
    want = A.double() @ B.double().T + bias.double()
    for cfg in (dict(bm=256, bn=256, bk=64), dict(bm=64, bn=64, bk=32, schedule="basic", fixup="reduce", grid=12)):
        C = sk.streamk_bf16(A.cuda(), B.cuda(), bias=bias.cuda(), **cfg)
        assert torch.equal(C.double().cpu(), want), cfg
    # Q4: general small-M, single row, matrix-vector, tiled and per-group zero points
    M, N, K = 5, 1000, 1152
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    zp = rng.integers(0, 16, (N, K // 128)).astype(np.float16)
    bias = (rng.random(N, dtype=np.float32) * 8 - 4).astype(np.float16)
    for m in (M, 1):
        A = (rng.random((m, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.q4_gemm_ref(A, Wq, sc, 128, 8) + bias.astype(np.float32)
        refz = oracle.q4_zp_gemm_ref(A, Wq, sc, zp) + bias.astype(np.float32)
        for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48), dict(schedule="sk2", fixup="atomic", grid=40)):
            for variant in ((1,) if m > 1 else (1, 2, 3)):
                C = sk.streamk_q4(_t(A), _t(Wq), _t(sc), bias=_t(bias), variant=variant, **sch)
                assert _rel(oracle, C, ref) <= 2e-3, (m, variant, sch)
            C = sk.streamk_q4(_t(A), sk.tile_q4(_t(Wq)), _t(sc), tiled=True, bias=_t(bias), **sch)
            assert _rel(oracle, C, ref) <= 2e-3, (m, "tiled", sch)
            C = sk.streamk_q4(_t(A), _t(Wq), _t(sc), zeros=_t(zp), bias=_t(bias), **sch)
            assert _rel(oracle, C, refz) <= 2e-3, (m, "zp", sch)
    X, Y = torch.zeros(8, 64, dtype=torch.float16, device="cuda"), torch.zeros(24, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        sk.streamk_fp16(X, Y, bias=torch.zeros(10, dtype=torch.float16, device="cuda"))
    with pytest.raises(ValueError):
        sk.streamk_fp16(X, Y, bias=torch.zeros(24, dtype=torch.float32, device="cuda"))
    with pytest.raises(ValueError):
        sk.streamk_fp16(X, Y, bias=torch.zeros(24, dtype=torch.float16))
    sk.workspace_status()


def test_fused_activation_epilogue(sk, oracle):
    """activation applied after the bias in fp32, before the rounding: relu on {-1,0,1} operands with an integer
    bias is exact in every kernel family and schedule (and shows that a tile shared by several CTAs is activated
    once, after its partials are summed); gelu_tanh and silu against the host functions on the fp32 product
    (1e-3 of the largest value, as for the plain product); with and without a bias; bfloat16; Q4 in all formats;
    a linear layer with its activation fused."""
    import torch
    rng = np.random.default_rng(92)
    cases = [  # (M, N, K, layout, config)
        (200, 1000, 328, "nt", dict(bm=256, bn=256, bk=64, variant=5)), (200, 1000, 328, "nt", dict(bm=128, bn=128, bk=64, variant=2)),
        (200, 1000, 328, "nt", dict(bm=128, bn=128, bk=64, variant=1)), (200, 1000, 328, "nt", dict(bm=64, bn=64, bk=32, variant=6)),
        (200, 1000, 328, "nn", dict(bm=128, bn=128, bk=64, variant=5)),
        (40, 1000, 1024, "nt", dict(bm=64, bn=64, bk=128)), (9, 1000, 1024, "nt", dict(bm=16, bn=32, bk=512)),
        (1, 1000, 1024, "nt", dict(bm=16, bn=16, bk=512, variant=3)), (1, 1000, 1024, "nt", dict(bm=16, bn=64, bk=128, variant=2)),
    ]
    for (M, N, K, layout, cfg) in cases:
        A = rng.integers(-1, 2, (M, K)).astype(np.float16)
        B = rng.integers(-1, 2, (N, K) if layout == "nt" else (K, N)).astype(np.float16)
        bias = rng.integers(-20, 20, N).astype(np.float16)
        prod = A.astype(np.float64) @ (B.T if layout == "nt" else B).astype(np.float64)
        Af = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        Bf = (B.astype(np.float32) * 0.125).astype(np.float16)  # keeps the product in the curved part of gelu / silu
        bf = (rng.random(N, dtype=np.float32) * 4 - 2).astype(np.float16)
        reff = oracle.matmul_fp32(Af, Bf, trans_b=layout == "nt")
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=12), dict(schedule="sk2", fixup="atomic", grid=10)):
            plan = sk.make_plan(M, N, K, "float16", layout, dict(cfg, **sch))
            C = sk.streamk_fp16(_t(A), _t(B), layout=layout, plan=plan, bias=_t(bias), activation="relu")
            assert np.array_equal(C.double().cpu().numpy(), np.maximum(prod + bias, 0)), (M, N, K, layout, cfg, sch)
            C = sk.streamk_fp16(_t(A), _t(B), layout=layout, plan=plan, activation="relu")
            assert np.array_equal(C.double().cpu().numpy(), np.maximum(prod, 0)), (M, N, K, layout, cfg, sch)
            for act in ("gelu_tanh", "silu"):
                C = sk.streamk_fp16(_t(Af), _t(Bf), layout=layout, plan=plan, bias=_t(bf), activation=act)
                assert _rel(oracle, C, oracle.activation_ref(reff + bf.astype(np.float32), act)) <= 1e-3, (M, N, K, layout, cfg, sch, act)
                C = sk.streamk_fp16(_t(Af), _t(Bf), layout=layout, plan=plan, activation=act)
                assert _rel(oracle, C, oracle.activation_ref(reff, act)) <= 1e-3, (M, N, K, layout, cfg, sch, act)
    # bfloat16
    A, B = torch.randint(-1, 2, (200, 328)).bfloat16(), torch.randint(-1, 2, (1000, 328)).bfloat16()
    bias = torch.randint(-20, 20, (1000,)).bfloat16()
    want = torch.relu(A.double() @ B.double().T + bias.double())
    for cfg in (dict(bm=256, bn=256, bk=64), dict(bm=64, bn=64, bk=32, schedule="basic", fixup="reduce", grid=12)):
        C = sk.streamk_bf16(A.cuda(), B.cuda(), bias=bias.cuda(), activation="relu", **cfg)
        assert torch.equal(C.double().cpu(), want), cfg
        C = sk.streamk_bf16(A.cuda(), (B * 0.125).cuda(), activation="silu", **cfg)
        ref = oracle.activation_ref((A.double() @ B.double().T * 0.125).numpy(), "silu")
        assert _rel(oracle, C, ref) <= 6e-3, cfg  # bfloat16 carries 8 bits
    # Q4: general small-M, single row, matrix-vector, tiled and per-group zero points
    M, N, K = 5, 1000, 1152
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    zp = rng.integers(0, 16, (N, K // 128)).astype(np.float16)
    bias = (rng.random(N, dtype=np.float32) * 2 - 1).astype(np.float16)
    for m in (M, 1):
        A = (rng.random((m, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        for act in ("relu", "gelu_tanh", "silu"):
            ref = oracle.activation_ref(oracle.q4_gemm_ref(A, Wq, sc, 128, 8) + bias.astype(np.float32), act)
            refz = oracle.activation_ref(oracle.q4_zp_gemm_ref(A, Wq, sc, zp), act)
            for sch in (dict(schedule="dp"), dict(schedule="sk2", fixup="reduce", grid=48)):
                for variant in ((1,) if m > 1 else (1, 2, 3)):
                    C = sk.streamk_q4(_t(A), _t(Wq), _t(sc), bias=_t(bias), activation=act, variant=variant, **sch)
                    assert _rel(oracle, C, ref) <= 2e-3, (m, variant, sch, act)
                C = sk.streamk_q4(_t(A), sk.tile_q4(_t(Wq)), _t(sc), tiled=True, bias=_t(bias), activation=act, **sch)
                assert _rel(oracle, C, ref) <= 2e-3, (m, "tiled", sch, act)
                C = sk.streamk_q4(_t(A), _t(Wq), _t(sc), zeros=_t(zp), activation=act, **sch)
                assert _rel(oracle, C, refz) <= 2e-3, (m, "zp", sch, act)
    # fp8 (both formats, raw bytes): alpha first, then bias, then the activation; exact with relu on {-1,0,1} data
    for fmt, dt, ref_fmt in (("e4m3", torch.float8_e4m3fn, "e4m3"), ("e5m2", torch.float8_e5m2, "e5m2")):
        Ai, Bi = torch.randint(-1, 2, (200, 336)).float().to(dt), torch.randint(-1, 2, (1000, 336)).float().to(dt)
        bias = torch.randint(-20, 20, (1000,)).half()
        prod = oracle.f8_gemm_ref(Ai.view(torch.uint8).numpy(), Bi.view(torch.uint8).numpy(), ref_fmt)
        Af, Bf = torch.randn(200, 336).to(dt), torch.randn(1000, 336).to(dt)
        reff = oracle.f8_gemm_ref(Af.view(torch.uint8).numpy(), Bf.view(torch.uint8).numpy(), ref_fmt)
        for cfg in (dict(bm=256, bn=256), dict(bm=128, bn=128, schedule="basic", fixup="reduce", grid=12),
                    dict(bm=128, bn=256, schedule="sk2", fixup="atomic", grid=10)):
            C = sk.streamk_fp8(Ai.cuda(), Bi.cuda(), alpha=0.5, bias=bias.cuda(), activation="relu", **cfg)
            assert np.array_equal(C.double().cpu().numpy(), np.maximum(0.5 * prod + bias.double().numpy(), 0)), (fmt, cfg)
            C = sk.streamk_fp8(Af.cuda(), Bf.cuda(), alpha=0.0625, bias=bias.cuda(), activation="silu", **cfg)
            assert _rel(oracle, C, oracle.activation_ref(0.0625 * reff + bias.float().numpy(), "silu")) <= 1e-3, (fmt, cfg)
            C = sk.streamk_fp8(Af.cuda(), Bf.cuda(), alpha=0.0625, activation="gelu_tanh", **cfg)
            assert _rel(oracle, C, oracle.activation_ref(0.0625 * reff, "gelu_tanh")) <= 1e-3, (fmt, cfg)
    # a linear layer with its activation in the epilogue, against torch's own layer + activation
    lin = torch.nn.Linear(1024, 1000, bias=True).half().cuda()
    x = torch.randn(3, 7, 1024, dtype=torch.float16, device="cuda") * 0.5
    for act, fn in (("relu", torch.relu), ("silu", torch.nn.functional.silu),
                    ("gelu_tanh", lambda v: torch.nn.functional.gelu(v, approximate="tanh"))):
        m = sk.StreamKLinear.from_linear(lin, activation=act)
        want = fn(x.float() @ lin.weight.float().T + lin.bias.float())
        assert _rel(oracle, m(x).reshape(21, 1000), want.detach().reshape(21, 1000).cpu().numpy()) <= 1e-3, act
    # the same layer in bfloat16 (weights, activations, bias and output), from one row to a prefill-sized batch
    linb = torch.nn.Linear(1024, 1000, bias=True).bfloat16().cuda()
    m = sk.StreamKLinear.from_linear(linb, weight_format="bfloat16", activation="silu")
    for rows in ((1,), (3, 7), (300,)):
        xb = (torch.randn(*rows, 1024, device="cuda") * 0.5).bfloat16()
        want = torch.nn.functional.silu(xb.float() @ linb.weight.float().T + linb.bias.float()).detach()
        got = m(xb)
        assert got.dtype == torch.bfloat16 and tuple(got.shape) == rows + (1000,)
        assert _rel(oracle, got.reshape(-1, 1000), want.reshape(-1, 1000).cpu().numpy()) <= 6e-3, rows
    with pytest.raises(ValueError):
        m(x)  # an fp16 input to the bfloat16 layer
    X, Y = torch.zeros(8, 64, dtype=torch.float16, device="cuda"), torch.zeros(24, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        sk.streamk_fp16(X, Y, activation="tanh")
    with pytest.raises(ValueError):
        sk.StreamKLinear(64, 24, activation="tanh")
    sk.workspace_status()


def test_one_byte_operands_at_full_size(sk, oracle):
    """fp8 and int8 at M = N = K = 8192 with the plans the library picks there (tuned cache or heuristic) and with
    an explicit Stream-K plan: 48 random rows against the host product (int8: equal; fp8: 1e-3), and the exact
    {-1,0,1} product checked through row and column checksums in int64 for every row and column."""
    import torch
    M = N = K = 8192
    g = torch.Generator(device="cpu").manual_seed(8)
    rows = np.random.RandomState(8).choice(M, size=48, replace=False)
    Ai = torch.randint(-1, 2, (M, K), generator=g, dtype=torch.int8)
    Bi = torch.randint(-1, 2, (N, K), generator=g, dtype=torch.int8)
    # checksums of the exact product: sum_j C[i][j] = A[i] . (sum_j B[j]),  sum_i C[i][j] = (sum_i A[i]) . B[j]
    row_sum = (Ai.long() @ Bi.long().sum(0)).numpy()
    col_sum = (Ai.long().sum(0) @ Bi.long().T).numpy()
    A8 = torch.randint(-128, 128, (M, K), generator=g, dtype=torch.int8)
    B8 = torch.randint(-128, 128, (N, K), generator=g, dtype=torch.int8)
    ref8 = torch.from_numpy(oracle.i8_gemm_ref(A8.numpy()[rows], B8.numpy()))
    Af = torch.randn(M, K, generator=g).to(torch.float8_e4m3fn)
    Bf = torch.randn(N, K, generator=g).to(torch.float8_e4m3fn)
    reff = oracle.f8_gemm_ref(Af.view(torch.uint8).numpy()[rows], Bf.view(torch.uint8).numpy())
    dAi, dBi, dA8, dB8, dAf, dBf = (t.cuda() for t in (Ai, Bi, A8, B8, Af, Bf))
    for cfg in (None, dict(bm=256, bn=256, schedule="sk2", fixup="reduce", grid=200), dict(bm=128, bn=256, schedule="basic", fixup="atomic")):
        kw = dict(config=cfg) if cfg else {}
        C = sk.streamk_int8(dA8, dB8, **kw)
        assert torch.equal(C[torch.from_numpy(rows).cuda()].cpu().long(), ref8), cfg
        C = sk.streamk_int8(dAi, dBi, **kw)
        assert np.array_equal(C.sum(1, dtype=torch.int64).cpu().numpy(), row_sum) and np.array_equal(C.sum(0, dtype=torch.int64).cpu().numpy(), col_sum), cfg
        C = sk.streamk_fp8(dAf, dBf, **kw)
        assert oracle.max_abs_rel(C[torch.from_numpy(rows).cuda()].float().cpu().numpy(), reff) <= 1e-3, cfg
        C = sk.streamk_fp8(dAi.to(torch.float16).to(torch.float8_e4m3fn), dBi.to(torch.float16).to(torch.float8_e4m3fn), **kw)
        assert np.array_equal(C.double().sum(1).cpu().numpy(), row_sum) and np.array_equal(C.double().sum(0).cpu().numpy(), col_sum), cfg
    sk.workspace_status()


@pytest.mark.parametrize("layout", ["nn", "nt"])
def test_cfg5_large_dense(sk, oracle, layout):
    """M = N = K = 8192 and the irregular 3000 x 5120 x 12288, U[-1,1), in the NN layout the large dense
    configuration names (B is [K,N], streamk.fp16.breakdown/streamk_fp16_nn.py) and in NT: a random subset
    of rows is checked against an fp64 host product; the Stream-K and data-parallel schedules of the same
    kernel must agree within tolerance."""
    import torch
    for (M, N, K) in [(8192, 8192, 8192), (3000, 5120, 12288)]:
        A, B = _uniform16((M, K), 5), _uniform16((N, K), 6)
        rows = np.sort(np.random.default_rng(7).choice(M, 96, replace=False))
        ref = A[rows].astype(np.float64) @ B.astype(np.float64).T
        if layout == "nn":
            B = np.ascontiguousarray(B.T)
        dA, dB = _t(A), _t(B)
        outs = {}
        for name, cfg in [("auto", dict()), ("sk128", dict(bm=128, bn=128, bk=64, schedule="sk2")),
                          ("dp128", dict(bm=128, bn=128, bk=64, schedule="dp")),
                          ("sk256", dict(bm=256, bn=256, bk=64, schedule="sk2", raster=8))]:
            C = sk.streamk_fp16(dA, dB, layout=layout, **cfg)
            outs[name] = C
            got = C[torch.from_numpy(rows).cuda()].float().cpu().numpy()
            assert oracle.max_abs_rel(got, ref) <= 1e-3 <= TOL, (M, name)
        scale = outs["auto"].float().abs().max().item()
        assert (outs["sk128"].float() - outs["dp128"].float()).abs().max().item() <= 2e-3 * scale
    sk.workspace_status()


@pytest.mark.parametrize("shape", [(8192, 8192, 8192), (8192, 8192, 8192, "nn"), (3000, 5120, 12288), (1024, 1024, 8192),
                                   (16, 8192, 8192)], ids=lambda s: "x".join(map(str, s)))
def test_full_size_exact_integer_checksums(sk, shape):
    """With entries in {-1, 0, 1} every product and partial sum is an integer far below 2^24 and the
    results stay below 2048, so fp32 accumulation and the fp16 store are exact: C must equal the
    integer product bit for bit, whatever the tile shape, split or summation order.  Checked at the
    full benchmark sizes through row and column checksums (C 1 = A (B^T 1), 1^T C = (1^T A) B^T) in
    int64 on the host, plus a block of rows against the full integer product."""
    import torch
    M, N, K = shape[:3]
    layout = shape[3] if len(shape) > 3 else "nt"   # "nn": B handed over as [K,N] (the large dense configuration)
    rng = np.random.default_rng(11)
    A = rng.integers(-1, 2, (M, K)).astype(np.int8)
    B = rng.integers(-1, 2, (N, K)).astype(np.int8)
    row_sum = A.astype(np.int64) @ B.astype(np.int64).sum(axis=0)
    col_sum = A.astype(np.int64).sum(axis=0) @ B.astype(np.int64).T
    rows = slice(0, min(M, 64))
    block = A[rows].astype(np.int32) @ B.astype(np.int32).T
    assert np.abs(block).max() < 2048
    dA, dB = _t(A.astype(np.float16)), _t(np.ascontiguousarray(B.T if layout == "nn" else B).astype(np.float16))
    cfgs = [dict(), dict(fixup="atomic"), dict(schedule="basic")]
    if M > 64:
        cfgs += [dict(bm=128, bn=128, bk=64, schedule="sk2", fixup="atomic"),
                 dict(bm=256, bn=256, bk=64, schedule="sk2", raster=8), dict(bm=128, bn=256, bk=64)]
    cfgs = [dict(c, layout=layout) for c in cfgs]
    for cfg in cfgs:
        C = sk.streamk_fp16(dA, dB, **cfg)
        Cd = C.double()
        assert np.array_equal(Cd.sum(dim=1).cpu().numpy().astype(np.int64), row_sum), cfg
        assert np.array_equal(Cd.sum(dim=0).cpu().numpy().astype(np.int64), col_sum), cfg
        assert np.array_equal(C[rows].cpu().numpy().astype(np.int32), block), cfg
        # linearity under an exact scaling
        assert torch.equal(sk.streamk_fp16(dA * 2, dB, **cfg), C * 2), cfg
    sk.workspace_status()


def test_full_size_one_byte_operands_exact_checksums(sk):
    """The one-byte kernels at M = N = K = 8192 (the assembly-loop instances by default): int8 over its full
    range against int64 row and column checksums and a block of rows (sums stay below 2^31); fp8 on {-1, 0, 1}
    (sums stay below 2048, exact in fp16), both formats; data-parallel and a Stream-K schedule with either fix-up."""
    import torch
    M = N = K = 8192
    rng = np.random.default_rng(13)
    A = rng.integers(-128, 128, (M, K)).astype(np.int8)
    B = rng.integers(-128, 128, (N, K)).astype(np.int8)
    row_sum = A.astype(np.int64) @ B.astype(np.int64).sum(axis=0)
    col_sum = A.astype(np.int64).sum(axis=0) @ B.astype(np.int64).T
    block = A[:32].astype(np.int64) @ B.astype(np.int64).T
    dA, dB = _t(A), _t(B)
    assert sk.kernel_name(sk.make_plan(M, N, K, "int8", "nt").kernel_id) == "tile_i8_nt_asm_256x256x128"
    for cfg in (dict(), dict(bm=256, bn=256, schedule="sk2", fixup="reduce", grid=250), dict(bm=256, bn=256, schedule="sk2", fixup="atomic", grid=250)):
        C = sk.streamk_int8(dA, dB, **cfg)
        assert np.array_equal(C.sum(dim=1, dtype=torch.int64).cpu().numpy(), row_sum), cfg
        assert np.array_equal(C.sum(dim=0, dtype=torch.int64).cpu().numpy(), col_sum), cfg
        assert np.array_equal(C[:32].cpu().numpy().astype(np.int64), block), cfg
    del dA, dB
    A = rng.integers(-1, 2, (M, K)).astype(np.int8)
    B = rng.integers(-1, 2, (N, K)).astype(np.int8)
    row_sum = A.astype(np.int64) @ B.astype(np.int64).sum(axis=0)
    col_sum = A.astype(np.int64).sum(axis=0) @ B.astype(np.int64).T
    block = A[:32].astype(np.int32) @ B.astype(np.int32).T
    assert np.abs(block).max() < 2048
    for fmt, name in ((torch.float8_e4m3fn, "float8_e4m3"), (torch.float8_e5m2, "float8_e5m2")):
        dA, dB = _t(A.astype(np.float32)).to(fmt), _t(B.astype(np.float32)).to(fmt)
        assert "asm" in sk.kernel_name(sk.make_plan(M, N, K, name, "nt").kernel_id)
        for cfg in (dict(), dict(bm=256, bn=256, schedule="sk2", fixup="reduce", grid=250)):
            C = sk.streamk_fp8(dA, dB, **cfg)
            Cd = C.double()
            assert np.array_equal(Cd.sum(dim=1).cpu().numpy().astype(np.int64), row_sum), (name, cfg)
            assert np.array_equal(Cd.sum(dim=0).cpu().numpy().astype(np.int64), col_sum), (name, cfg)
            assert np.array_equal(C[:32].cpu().numpy().astype(np.int32), block), (name, cfg)
    sk.workspace_status()


# (256 x 256 exists with 16x16x32 MFMAs only)
@pytest.mark.parametrize("cfg,variant", [(dict(bm=bm, bn=bn), v) for (bm, bn) in ((256, 256), (128, 128), (128, 256), (256, 128))
                                         for v in (2, 5) if not ((bm, bn) == (256, 256) and v == 2)],
                         ids=lambda x: f"{x['bm']}x{x['bn']}" if isinstance(x, dict) else {2: "mfma32", 5: "mfma16"}[x])
def test_nn_layout(sk, oracle, cfg, variant):
    """B given as [K,N] (the layout of the reference's fp32 script and of the large dense
    configuration), both MFMA forms: ragged shapes against the oracle, all schedules; then exact
    integer data at 3000 x 5120 x 12288."""
    cfg = dict(cfg, variant=variant)
    rng = np.random.default_rng(21)
    for (M, N, K) in [(200, 136, 328), (1000, 1096, 4104), (520, 264, 64)]:
        A = (rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16)
        B = (rng.random((K, N), dtype=np.float32) * 2 - 1).astype(np.float16)
        ref = oracle.matmul_fp32(A, B)
        for sch in (dict(schedule="dp"), dict(schedule="basic", fixup="reduce", grid=24),
                    dict(schedule="sk2", fixup="atomic", grid=16)):
            C = sk.streamk_fp16(_t(A), _t(B), layout="nn", bk=64, **cfg, **sch)
            assert _rel(oracle, C, ref) <= 2e-3 <= TOL, (M, N, K, sch)
    M, N, K = 3000, 5120, 12288
    A = rng.integers(-1, 2, (M, K)).astype(np.int8)
    B = rng.integers(-1, 2, (K, N)).astype(np.int8)
    row_sum = A.astype(np.int64) @ B.astype(np.int64).sum(axis=1)
    col_sum = A.astype(np.int64).sum(axis=0) @ B.astype(np.int64)
    C = sk.streamk_fp16(_t(A.astype(np.float16)), _t(B.astype(np.float16)), layout="nn", bk=64, **cfg).double()
    assert np.array_equal(C.sum(dim=1).cpu().numpy().astype(np.int64), row_sum)
    assert np.array_equal(C.sum(dim=0).cpu().numpy().astype(np.int64), col_sum)
    sk.workspace_status()


@pytest.mark.parametrize("fixup", ["atomic", "reduce"])
def test_fp32_cfg1_and_fixture(sk, oracle, golden_dir, fixup):
    """fp32 Stream-K GEMM: the 256 x 256 x 1024 U[-1,1) seed-0 problem of the CPU configuration
    (there simulated with 64x64x16 tiles on 4 CTAs) on the GPU's 128x128x16 fp32-MFMA tiles, split
    over 3 / 5 / 7 CTAs, against the oracle's CPU Stream-K run and numpy; plus the committed
    48 x 40 x 72 fixture, the [N,K] layout and exact integer data."""
    rng = np.random.default_rng(0)
    A = rng.random((256, 1024), dtype=np.float32) * 2 - 1
    B = rng.random((1024, 256), dtype=np.float32) * 2 - 1
    ref_sim = oracle.streamk_gemm_f32(A, B, 64, 64, 16, 4, fixup=fixup)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    for grid in (3, 5, 7, 4):
        C = sk.streamk_fp32(_t(A), _t(B), schedule="basic", fixup=fixup, grid=grid).cpu().numpy()
        assert oracle.max_abs_rel(C, ref) <= 1e-5
        assert oracle.max_abs_rel(C, ref_sim) <= 1e-5
    g = np.load(os.path.join(golden_dir, "streamk_f32_48x40x72.npz"))
    C = sk.streamk_fp32(_t(g["A"]), _t(g["B"]), schedule="basic", fixup=fixup, grid=2).cpu().numpy()
    assert oracle.max_abs_rel(C, g["C_reduce"]) <= 1e-5
    # [N,K] layout and ragged shapes
    A2 = rng.random((300, 520), dtype=np.float32) * 2 - 1
    B2 = rng.random((200, 520), dtype=np.float32) * 2 - 1
    C = sk.streamk_fp32(_t(A2), _t(B2), layout="nt", schedule="sk2", fixup=fixup, grid=5).cpu().numpy()
    assert oracle.max_abs_rel(C, A2.astype(np.float64) @ B2.astype(np.float64).T) <= 1e-5
    # exact: integer entries keep every fp32 partial sum exact
    Ai = rng.integers(-4, 5, (260, 1032)).astype(np.float32)
    Bi = rng.integers(-4, 5, (1032, 388)).astype(np.float32)
    C = sk.streamk_fp32(_t(Ai), _t(Bi), schedule="basic", fixup=fixup, grid=9).cpu().numpy()
    assert np.array_equal(C, Ai @ Bi)
    # the 32 x 256 tile (the plan for M <= 32) and the 128 x 128 one on the same ragged problems, both layouts
    for (M, N, K) in [(16, 1000, 1032), (40, 388, 260), (1, 264, 72), (260, 520, 1032)]:
        Ai = rng.integers(-4, 5, (M, K)).astype(np.float32)
        Bi = rng.integers(-4, 5, (K, N)).astype(np.float32)
        Ar = rng.random((M, K), dtype=np.float32) * 2 - 1
        for (bm, bn) in ((32, 256), (128, 128)):
            for sch in (dict(schedule="dp"), dict(schedule="basic", fixup=fixup, grid=7), dict(schedule="sk2", fixup=fixup, grid=3)):
                C = sk.streamk_fp32(_t(Ai), _t(Bi), bm=bm, bn=bn, **sch).cpu().numpy()
                assert np.array_equal(C, Ai @ Bi), (M, N, K, bm, bn, sch)
                C = sk.streamk_fp32(_t(Ai), _t(np.ascontiguousarray(Bi.T)), layout="nt", bm=bm, bn=bn, **sch).cpu().numpy()
                assert np.array_equal(C, Ai @ Bi), (M, N, K, bm, bn, sch, "nt")
                C = sk.streamk_fp32(_t(Ar), _t(Bi), bm=bm, bn=bn, **sch).cpu().numpy()
                assert oracle.max_abs_rel(C, Ar.astype(np.float64) @ Bi.astype(np.float64)) <= 1e-5
    sk.workspace_status()


def test_fp32_reference_shape(sk, oracle):
    """The shape the reference's fp32 script runs (16 x 16384 x 8192, streamk_fp32.py:15), B as
    [K,N]: checked against an fp64 host product on a slice of columns."""
    rng = np.random.default_rng(3)
    A = rng.random((16, 8192), dtype=np.float32) * 2 - 1
    B = rng.random((8192, 16384), dtype=np.float32) * 2 - 1
    plan = sk.make_plan(16, 16384, 8192, "float32", "nn")
    assert (plan.bm, plan.bn) == (32, 256)
    C = sk.streamk_fp32(_t(A), _t(B), plan=plan).cpu().numpy()
    cols = slice(4000, 4512)
    ref = A.astype(np.float64) @ B[:, cols].astype(np.float64)
    assert oracle.max_abs_rel(C[:, cols], ref) <= 1e-5
    C = sk.streamk_fp32(_t(A), _t(B), bm=128, bn=128).cpu().numpy()
    assert oracle.max_abs_rel(C[:, cols], ref) <= 1e-5
    sk.workspace_status()


def test_reference_run_shapes(sk, oracle):
    """The shapes the reference's own scripts run: fp16 NT 16 x 16384 x 8192 (streamk.fp16.breakdown/
    streamk_fp16_nt.py:15, streamk_fp16_block_reduce.py:66) and Q4 16 x 16384 x 16384 (streamk_fp16_ladder_block_reduce_q4
    .py:73), with the tuned plan, the untuned default and the schedules the reference uses there (Stream-K over every
    tile, both fix-ups).  fp16: against the fp32 host product of the same fp16 inputs; Q4: against the host product with
    the dequantised weights on a slice of 1024 weight rows (the full host product takes a minute), and the standalone
    dequant of all rows bit for bit."""
    rng = np.random.default_rng(16384)
    M, N, K = 16, 16384, 8192
    A, B = _uniform16((M, K), 31), _uniform16((N, K), 32)
    ref = oracle.matmul_fp32(A, B, trans_b=True)
    dA, dB = _t(A), _t(B)
    tuned, untuned = sk.make_plan(M, N, K, "float16", "nt"), sk.make_plan(M, N, K, "float16", "nt", use_tuned=False)
    for cfg in (dict(plan=tuned), dict(plan=untuned), dict(bm=16, bn=16, bk=512, schedule="dp"),
                dict(schedule="basic", fixup="reduce"), dict(schedule="basic", fixup="atomic"),
                dict(bm=16, bn=64, bk=128, schedule="sk2", grid=512, fixup="reduce")):
        C = sk.streamk_fp16(dA, dB, **cfg)
        assert _rel(oracle, C, ref) <= 2e-3 <= TOL, cfg
    del dB
    N, K = 16384, 16384
    A = rng.standard_normal((M, K), dtype=np.float32).astype(np.float16)
    Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
    sc = rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16)
    rows = slice(9000, 10024)
    ref = oracle.q4_gemm_ref(A, Wq[rows], sc[rows], 128, 8)
    dA, dW, dS = _t(A), _t(Wq), _t(sc)
    W = sk.dequant_q4(dW[rows], dS[rows]).cpu().numpy()
    assert np.array_equal(W.view(np.uint16), oracle.dequant_q4(Wq[rows], sc[rows], 128, 8).view(np.uint16))
    first = None
    for cfg in (dict(), dict(plan=sk.make_plan(M, N, K, "q4", "nt", use_tuned=False)), dict(schedule="dp"),
                dict(fixup="reduce", schedule="basic", grid=256),
                dict(fixup="atomic", schedule="basic", grid=256), dict(bm=16, bn=64, bk=512, schedule="dp")):
        C = sk.streamk_q4(dA, dW, dS, **cfg)
        assert _rel(oracle, C[:, rows], ref) <= 2e-3 <= TOL, cfg
        # every plan multiplies the same decoded weights: outside the checked slice the results agree with each other
        if first is None:
            first = C.float()
        else:
            assert float((C.float() - first).abs().max()) <= 2e-3 * float(first.abs().max()), cfg
    sk.workspace_status()


def test_linear_layers_replay_in_a_graph(sk):
    """A decode step as a serving loop would capture it: three StreamKLinear layers (fp16, Q4 with bias, Q4 with
    per-group zero points and bias) for a batch of 4 rows in one graph, replayed several times with new inputs
    copied into the static input buffer and eager work in between; every replay must equal the eager result of
    the same layers on the same input bit for bit (all three use the ordered reduce or no fix-up)."""
    import torch
    torch.manual_seed(21)
    K, H = 1024, 1536
    l1 = sk.StreamKLinear.from_linear(torch.nn.Linear(K, H, bias=False).cuda().half())
    l2 = sk.StreamKLinear.from_linear(torch.nn.Linear(H, K, bias=True).cuda().half(), weight_format="q4")
    l3 = sk.StreamKLinear.from_linear(torch.nn.Linear(K, H, bias=True).cuda().half(), weight_format="q4_zp")
    x = torch.zeros(4, K, dtype=torch.float16, device="cuda")
    step = lambda t: l3(l2(l1(t)))
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        for _ in range(2):
            step(x)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            y = step(x)
    for replay in range(4):
        xin = torch.randn(4, K, device="cuda").half()
        want = step(xin)                       # eager, default stream
        torch.cuda.synchronize()
        x.copy_(xin)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), replay
    sk.workspace_status()


def test_graph_capture_replays_match_eager(sk, oracle):
    """The launches are capturable (no host synchronisation, no allocation; the workspace is cleared
    by a fill kernel, not by a memset node): a captured sequence reduce fix-up -> atomic fix-up ->
    Q4 matrix-vector is replayed several times, with eager launches and synchronisations in
    between, and every replay must reproduce the eager results bit for bit (reduce, Q4) or within
    tolerance (atomic: summation order varies)."""
    import torch
    rng = np.random.default_rng(77)
    M, N, K = 512, 1024, 2048
    A = _t((rng.random((M, K), dtype=np.float32) * 2 - 1).astype(np.float16))
    B = _t((rng.random((N, K), dtype=np.float32) * 2 - 1).astype(np.float16))
    a1 = _t((rng.random((1, K), dtype=np.float32) * 2 - 1).astype(np.float16))
    Wq = _t(rng.integers(0, 256, (N, K // 2), dtype=np.uint8))
    sc = _t(rng.uniform(0.005, 0.02, (N, K // 128)).astype(np.float16))
    red = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=40)
    atm = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="atomic", grid=40)
    eager_red = sk.streamk_fp16(A, B, **red)
    eager_q4 = sk.streamk_q4(a1, Wq, sc, schedule="sk2", grid=48, fixup="reduce")
    ref = oracle.matmul_fp32(A.cpu().numpy(), B.cpu().numpy(), trans_b=True)
    side = torch.cuda.Stream()
    c_red = torch.empty(M, N, dtype=torch.float16, device="cuda")
    c_atm = torch.empty(M, N, dtype=torch.float16, device="cuda")
    c_q4 = torch.empty(1, N, dtype=torch.float16, device="cuda")
    with torch.cuda.stream(side):
        p_red = sk.make_plan(M, N, K, "float16", "nt", red)
        p_atm = sk.make_plan(M, N, K, "float16", "nt", atm)
        p_q4 = sk.make_plan(1, N, K, "q4", "nt", dict(schedule="sk2", grid=48, fixup="reduce"))
        for _ in range(2):  # warm up on the capture stream: its workspace is created and initialised here
            sk.streamk_fp16(A, B, out=c_red, plan=p_red)
            sk.streamk_fp16(A, B, out=c_atm, plan=p_atm)
            sk.streamk_q4(a1, Wq, sc, out=c_q4, plan=p_q4)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            sk.streamk_fp16(A, B, out=c_red, plan=p_red)
            sk.streamk_fp16(A, B, out=c_atm, plan=p_atm)
            sk.streamk_q4(a1, Wq, sc, out=c_q4, plan=p_q4)
    for replay in range(4):
        c_red.zero_(); c_atm.zero_(); c_q4.zero_()
        sk.streamk_fp16(A, B, **atm)  # eager work on the default stream between the replays
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(c_red, eager_red), replay
        assert torch.equal(c_q4, eager_q4), replay
        assert _rel(oracle, c_atm, ref) <= 2e-3 <= TOL, replay
    sk.workspace_status()


def test_one_workspace_serves_graph_and_eager_launches_of_both_fixups(sk, oracle):
    """Whether the partial area needs zeroing before an atomic launch is recorded in the workspace, not
    on the host: an atomic launch captured while the workspace was clean must still be right when an
    eager reduce launch on the SAME stream and workspace has left partial tiles behind before the
    replay (and the other way round).  Integer data: the result is exact whatever the order."""
    import torch
    rng = np.random.default_rng(78)
    M, N, K = 512, 1024, 2048
    A = rng.integers(-1, 2, (M, K)).astype(np.float16)
    B = rng.integers(-1, 2, (N, K)).astype(np.float16)
    want = torch.from_numpy((A.astype(np.int32) @ B.astype(np.int32).T).astype(np.float16)).cuda()
    dA, dB = _t(A), _t(B)
    red = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=40)
    atm = dict(bm=128, bn=128, bk=64, schedule="basic", fixup="atomic", grid=40)
    c_atm = torch.empty(M, N, dtype=torch.float16, device="cuda")
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        p_red = sk.make_plan(M, N, K, "float16", "nt", red)
        p_atm = sk.make_plan(M, N, K, "float16", "nt", atm)
        sk.streamk_fp16(dA, dB, out=c_atm, plan=p_atm)   # creates this stream's workspace; leaves it clean
        torch.cuda.synchronize()
        assert torch.equal(c_atm, want)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            sk.streamk_fp16(dA, dB, out=c_atm, plan=p_atm)
        for replay in range(3):
            c_atm.zero_()
            got = sk.streamk_fp16(dA, dB, plan=p_red)    # eager, same stream, same workspace: dirties the partials
            torch.cuda.synchronize()
            assert torch.equal(got, want), replay
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(c_atm, want), replay
            graph.replay()                               # and twice in a row
            torch.cuda.synchronize()
            assert torch.equal(c_atm, want), replay
        # eager atomic after eager reduce, larger tiles than before (other slot sizes)
        for cfg in (dict(bm=256, bn=256, bk=64, schedule="basic", fixup="reduce", grid=16),
                    dict(bm=256, bn=256, bk=64, schedule="basic", fixup="atomic", grid=16),
                    dict(bm=128, bn=128, bk=64, schedule="basic", fixup="atomic", grid=24)):
            assert torch.equal(sk.streamk_fp16(dA, dB, **cfg), want), cfg
    torch.cuda.synchronize()
    sk.workspace_status()


def test_strided_operands_and_out(sk, oracle):
    """Leading dimensions larger than the rows, and writing into a caller-provided C."""
    import torch
    A_full, B_full = _t(_uniform16((300, 1024), 8)), _t(_uniform16((520, 1024), 9))
    A, B = A_full[:, :512], B_full[:, 256:768]
    out_full = torch.zeros(300, 1040, dtype=torch.float16, device="cuda")
    out = out_full[:, 8:528]
    sk.streamk_fp16(A, B, out=out, bm=128, bn=128, bk=64, schedule="basic", grid=40)
    ref = oracle.matmul_fp32(A.cpu().numpy(), B.cpu().numpy(), trans_b=True)
    assert _rel(oracle, out, ref) <= 2e-3
    assert out_full[:, :8].abs().max().item() == 0 and out_full[:, 528:].abs().max().item() == 0


def test_wait_gives_up_instead_of_hanging(sk):
    """A fix-up wait that runs out of polls must end the kernel and report SK_ERR_TIMEOUT; the
    condition is forced from the host with a poll limit of 1 on a schedule where the followers
    cannot have finished yet."""
    A, B = _t(_uniform16((1024, 8192), 10)), _t(_uniform16((1024, 8192), 11))
    sk.streamk_fp16(A, B, bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=256, spin_limit=1)
    with pytest.raises(sk.StreamKError) as e:
        sk.workspace_status()
    assert e.value.status == -8
    # flags of the abandoned wait may still be raised: the workspace is refused until it is initialised again
    with pytest.raises(sk.StreamKError) as e:
        sk.streamk_fp16(A, B, bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=256)
    assert e.value.status == -8
    sk.reset_workspaces()
    # and the library is usable again afterwards
    C = sk.streamk_fp16(A, B, bm=128, bn=128, bk=64, schedule="basic", fixup="reduce", grid=256)
    C2 = sk.streamk_fp16(A, B, bm=128, bn=128, bk=64, schedule="dp")
    sk.workspace_status()
    assert (C.float() - C2.float()).abs().max().item() <= 2e-3 * C2.float().abs().max().item()


def test_extreme_aspect_ratios(sk, oracle):
    """Very long and very wide problems: tile bases are 64-bit, offsets inside a tile 32-bit.  Rows
    and columns sampled from both ends are checked against the fp32 host product; exact {-1,0,1}
    data gives bit-exact row and column checksums over the whole result."""
    import torch
    rng = np.random.default_rng(33)
    for (M, N, K) in [(300000, 136, 64), (24, 1000000, 128), (1, 2000000, 64), (70000, 70000, 8)]:
        A = rng.integers(-1, 2, (M, K)).astype(np.float16)
        B = rng.integers(-1, 2, (N, K)).astype(np.float16)
        dA, dB = _t(A), _t(B)
        C = sk.streamk_fp16(dA, dB)
        rows = np.unique(np.concatenate([np.arange(min(M, 40)), np.arange(max(M - 40, 0), M)]))
        cols = np.unique(np.concatenate([np.arange(min(N, 40)), np.arange(max(N - 40, 0), N)]))
        got_r = C[torch.from_numpy(rows).cuda()].cpu().numpy().astype(np.int32)
        assert np.array_equal(got_r, (A[rows].astype(np.int32) @ B.astype(np.int32).T))
        got_c = C[:, torch.from_numpy(cols).cuda()].cpu().numpy().astype(np.int32)
        assert np.array_equal(got_c, (A.astype(np.int32) @ B[cols].astype(np.int32).T))
        # whole-result checksums: sum_j C[i][j] = A[i] . sum_j B[j]
        Cd = C.double()
        assert np.array_equal(Cd.sum(dim=1).cpu().numpy().astype(np.int64), A.astype(np.int64) @ B.astype(np.int64).sum(axis=0))
        assert np.array_equal(Cd.sum(dim=0).cpu().numpy().astype(np.int64), B.astype(np.int64) @ A.astype(np.int64).sum(axis=0))
        del C, Cd, dA, dB
    sk.workspace_status()


def test_bad_calls_are_refused(sk):
    import torch
    A = torch.zeros(64, 128, dtype=torch.float16, device="cuda")
    with pytest.raises(TypeError):
        sk.streamk_fp16(A.float(), A)
    with pytest.raises(ValueError):
        sk.streamk_fp16(A, torch.zeros(64, 136, dtype=torch.float16, device="cuda"))
    with pytest.raises(sk.StreamKError):
        sk.streamk_fp16(A[:, :100], A[:, :100])  # K = 100 is not a multiple of 8
    # an `out` of the wrong shape is refused on the host by every wrapper (the kernel would write past it)
    A32 = torch.zeros(64, 128, dtype=torch.float32, device="cuda")
    with pytest.raises(ValueError):
        sk.streamk_fp32(A32, A32, layout="nt", out=torch.zeros(32, 64, dtype=torch.float32, device="cuda"))
    with pytest.raises(ValueError):
        sk.streamk_fp16(A, A, out=torch.zeros(32, 64, dtype=torch.float16, device="cuda"))


def test_autotune_search_and_cache(sk, oracle, tmp_path):
    """The per-shape search (autotune/streamk_fp16_autotune.py:376-386 in the reference): every dtype it covers on a
    small problem with a short candidate list -- the winner is one of the candidates, candidates agree with each
    other (the tuner checks them), an impossible candidate is skipped, and the result lands in the cache file under
    the key plans are looked up by."""
    import json
    import sys
    at = sys.modules["streamk.autotune"]
    cache = str(tmp_path / "tuned.json")
    cases = [
        ("float16", 200, 512, 1024, [dict(bm=128, bn=128, bk=64, schedule="dp"), dict(bm=64, bn=64, bk=32, schedule="sk2", fixup="reduce"),
                                     dict(bm=48, bn=48, bk=64, schedule="dp")]),
        ("bfloat16", 200, 512, 1024, [dict(bm=128, bn=128, bk=64, schedule="dp"), dict(bm=64, bn=64, bk=32, schedule="basic", fixup="atomic")]),
        ("bfloat16", 8, 512, 1024, None),
        ("float16", 1, 512, 1024, None),
        ("q4", 4, 512, 1024, None),
        ("float8_e4m3", 200, 512, 1024, [dict(bm=128, bn=128, schedule="dp"), dict(bm=128, bn=128, schedule="sk2", fixup="reduce")]),
        ("int8", 200, 512, 1024, [dict(bm=128, bn=128, schedule="dp"), dict(bm=256, bn=128, schedule="basic", fixup="atomic")]),
    ]
    for dtype, M, N, K, configs in cases:
        ms, cfg, ref = at.autotune(M, N, K, dtype, "nt", configs=configs, warmup=2, rep=5, cache_path=cache)
        assert ms > 0 and cfg in (configs if configs is not None else at.candidate_configs(M, N, K, dtype)), (dtype, cfg)
        assert cfg.get("bm") != 48
        hit = json.load(open(cache))[f"gfx950/{dtype}/nt/{M}x{N}x{K}"]
        assert hit["config"] == cfg and hit["latency_ms"] == ms
        plan = sk.make_plan(M, N, K, dtype, "nt", cfg)   # the recorded configuration makes a plan again
        assert plan.bm == cfg["bm"] and plan.bn == cfg["bn"]
    with pytest.raises(RuntimeError):
        at.autotune(200, 512, 1024, "float16", "nt", configs=[dict(bm=48, bn=48, bk=64)], cache=False)
    sk.workspace_status()

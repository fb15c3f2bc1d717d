"""CPU-side checks of the shipped library: it loads, exports what include/streamk.h declares, its
partitioner agrees with the oracle's restatement of the reference, and bad calls are refused with
error codes (no compute entry point is launched here)."""
import ctypes
import os
import re
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def sk():
    import streamk
    streamk.lib()
    return streamk


def test_exports_every_declared_symbol(sk):
    header = open(os.path.join(ROOT, "include", "streamk.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    names = set(re.findall(r"\b(sk_[a-z0-9_]+)\s*\(", header))
    assert {"sk_make_plan", "sk_gemm_f16", "sk_gemm_f32", "sk_gemm_q4", "sk_dequant_q4",
            "sk_workspace_init", "sk_workspace_bytes", "sk_strerror", "sk_version"} <= names
    L = sk.lib()
    for n in sorted(names):
        assert hasattr(L, n), f"{n} is declared in streamk.h but not exported"
    assert L.sk_version() == 100
    assert L.sk_selfcheck() == 0        # kernel ids are unique, every instance is named
    assert sk.strerror(0) == "ok" and "workspace" in sk.strerror(-5)


@pytest.mark.parametrize("shape,tile,P", [
    ((1024, 1024, 8192), (128, 128, 64), 256),
    ((3000, 5120, 12288), (128, 128, 64), 256),
    ((8192, 8192, 8192), (256, 256, 64), 256),
    ((256, 4096, 4096), (128, 128, 64), 200),
    ((300, 700, 1000), (64, 64, 64), 24),
])
def test_plan_matches_oracle(sk, oracle, shape, tile, P):
    """Two-tile hybrid schedule == the reference's partition (streamk_fp32.py:33-54) as the oracle
    restates it, for the product's own tile shapes."""
    M, N, K = shape
    plan = sk.make_plan(M, N, K, "float16", "nt", cus=256, bm=tile[0], bn=tile[1], bk=tile[2],
                        grid=P, schedule="sk2", raster=1)
    assert sk.make_plan(M, N, K, "float16", "nt", cus=256, bm=tile[0], bn=tile[1], bk=tile[2]).raster == 8  # default
    ref = oracle.partition(M, N, K, *tile, P)
    for k in ("num_block_m", "num_block_n", "iters_per_tile", "total_tiles", "streamk_tiles",
              "blocking_tiles", "streamk_iters", "streamk_full_tiles", "streamk_partial_tiles"):
        assert getattr(plan, k) == ref[k], k
    assert plan.dp_waves == ref["sm_partition_factor"]
    for pid in (0, 1, P // 2, P - 1):
        assert sk.cta_range(plan, pid) == oracle.cta_range(ref, pid)
    nbn = ref["num_block_n"]
    for t in (0, 1, nbn, ref["total_tiles"] - 1):
        assert sk.tile_coords(plan, t) == (t // nbn, t % nbn)  # streamk_fp32.py:106-107


def test_schedules(sk):
    kw = dict(cus=256, bm=128, bn=128, bk=64, grid=256)
    dp = sk.make_plan(1024, 8192, 8192, "float16", "nt", schedule="dp", **kw)
    assert (dp.streamk_tiles, dp.blocking_tiles, dp.dp_waves, dp.workspace_bytes) == (0, 512, 2, 0)
    basic = sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="basic", **kw)
    assert (basic.streamk_tiles, basic.blocking_tiles) == (64, 0)
    one = sk.make_plan(3000, 5120, 12288, "float16", "nt", schedule="sk1", **kw)
    assert (one.total_tiles, one.streamk_tiles, one.blocking_tiles) == (960, 192, 768)
    f32 = sk.make_plan(16, 16384, 8192, "float32", "nn", cus=256)
    assert (f32.bm, f32.bn, f32.bk, f32.kernel_id) == (32, 256, 16, 202)  # M <= 32: the 32-row tile
    f32 = sk.make_plan(256, 256, 1024, "float32", "nn", cus=256)
    assert (f32.bm, f32.bn, f32.bk, f32.kernel_id) == (128, 128, 16, 200)
    auto = sk.make_plan(8192, 8192, 8192, "float16", "nt", cus=256)
    assert (auto.bm, auto.bn, auto.schedule, auto.streamk_tiles) == (256, 256, 1, 0)


def test_fixed_split_k_schedule(sk):
    """Every tile is cut into `split` equal K ranges, CTA g owning range g % split of tile g // split:
    the grid of thread_level_gemm_with_macro_ladder_atomic_reduce.py:129-131 flattened, K range of
    :153-154."""
    kw = dict(cus=256, bm=128, bn=128, bk=64)
    p = sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="splitk", split=4, **kw)
    assert (p.grid, p.streamk_tiles, p.blocking_tiles, p.iters_per_tile) == (256, 64, 0, 128)
    for g in range(p.grid):
        tile, part = divmod(g, 4)
        assert sk.cta_range(p, g) == (tile * 128 + part * 32, tile * 128 + (part + 1) * 32)
    # split 0: the largest factor of 128 that keeps 64 * split CTAs resident (2 per CU here)
    p = sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="splitk", **kw)
    assert p.grid == 64 * 8 and sk.cta_range(p, 9) == (128 + 16, 128 + 32)
    # split 1 is the data-parallel schedule; a factor that does not divide the K-iterations, or a
    # grid beyond what stays resident, is refused
    p = sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="splitk", split=1, **kw)
    assert (p.grid, p.streamk_tiles, p.workspace_bytes) == (64, 0, 0)
    for bad in (3, 16):
        with pytest.raises(sk.StreamKError):
            sk.make_plan(1024, 1024, 8192, "float16", "nt", schedule="splitk", split=bad, **kw)


def test_fp8_plans(sk):
    """fp8 / int8 plans: tile kernels from 65 rows, weight-streaming kernels up to 64 rows; bk counts one-byte
    elements; NT only."""
    for (M, bm, name) in [(1, 16, "mb1_wn4_rk1_row1_1"), (16, 16, "mb1_wn4_rk1_row1_0"), (32, 32, "mb2_wn4_rk1_row1_0"),
                          (64, 64, "mb4_wn4_rk1_row1_0")]:
        for dtype, tag in (("float8_e4m3", "f8e4m3"), ("float8_e5m2", "f8e5m2")):
            p = sk.make_plan(M, 4096, 4096, dtype, "nt", cus=256)
            assert (p.bm, p.bn, p.bk) == (bm, 64, 256) and p.iters_per_tile == 4096 // 256
            assert sk.kernel_name(p.kernel_id) == f"skinny_{tag}_{name}"
        q = sk.make_plan(M, 4096, 4096, "int8", "nt", cus=256)
        assert (q.bm, q.bn, q.bk) == (bm, 64, 256) and sk.kernel_name(q.kernel_id) == f"skinny_i8_{name}"
    for (M, N, K, bm, bn) in [(8192, 8192, 8192, 256, 256), (512, 512, 4096, 128, 128), (65, 4096, 4096, 64, 128), (300, 4096, 4096, 128, 256)]:
        p = sk.make_plan(M, N, K, "float8_e4m3", "nt", cus=256, bm=bm, bn=bn)
        assert (p.bm, p.bn, p.bk) == (bm, bn, 128) and p.iters_per_tile == K // 128
        # (256 x 256 with K a multiple of 128: the four-wave kernels whose K loop is assembly)
        assert sk.kernel_name(p.kernel_id) == ("tile_f8e4m3_nt_asm_256x256x128" if bm == 256 else f"tile_f8e4m3_nt_dma_{bm}x{bn}x128")
        r = sk.make_plan(M, N, K, "float8_e5m2", "nt", cus=256, bm=bm, bn=bn)
        assert (r.bm, r.bn, r.bk, r.grid) == (p.bm, p.bn, 128, p.grid)
        assert sk.kernel_name(r.kernel_id) == ("tile_f8e5m2_nt_asm_256x256x128" if bm == 256 else f"tile_f8e5m2_nt_dma_{bm}x{bn}x128")
        q = sk.make_plan(M, N, K, "int8", "nt", cus=256, bm=bm, bn=bn)
        assert (q.bm, q.bn, q.bk) == (p.bm, p.bn, 128)
        assert sk.kernel_name(q.kernel_id) == ("tile_i8_nt_asm_256x256x128" if bm == 256 else f"tile_i8_nt_dma16_{bm}x{bn}x128")
    # the planner's own choice: the assembly-loop kernel where 256 x 256 tiles fill the device, 64 x 128 tiles for few
    # rows (the four-stage kernels, 64 K-values per stage)
    for dtype, tag in (("float8_e4m3", "f8e4m3_nt_dma_64x128x64"), ("float8_e5m2", "f8e5m2_nt_dma_64x128x64"), ("int8", "i8_nt_dma16_64x128x64")):
        assert sk.kernel_name(sk.make_plan(8192, 8192, 8192, dtype, "nt", cus=256, use_tuned=False).kernel_id).endswith("_nt_asm_256x256x128")
        assert sk.kernel_name(sk.make_plan(65, 4096, 4096, dtype, "nt", cus=256, use_tuned=False).kernel_id) == f"tile_{tag}"
    with pytest.raises(sk.StreamKError):
        sk.make_plan(256, 256, 256, "int8", "nn", cus=256)
    with pytest.raises(sk.StreamKError):
        sk.make_plan(256, 256, 256, "float8_e4m3", "nn", cus=256)
    with pytest.raises(sk.StreamKError):
        sk.make_plan(256, 256, 264, "float8_e4m3", "nt", cus=256)   # K not a multiple of 16


def test_raster_is_a_permutation(sk):
    plan = sk.make_plan(3000, 5120, 4096, "float16", "nt", cus=256, bm=128, bn=128, bk=64, raster=8)
    seen = {sk.tile_coords(plan, t) for t in range(plan.total_tiles)}
    assert len(seen) == plan.total_tiles == plan.num_block_m * plan.num_block_n
    # walks 8 tile rows down before stepping to the next column (triton_impl.py:14-28)
    assert [sk.tile_coords(plan, t) for t in range(3)] == [(0, 0), (1, 0), (2, 0)]
    assert sk.tile_coords(plan, 8) == (0, 1)


def test_untuned_plans_keep_cta_ranges_aligned(sk):
    """With tile, schedule and grid left to the planner, a tile kernel never gets CTA ranges that start anywhere in
    their tiles and in raster order: the plan is data-parallel, a fixed split of K in two or four, a Stream-K
    schedule whose ranges start at the beginning or in the middle of a tile or close to each other, or (one CTA per
    CU only) a Stream-K schedule in the interleaved tile order with at least eight CTAs at every offset; and a
    Stream-K tile never has more than four contributors."""
    import math
    SPLITK, DP = sk._lib.SCHEDULES["splitk"], sk._lib.SCHEDULES["dp"]
    seen, streamk_seen = set(), set()
    for dtype, layout in (("float16", "nt"), ("float16", "nn"), ("bfloat16", "nt"), ("float8_e4m3", "nt"), ("int8", "nt"), ("q4", "nt")):
        for (N, K) in ((4096, 4096), (8192, 8192), (11008, 4096), (4096, 11008 if dtype != "q4" else 11008 + 128 - 11008 % 128), (5120, 5120), (6144, 4096)):
            for M in (65, 128, 200, 384, 768, 1000, 1536, 2048, 2560, 3000, 3584, 4096, 8192):
                if dtype in ("float8_e4m3", "int8") and K % 16:
                    continue
                plan = sk.make_plan(M, N, K, dtype, layout, cus=256, use_tuned=False)
                name = sk.kernel_name(plan.kernel_id)
                if not name.startswith("tile_"):
                    continue
                seen.add(plan.schedule)
                if plan.streamk_tiles == 0:
                    continue
                per_cta, ipt = plan.streamk_iters / plan.grid, plan.iters_per_tile
                if plan.schedule == SPLITK:
                    assert ipt / per_cta in (2, 4) and plan.streamk_partial_tiles == 0, (dtype, M, N, K, name)
                else:
                    # at least a tile's worth of iterations per CTA (a tile has at most three contributors), and
                    # either ranges that start at the beginning or in the middle of a tile, or consecutive ranges
                    # that stay within half a tile of each other across the CTAs of an XCD
                    assert ipt <= per_cta < 2 * ipt, (dtype, M, N, K, name)
                    drift = min(per_cta - ipt, 2 * ipt - per_cta)
                    g = math.gcd(plan.streamk_tiles, plan.grid)
                    aligned = plan.grid // g <= 2
                    if plan.interleave > 1:
                        assert not aligned and g >= 8 and plan.interleave == plan.streamk_tiles // g, (dtype, M, N, K)
                        assert plan.grid == 256 and "256x256" in name, (dtype, M, N, K, name)
                        streamk_seen.add("interleaved")
                        continue
                    assert aligned or drift * (plan.grid // 8) <= ipt / 2, (dtype, M, N, K, name, plan.as_dict())
                    streamk_seen.add(aligned)
    assert SPLITK in seen and DP in seen and streamk_seen == {True, False, "interleaved"}   # every kind occurs
    # 258 tiles on 256 CUs: every tile is split (64.5 iterations per CTA), not the two remainder tiles alone
    p = sk.make_plan(1536, 11008, 4096, "float16", "nt", cus=256, use_tuned=False)
    assert (p.bm, p.bn, p.schedule, p.streamk_tiles, p.grid) == (256, 256, sk._lib.SCHEDULES["basic"], 258, 256)
    # 320 tiles of 80 iterations: 100 per CTA, five distinct offsets, 64 CTAs at each: the interleaved order
    p = sk.make_plan(4096, 5120, 5120, "float16", "nt", cus=256, use_tuned=False)
    assert (p.bm, p.bn, p.schedule, p.streamk_tiles, p.grid, p.interleave) == (256, 256, sk._lib.SCHEDULES["basic"], 320, 256, 5)
    # the assembly-loop kernel where it applies and the device is filled; a split in two halves below that
    p = sk.make_plan(8192, 8192, 8192, "float16", "nt", cus=256, use_tuned=False)
    assert (sk.kernel_name(p.kernel_id), p.schedule, p.grid) == ("tile_f16_nt_asm_256x256x64", DP, 256)
    p = sk.make_plan(1024, 8192, 8192, "float16", "nt", cus=256, use_tuned=False)
    assert (sk.kernel_name(p.kernel_id), p.schedule, p.grid) == ("tile_f16_nt_asm_256x256x64", SPLITK, 256)
    # few rows of A: the kernels that stream the weights through LDS, a tile per CU and no fix-up where N allows it
    for (M, N, K, dtype, want, grid) in [(16, 8192, 8192, "float16", "stream_f16_mb1_wm1_wn2_rk2_d3", 256),
                                         (5, 8192, 8192, "bfloat16", "stream_bf16_mb1_wm1_wn2_rk2_d3", 256),
                                         (16, 16384, 8192, "float16", "stream_f16_mb1_wm1_wn4_rk1_d4", 256),
                                         (16, 28672, 8192, "float16", "stream_f16_mb1_wm1_wn4_rk1_d4", 256),
                                         (16, 11008, 4096, "float16", "stream_f16_mb1_wm1_wn4_rk1_d4", 172),
                                         (16, 4096, 11008, "float16", "stream_f16_mb1_nb1_wm1_wn1_rk4_d3", 256),
                                         (8, 2048, 8192, "bfloat16", "stream_bf16_mb1_nb1_wm1_wn1_rk4_d3", 128),
                                         (32, 8192, 8192, "float16", "stream_f16_mb1_wm2_wn2_rk1_d4", 256),
                                         (64, 8192, 8192, "float16", "stream_f16_mb2_wm2_wn2_rk1_d3", 256),
                                         (64, 16384, 8192, "float16", "stream_f16_mb2_nb2_wm2_wn2_rk1_d3", 256),
                                         (64, 11008, 4096, "bfloat16", "stream_bf16_mb2_nb2_wm2_wn2_rk1_d3", 172),
                                         (4, 8192, 8192, "float16", "stream_f16_mb1_wm1_wn2_rk2_d3", 256),
                                         (4, 4096, 4096, "float16", "stream_f16_mb1_nb1_wm1_wn1_rk4_d3", 256),
                                         (2, 11008, 4096, "float16", "stream_f16_mb1_wm1_wn4_rk1_d4", 172),
                                         (32, 11008, 4096, "float16", "stream_f16_mb2_wm1_wn4_rk1_d3", 172),
                                         (80, 8192, 8192, "float16", "stream_f16_mb3_nb1_wm2_wn2_rk1_d4", 256),
                                         (96, 7168, 4096, "bfloat16", "stream_bf16_mb3_nb1_wm2_wn2_rk1_d4", 224),
                                         (3, 4096, 4160, "float16", "stream_f16_mb1_nb1_wm1_wn1_rk4_d3", 256),
                                         (16, 8192, 8192, "q4", "stream_q4_wn2_rk2_kh4_d3", 256),
                                         (16, 28672, 8192, "q4", "skinny_q4_mb1_wn4_rk2_row1_0", 448),
                                         (16, 4096, 4096, "q4", "stream_q4_wn2_rk2_kh4_d3", 128)]:
        p = sk.make_plan(M, N, K, dtype, "nt", cus=256, use_tuned=False)
        assert (sk.kernel_name(p.kernel_id), p.schedule, p.grid) == (want, DP, grid), (M, N, K, dtype, sk.kernel_name(p.kernel_id), p.grid)
    # a caller's tile or schedule is not overridden
    p = sk.make_plan(1024, 8192, 8192, "float16", "nt", cus=256, use_tuned=False, bm=128, bn=128)
    assert (p.bm, p.bn) == (128, 128)
    p = sk.make_plan(3000, 5120, 12288, "float16", "nt", cus=256, use_tuned=False, schedule="basic")
    assert p.schedule == sk._lib.SCHEDULES["basic"] and p.streamk_tiles == p.total_tiles


def test_interleaved_streamk_tile_order(sk):
    """interleave=1: with g = gcd(streamk_tiles, grid) and S = streamk_tiles / g, the CTAs pid, pid + grid/g, ...
    start S tiles apart at the same K offset; the interleaved order puts the tiles they work on next to each other.
    It permutes the Stream-K tiles among themselves and leaves the data-parallel ones alone."""
    base = dict(bm=256, bn=256, bk=64, raster=4, schedule="basic", fixup="reduce")
    plain = sk.make_plan(3000, 5120, 12288, "float16", "nt", cus=256, **base)
    plan = sk.make_plan(3000, 5120, 12288, "float16", "nt", cus=256, interleave=1, **base)
    assert (plan.grid, plan.streamk_tiles, plan.streamk_full_tiles, plan.streamk_partial_tiles) == (256, 240, 180, 0)
    assert plain.interleave == 0 and plan.interleave == 15        # g = gcd(240, 256) = 16, S = 15
    for v in range(plan.streamk_tiles):
        assert sk.tile_coords(plan, v) == sk.tile_coords(plain, (v % 15) * 16 + v // 15)
    assert len({sk.tile_coords(plan, v) for v in range(plan.total_tiles)}) == plan.total_tiles
    # the CTAs 16 apart are at the same offset of their tiles, and their tiles form one 4 x 4 block of the tile grid
    for pid in range(16):
        starts = [sk.cta_range(plan, pid + 16 * j)[0] for j in range(16)]
        assert len({s % plan.iters_per_tile for s in starts}) == 1
        tiles = [sk.tile_coords(plan, s // plan.iters_per_tile) for s in starts]
        assert max(m for m, _ in tiles) - min(m for m, _ in tiles) == 3 and max(n for _, n in tiles) - min(n for _, n in tiles) == 3
    # a hybrid schedule: only the Stream-K tiles move
    hy = sk.make_plan(8192, 8192 + 1280, 4096, "float16", "nt", cus=256, bm=256, bn=256, bk=64, raster=8, schedule="sk1",
                      fixup="reduce", interleave=1)
    hy0 = sk.make_plan(8192, 8192 + 1280, 4096, "float16", "nt", cus=256, bm=256, bn=256, bk=64, raster=8, schedule="sk1",
                       fixup="reduce")
    assert 0 < hy.streamk_tiles < hy.total_tiles and hy.interleave > 1
    assert {sk.tile_coords(hy, v) for v in range(hy.streamk_tiles)} == {sk.tile_coords(hy0, v) for v in range(hy.streamk_tiles)}
    assert all(sk.tile_coords(hy, v) == sk.tile_coords(hy0, v) for v in range(hy.streamk_tiles, hy.total_tiles))
    # nothing to interleave: every tile cut in two equal halves (all CTAs at offset 0 or ipt/2), data-parallel plans
    assert sk.make_plan(1024, 8192, 8192, "float16", "nt", cus=256, interleave=1, **base).interleave == 0
    assert sk.make_plan(8192, 8192, 8192, "float16", "nt", cus=256, bm=256, bn=256, schedule="dp", interleave=1).interleave == 0
    with pytest.raises(sk.StreamKError):
        sk.make_plan(3000, 5120, 12288, "float16", "nt", cus=256, interleave=2, **base)


def test_error_codes(sk):
    L = sk.lib()
    with pytest.raises(sk.StreamKError) as e:
        sk.make_plan(0, 10, 10, cus=256)
    assert e.value.status == -2
    with pytest.raises(sk.StreamKError) as e:
        sk.make_plan(128, 128, 100, cus=256)  # K not a multiple of 8
    assert e.value.status == -3
    with pytest.raises(sk.StreamKError) as e:
        sk.make_plan(128, 128, 128, cus=256, bm=48, bn=48)  # no such kernel
    assert e.value.status == -4
    with pytest.raises(sk.StreamKError) as e:
        sk.make_plan(4096, 4096, 4096, cus=256, bm=256, bn=256, grid=512)  # not co-resident
    assert e.value.status == -4
    plan = sk.make_plan(1024, 1024, 8192, cus=256, bm=128, bn=128, bk=64, grid=256)
    assert L.sk_gemm_f16(None, None, None, 1024, 1024, 8192, 8192, 8192, 1024, ctypes.byref(plan),
                         None, 0, None) == -1
    fake = ctypes.c_void_p(4096)
    # plan made for another shape
    assert L.sk_gemm_f16(fake, fake, fake, 512, 1024, 8192, 8192, 8192, 1024, ctypes.byref(plan),
                         None, 0, None) == -4
    # leading dimension smaller than the row / misaligned
    assert L.sk_gemm_f16(fake, fake, fake, 1024, 1024, 8192, 100, 8192, 1024, ctypes.byref(plan),
                         None, 0, None) == -2
    assert L.sk_gemm_f16(fake, fake, fake, 1024, 1024, 8192, 8196, 8192, 1024, ctypes.byref(plan),
                         None, 0, None) == -3
    assert L.sk_gemm_f16(ctypes.c_void_p(4098), fake, fake, 1024, 1024, 8192, 8192, 8192, 1024,
                         ctypes.byref(plan), None, 0, None) == -3
    # the extended entry points: reserved fields must be zero, the bias 2-byte aligned, the activation known; checked before anything runs
    from streamk._lib import SkEpilogue
    epi = SkEpilogue(bias=4096)
    epi.reserved[1] = 7
    assert L.sk_gemm_f16_ex(fake, fake, fake, 1024, 1024, 8192, 8192, 8192, 1024, ctypes.byref(plan), None, 0, None,
                            ctypes.byref(epi)) == -4
    assert L.sk_gemm_f16_ex(fake, fake, fake, 1024, 1024, 8192, 8192, 8192, 1024, ctypes.byref(plan), None, 0, None,
                            ctypes.byref(SkEpilogue(bias=4097))) == -3
    # activation codes outside sk_activation, and a bias that cannot be a device address
    for bad in (SkEpilogue(bias=4096, activation=4), SkEpilogue(bias=None, activation=-1), SkEpilogue(bias=1 << 61)):
        assert L.sk_gemm_f16_ex(fake, fake, fake, 1024, 1024, 8192, 8192, 8192, 1024, ctypes.byref(plan), None, 0, None,
                                ctypes.byref(bad)) == -4
    assert L.sk_gemm_f16_ex(None, fake, fake, 1024, 1024, 8192, 8192, 8192, 1024, ctypes.byref(plan), None, 0, None,
                            None) == -1
    assert L.sk_dequant_q4(fake, fake, fake, 16, 100, 128, 8, None) == -4
    assert L.sk_workspace_init(None, 16, None) == -1


def test_product_does_not_touch_the_oracle():
    """The shipped package must never import or call the CPU checker."""
    pkg = os.path.join(ROOT, "stream-k.tvm_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".h", ".hip", ".cpp", "Makefile")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_autotune_candidates_make_plans():
    """The tuner's search space on the host: for every dtype and a decode-, a batch- and a prefill-sized M the
    candidates are distinct, and each either makes a plan for the shape or is refused as a configuration (-4) --
    never another error; at least one per list is valid."""
    import streamk
    from streamk._lib import StreamKError
    at = sys.modules["streamk.autotune"]
    for dtype in ("float16", "bfloat16", "q4", "q4_zp", "float8_e4m3", "float8_e5m2", "int8"):
        for M in (1, 16, 64, 512, 4096):
            if dtype in ("q4", "q4_zp") and M > 64:
                continue
            cands = at.candidate_configs(M, 4096, 4096, dtype, cus=256)
            assert cands and len({tuple(sorted(c.items())) for c in cands}) == len(cands), (dtype, M)
            valid = 0
            for c in cands:
                try:
                    p = streamk.make_plan(M, 4096, 4096, dtype, "nt", c, cus=256)
                    assert p.total_tiles > 0 and p.grid > 0
                    valid += 1
                except StreamKError as e:
                    assert e.status == -4, (dtype, M, c, e.status)
            assert valid > 0, (dtype, M)


def test_operator_plans_follow_the_tuned_cache(monkeypatch):
    """The operator layer keeps the plans it made from the tuned cache; an autotune run that writes a new entry
    invalidates the cache, and the next call of the operator for that shape must run the new plan."""
    import sys
    import streamk  # noqa: F401
    from streamk import ops
    from streamk import plan as P
    autotune = sys.modules["streamk.autotune"]   # (the package exports a function of the same name)
    monkeypatch.setattr(P, "num_cus", lambda: 256)
    key = "gfx950/float16/nt/512x4096x4096"
    entries = {key: {"config": dict(bm=128, bn=128, bk=64, schedule="dp")}}
    monkeypatch.setattr(autotune, "load_cache", lambda path=None: dict(entries))
    P.invalidate_tuned_cache()
    p1 = ops._plan_for("", 512, 4096, 4096, "float16", "nt")
    assert (p1.bm, p1.bn) == (128, 128)
    assert ops._plan_for("", 512, 4096, 4096, "float16", "nt") is p1
    entries[key] = {"config": dict(bm=256, bn=256, bk=64, schedule="dp")}
    P.invalidate_tuned_cache()      # what autotune(..., cache=True) does after writing its entry
    p2 = ops._plan_for("", 512, 4096, 4096, "float16", "nt")
    assert (p2.bm, p2.bn) == (256, 256)
    monkeypatch.undo()
    P.invalidate_tuned_cache()

"""Pins the oracle's partitioner (restating streamk_fp32.py:33-54, 93-136 of the reference) against
hand-worked numbers, the paper schematic in figures/image.png, invariants and a Python twin."""
import itertools

import pytest
from hypothesis import given, settings, strategies as st


# Values of the reference's own variables at the shapes its scripts run (P = total_sm = 108),
# worked by hand from streamk_fp32.py:15-54 and streamk_fp16_block_reduce.py:66-71.
REFERENCE_SHAPES = [
    # M, N, K, BM, BN, BK, P -> expected
    ((16, 16384, 8192, 32, 64, 32, 108),
     dict(total_tiles=256, iters_per_tile=256, streamk_tiles=148, blocking_tiles=108,
          streamk_full_tiles=350, streamk_partial_tiles=88, sm_partition_factor=1)),
    ((256, 1024, 512, 16, 16, 32, 108),
     dict(total_tiles=1024, iters_per_tile=16, streamk_tiles=160, blocking_tiles=864,
          streamk_full_tiles=23, streamk_partial_tiles=76, sm_partition_factor=8)),
    # the repository's CPU configuration: 256x256x1024, 64x64x16 tiles, 4 CTAs
    ((256, 256, 1024, 64, 64, 16, 4),
     dict(total_tiles=16, iters_per_tile=64, streamk_tiles=4, blocking_tiles=12,
          streamk_iters=256, streamk_full_tiles=64, streamk_partial_tiles=0, sm_partition_factor=3)),
    # 1024x1024x8192 with 128x128x32 tiles on 256 CUs: no data-parallel tiles at all, where the
    # reference's max(..., 1) would run an out-of-range tile
    ((1024, 1024, 8192, 128, 128, 32, 256),
     dict(total_tiles=64, iters_per_tile=256, streamk_tiles=64, blocking_tiles=0,
          streamk_full_tiles=64, streamk_partial_tiles=0, sm_partition_factor=0)),
]


@pytest.mark.parametrize("args,expected", REFERENCE_SHAPES)
def test_reference_shapes(oracle, args, expected):
    got = oracle.partition(*args)
    for k, v in expected.items():
        assert got[k] == v, (k, got)
    assert got == oracle.partition_py(*args)


def test_paper_figure_hybrid(oracle):
    """figures/image.png: 384x384x128 GEMM, 128x128 tiles (9 tiles), 4 SMs, 4 K-iterations per tile.
    The reference's two-tile rule turns 9 tiles on 4 CTAs into 5 Stream-K + 4 data-parallel tiles,
    5 iterations per CTA."""
    p = oracle.partition(384, 384, 128, 128, 128, 32, 4)
    assert (p["total_tiles"], p["iters_per_tile"]) == (9, 4)
    assert (p["streamk_tiles"], p["blocking_tiles"]) == (5, 4)
    assert (p["streamk_full_tiles"], p["streamk_partial_tiles"], p["sm_partition_factor"]) == (5, 0, 1)
    segs = [oracle.cta_segments_py(p, pid) for pid in range(4)]
    # CTA0: tile0 whole + 1/4 of tile1; CTA1: 3/4 of tile1 + 2/4 of tile2; ...
    assert segs[0] == [(0, 0, 4, True), (1, 0, 1, False)]
    assert segs[1] == [(1, 1, 3, False), (2, 0, 2, False)]
    assert segs[2] == [(2, 2, 2, False), (3, 0, 3, False)]
    assert segs[3] == [(3, 3, 1, False), (4, 0, 4, True)]
    assert [oracle.dp_tiles_py(p, pid, 4) for pid in range(4)] == [[5], [6], [7], [8]]


def test_paper_figure_basic_streamk(oracle):
    """Basic Stream-K of the same figure: 36 iterations over 4 CTAs = 9 each, i.e. 2.25 tiles per
    CTA: {0, 1, 1/4 of 2}, {3/4 of 2, 3, 1/2 of 4}, {1/2 of 4, 5, 3/4 of 6}, {1/4 of 6, 7, 8}."""
    part = dict(streamk_full_tiles=9, streamk_partial_tiles=0, iters_per_tile=4)
    segs = [oracle.cta_segments_py(part, pid) for pid in range(4)]
    assert segs[0] == [(0, 0, 4, True), (1, 0, 4, True), (2, 0, 1, False)]
    assert segs[1] == [(2, 1, 3, False), (3, 0, 4, True), (4, 0, 2, False)]
    assert segs[2] == [(4, 2, 2, False), (5, 0, 4, True), (6, 0, 3, False)]
    assert segs[3] == [(6, 3, 1, False), (7, 0, 4, True), (8, 0, 4, True)]


@settings(max_examples=300, deadline=None)
@given(M=st.integers(1, 300), N=st.integers(1, 300), K=st.integers(1, 400),
       BM=st.sampled_from([8, 16, 32, 64]), BN=st.sampled_from([8, 16, 64]),
       BK=st.sampled_from([8, 16, 32]), P=st.integers(1, 40))
def test_invariants(oracle, M, N, K, BM, BN, BK, P):
    p = oracle.partition(M, N, K, BM, BN, BK, P)
    assert p == oracle.partition_py(M, N, K, BM, BN, BK, P)
    ipt = p["iters_per_tile"]
    assert p["streamk_tiles"] + p["blocking_tiles"] == p["total_tiles"]
    assert p["blocking_tiles"] % P == 0 and p["streamk_tiles"] < 2 * P
    # CTA ranges tile [0, streamk_iters) exactly once, balanced to within one iteration
    covered, lens, nonowner = [], [], 0
    prev_end = 0
    for pid in range(P):
        s, e = oracle.cta_range(p, pid)
        assert s == prev_end
        prev_end = e
        lens.append(e - s)
        segs = oracle.cta_segments_py(p, pid)
        assert sum(n for _, _, n, _ in segs) == e - s
        for tile, k0, n, whole in segs:
            assert 0 <= tile < p["streamk_tiles"] and k0 + n <= ipt  # a segment stays in one tile
            assert whole == (n == ipt)
            covered.extend((tile, k0 + i) for i in range(n))
        nonowner_here = sum(1 for _, k0, _, _ in segs if k0 != 0)
        assert nonowner_here <= 1  # at most one partial a CTA does not own: one slot per CTA suffices
    assert prev_end == p["streamk_iters"]
    assert max(lens) - min(lens) <= 1
    assert sorted(covered) == [(t, i) for t in range(p["streamk_tiles"]) for i in range(ipt)]
    # data-parallel tiles: disjoint from the Stream-K tiles, each exactly once
    dp = list(itertools.chain.from_iterable(oracle.dp_tiles_py(p, pid, P) for pid in range(P)))
    assert sorted(dp) == list(range(p["streamk_tiles"], p["total_tiles"]))

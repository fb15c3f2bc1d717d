"""Offline side of the Q4 path (host entry points of the C ABI): nibble packing in the order the
reference expands (streamk_fp16_ladder_block_reduce_q4.py:552) and this build's group-wise
quantiser, against hand-worked cases, the reference's own expansion expression and the oracle's
numpy restatement."""
import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def sk():
    import streamk
    streamk.lib()
    return streamk


def test_pack_is_inverse_of_the_reference_expansion(sk, oracle):
    rng = np.random.default_rng(0)
    for (N, K) in [(1, 2), (3, 128), (17, 384), (64, 4096)]:
        q = rng.integers(0, 16, (N, K), dtype=np.uint8)
        Wq = sk.pack_q4(torch.from_numpy(q))
        assert Wq.shape == (N, K // 2)
        # the reference's expansion of a packed array, streamk_fp16_ladder_block_reduce_q4.py:552
        expanded = ((Wq.unsqueeze(-1) >> (4 * torch.arange(2))) & 0xF).reshape(N, K)
        assert np.array_equal(expanded.numpy(), q)
        assert np.array_equal(Wq.numpy(), oracle.pack_q4_np(q))
        assert np.array_equal(sk.unpack_q4(Wq).numpy(), q)
        assert np.array_equal(oracle.unpack_q4_np(Wq.numpy()), q)
    # byte-level known answer: elements (k even, k odd) = (0x3, 0xA) -> byte 0xA3
    assert sk.pack_q4(torch.tensor([[3, 10, 15, 0]], dtype=torch.uint8)).tolist() == [[0xA3, 0x0F]]


def test_quantiser_hand_worked_groups(sk):
    # max|w| = 7, zero = 8: scale = 1, q = w + 8
    w = np.resize(np.arange(-7, 8), 128).astype(np.float16)[None, :]
    Wq, sc = sk.quantize_q4(torch.from_numpy(w), group=128, zero=8)
    assert sc.tolist() == [[1.0]]
    assert np.array_equal(sk.unpack_q4(Wq).numpy()[0], (w[0] + 8).astype(np.uint8))
    # max|w| = 3.5: scale = 0.5; ties go to even: 1.25 -> 2.5 -> 2, 1.75 -> 3.5 -> 4, -0.25 -> -0.5 -> -0
    w = np.zeros((1, 128), dtype=np.float16)
    w[0, :6] = [3.5, 1.25, 1.75, -0.25, -3.5, 0.74]
    Wq, sc = sk.quantize_q4(torch.from_numpy(w), group=128, zero=8)
    assert sc.tolist() == [[0.5]]
    assert sk.unpack_q4(Wq).numpy()[0, :7].tolist() == [15, 10, 12, 8, 1, 9, 8]
    # an all-zero group: scale 0, every nibble is the zero point
    Wq, sc = sk.quantize_q4(torch.zeros(2, 256, dtype=torch.float16), zero=5)
    assert sc.abs().max().item() == 0 and set(sk.unpack_q4(Wq).flatten().tolist()) == {5}
    # zero point at an end of the range: fifteen levels on one side, the other side clamps
    w = np.zeros((1, 128), dtype=np.float16)
    w[0, :4] = [30.0, 15.0, -30.0, 2.0]
    Wq, sc = sk.quantize_q4(torch.from_numpy(w), zero=0)
    assert sc.tolist() == [[2.0]] and sk.unpack_q4(Wq).numpy()[0, :4].tolist() == [15, 8, 0, 1]
    Wq, sc = sk.quantize_q4(torch.from_numpy(w), zero=15)
    assert sk.unpack_q4(Wq).numpy()[0, :4].tolist() == [15, 15, 0, 15]


@pytest.mark.parametrize("zero", [0, 5, 8, 15])
@pytest.mark.parametrize("group", [32, 128])
def test_quantiser_matches_numpy_restatement(sk, oracle, zero, group):
    rng = np.random.default_rng(zero * 10 + group)
    N, K, pad = 40, 1024, 24
    W = (rng.standard_normal((N, K + pad), dtype=np.float32) * 0.02).astype(np.float16)
    W[0, :group] = 0                                   # scale 0
    W[1, :group] = np.float16(6e-8) * rng.integers(-3, 4, group)   # subnormals: scale rounds to a subnormal or 0
    W[2, :group] = 65504 * rng.choice([-1, 1], group)  # largest finite values
    W[3, :group] = rng.integers(-40, 41, group) * 0.25  # many exact ties
    Wt = torch.from_numpy(W)[:, :K]                    # row pitch K + pad
    Wq, sc = sk.quantize_q4(Wt, group=group, zero=zero)
    Wq_np, sc_np = oracle.quantize_q4_np(W[:, :K], group=group, zero=zero)
    assert np.array_equal(sc.numpy().view(np.uint16), sc_np.view(np.uint16))
    assert np.array_equal(Wq.numpy(), Wq_np)


def test_quantisation_error_is_half_a_step(sk, oracle):
    """zero = 8: seven levels either side, nothing clamps, so every weight is reproduced to within
    half a quantisation step (plus the fp16 rounding of the product)."""
    rng = np.random.default_rng(3)
    W = (rng.standard_normal((64, 2048), dtype=np.float32)).astype(np.float16)
    Wq, sc = sk.quantize_q4(torch.from_numpy(W))
    back = oracle.dequant_q4(Wq.numpy(), sc.numpy()).astype(np.float32)
    step = np.repeat(sc.numpy().astype(np.float32), 128, axis=1)
    assert np.all(np.abs(back - W.astype(np.float32)) <= step * (0.5 + 2.0 ** -9))
    assert sk.unpack_q4(Wq).numpy().min() >= 1  # -8 is never used


def test_tiled_layout_round_trip_and_offsets(sk):
    """Byte b of row n goes to ((n/16) * (K/128) + b/64) * 1024 + (n%16) * 64 + b%64; rows are padded
    to a multiple of 16 with zeros; untile is the inverse."""
    rng = np.random.default_rng(9)
    for (N, K) in [(16, 128), (40, 384), (1000, 1152), (8, 256)]:
        Wq = rng.integers(0, 256, (N, K // 2), dtype=np.uint8)
        T = sk.tile_q4(torch.from_numpy(Wq))
        n16 = (N + 15) // 16 * 16
        assert T.shape == (n16, K // 2)
        flat = T.numpy().reshape(-1)
        runs = K // 128
        for (n, b) in [(0, 0), (N - 1, K // 2 - 1), (N // 2, 67 % (K // 2)), (min(17, N - 1), 64 % (K // 2))]:
            assert flat[((n // 16) * runs + b // 64) * 1024 + (n % 16) * 64 + b % 64] == Wq[n, b]
        # a tile holds 16 rows x 64 bytes, row by row
        tiles = flat.reshape(n16 // 16, runs, 16, 64)
        padded = np.zeros((n16, K // 2), dtype=np.uint8)
        padded[:N] = Wq
        assert np.array_equal(tiles, padded.reshape(n16 // 16, 16, runs, 64).transpose(0, 2, 1, 3))
        assert np.array_equal(sk.untile_q4(T, N).numpy(), Wq)
    with pytest.raises(sk.StreamKError):
        sk.tile_q4(torch.zeros(4, 100, dtype=torch.uint8))  # K not a multiple of 128


def test_bad_arguments(sk):
    with pytest.raises(sk.StreamKError):
        sk.pack_q4(torch.full((2, 4), 16, dtype=torch.uint8))       # not a nibble
    with pytest.raises(sk.StreamKError):
        sk.pack_q4(torch.zeros((2, 3), dtype=torch.uint8))          # odd K
    w = torch.zeros(2, 128, dtype=torch.float16)
    w[1, 5] = float("nan")
    with pytest.raises(sk.StreamKError):
        sk.quantize_q4(w)
    with pytest.raises(sk.StreamKError):
        sk.quantize_q4(torch.zeros(2, 100, dtype=torch.float16))    # K not a multiple of the group
    with pytest.raises(sk.StreamKError):
        sk.quantize_q4(torch.zeros(2, 128, dtype=torch.float16), zero=16)


def test_asymmetric_quantiser_hand_worked_groups(sk, oracle):
    """One zero point per group: hand-worked groups, then the host entry point against the oracle's numpy
    restatement, and the round trip error bound of one step."""
    # range [-5, 10]: scale = 1, z = 5, q = w + 5
    w = np.resize(np.arange(-5, 11), 128).astype(np.float16)[None, :]
    Wq, sc, zp = sk.quantize_q4(torch.from_numpy(w), asymmetric=True)
    assert sc.tolist() == [[1.0]] and zp.tolist() == [[5.0]] and zp.dtype == torch.float16
    assert np.array_equal(sk.unpack_q4(Wq).numpy()[0], (w[0] + 5).astype(np.uint8))
    # all positive [0.5 .. 7.5]: the range is widened to contain 0: scale 0.5, z = 0; ties to even (1.25 / 0.5 = 2.5 -> 2)
    w = np.zeros((1, 128), dtype=np.float16)
    w[0, :4] = [7.5, 0.5, 1.25, 1.75]
    Wq, sc, zp = sk.quantize_q4(torch.from_numpy(w), asymmetric=True)
    assert sc.tolist() == [[0.5]] and zp.tolist() == [[0.0]]
    assert sk.unpack_q4(Wq).numpy()[0, :5].tolist() == [15, 1, 2, 4, 0]
    # all negative: z = 15
    Wq, sc, zp = sk.quantize_q4(torch.from_numpy(-w), asymmetric=True)
    assert zp.tolist() == [[15.0]] and sk.unpack_q4(Wq).numpy()[0, :5].tolist() == [0, 14, 13, 11, 15]   # rint(-2.5) + 15 = 13
    # an all-zero group: scale 0, zero point 0, nibbles 0
    Wq, sc, zp = sk.quantize_q4(torch.zeros(2, 256, dtype=torch.float16), asymmetric=True)
    assert sc.abs().max().item() == 0 and zp.abs().max().item() == 0 and Wq.abs().max().item() == 0
    # two groups of one row get their own zero points
    w = np.concatenate([np.resize(np.arange(-5, 11), 128), np.resize(np.arange(-12, 4), 128)]).astype(np.float16)[None, :]
    Wq, sc, zp = sk.quantize_q4(torch.from_numpy(w), asymmetric=True)
    assert sc.tolist() == [[1.0, 1.0]] and zp.tolist() == [[5.0, 12.0]]
    rng = np.random.default_rng(3)
    for (N, K, group) in [(5, 256, 128), (33, 1024, 128), (4, 256, 32)]:
        W = (rng.standard_normal((N, K)) * rng.uniform(0.01, 4.0, (N, 1)) + rng.uniform(-2, 2, (N, 1))).astype(np.float16)
        Wq, sc, zp = sk.quantize_q4(torch.from_numpy(W), group=group, asymmetric=True)
        rq, rs, rz = oracle.quantize_q4_zp_np(W, group)
        assert np.array_equal(Wq.numpy(), rq) and np.array_equal(sc.numpy(), rs) and np.array_equal(zp.numpy(), rz)
        assert set(np.unique(rz)) <= set(np.arange(16, dtype=np.float16))
        back = oracle.dequant_q4_zp_np(rq, rs, rz, group).astype(np.float32)
        step = np.repeat(rs.astype(np.float32), group, axis=1)
        # half a step from rounding q, up to another half where the rounded zero point pushes the end of the range out
        assert np.all(np.abs(back - W.astype(np.float32)) <= step * 1.002 + 1e-6)
    with pytest.raises(sk.StreamKError):
        sk.quantize_q4(torch.full((1, 128), float("inf"), dtype=torch.float16), asymmetric=True)


def test_per_group_zero_point_dequant_reduces_to_the_scalar_form(oracle):
    """The oracle's per-group form with a constant zero point is the pinned scalar form (numpy and C), and a
    hand-worked row shows each group using its own zero point."""
    rng = np.random.default_rng(5)
    Wq = rng.integers(0, 256, (7, 192), dtype=np.uint8)
    sc = rng.uniform(0.01, 0.5, (7, 3)).astype(np.float16)
    for z in (0, 3, 8, 15):
        zs = np.full((7, 3), z, dtype=np.float16)
        assert np.array_equal(oracle.dequant_q4_zp_np(Wq, sc, zs).view(np.uint16), oracle.dequant_q4(Wq, sc, 128, z).view(np.uint16))
    Wq = np.tile(np.array([0x10, 0xF7], dtype=np.uint8), 64)[None, :]      # nibbles 0, 1, 7, 15 repeating; two groups
    out = oracle.dequant_q4_zp_np(Wq, np.array([[0.5, 2.0]], np.float16), np.array([[1, 7]], np.float16))
    assert out[0, :4].tolist() == [-0.5, 0.0, 3.0, 7.0] and out[0, 128:132].tolist() == [-14.0, -12.0, 0.0, 16.0]

"""Pins the oracle's CPU Stream-K GEMM (restating streamk_fp32.py:80-158) against dense matmul, and
the committed golden fixture against both."""
import os

import numpy as np
import pytest


def _inputs(M, N, K, seed=0):
    # uniform [-1, 1), the reference's distribution (streamk_fp32.py:19-22)
    rng = np.random.default_rng(seed)
    return (rng.random((M, K), dtype=np.float32) * 2 - 1, rng.random((K, N), dtype=np.float32) * 2 - 1)


@pytest.mark.parametrize("P", [4, 3, 5, 7])
@pytest.mark.parametrize("fixup", ["atomic", "reduce"])
def test_cpu_config_256x256x1024(oracle, P, fixup):
    """M=256, N=256, K=1024, 64x64 tiles, 16-wide K-iterations, 4 simulated CTAs (no tile is split at
    P=4; P=3,5,7 split tiles and exercise the fix-up), checked against numpy matmul with the
    reference's tolerance (streamk_fp32.py:208)."""
    A, B = _inputs(256, 256, 1024)
    C = oracle.streamk_gemm_f32(A, B, 64, 64, 16, P, fixup=fixup)
    ref = A.astype(np.float64) @ B.astype(np.float64)
    np.testing.assert_allclose(C, ref, rtol=1e-2, atol=1e-2)
    assert oracle.max_abs_rel(C, ref) < 1e-5


def test_exact_on_integers(oracle):
    """Small-integer inputs make every partial sum exact in fp32, so Stream-K must equal numpy
    bit for bit whatever the split: catches a dropped / doubled K-iteration or a wrong tile index."""
    rng = np.random.default_rng(1)
    A = rng.integers(-4, 5, (70, 90)).astype(np.float32)
    B = rng.integers(-4, 5, (90, 50)).astype(np.float32)
    ref = A @ B
    for P in (1, 2, 3, 5, 8, 13):
        for fixup in ("atomic", "reduce"):
            for bm, bn, bk in ((16, 8, 8), (32, 32, 16), (8, 64, 32)):
                C = oracle.streamk_gemm_f32(A, B, bm, bn, bk, P, fixup=fixup)
                assert np.array_equal(C, ref), (P, fixup, bm, bn, bk)
    Bt = np.ascontiguousarray(B.T)
    assert np.array_equal(oracle.streamk_gemm_f32(A, Bt, 16, 8, 8, 5, trans_b=True), ref)


def test_cta_order(oracle):
    """The ordered reduce does not depend on the order CTAs run in; the atomic flavour may differ in
    the last bits but stays within tolerance."""
    A, B = _inputs(96, 80, 200, seed=2)
    base = oracle.streamk_gemm_f32(A, B, 32, 16, 8, 7, fixup="reduce")
    rng = np.random.default_rng(3)
    for _ in range(5):
        order = rng.permutation(7)
        assert np.array_equal(oracle.streamk_gemm_f32(A, B, 32, 16, 8, 7, cta_order=order, fixup="reduce"), base)
        C = oracle.streamk_gemm_f32(A, B, 32, 16, 8, 7, cta_order=order, fixup="atomic")
        assert oracle.max_abs_rel(C, base) < 1e-5


def test_golden_fixture(oracle, golden_dir):
    g = np.load(os.path.join(golden_dir, "streamk_f32_48x40x72.npz"))
    A, B = g["A"], g["B"]
    assert np.array_equal(oracle.streamk_gemm_f32(A, B, 16, 8, 8, 7, fixup="atomic"), g["C_atomic"])
    assert np.array_equal(oracle.streamk_gemm_f32(A, B, 16, 8, 8, 7, fixup="reduce"), g["C_reduce"])
    ref = A.astype(np.float64) @ B.astype(np.float64)
    assert oracle.max_abs_rel(g["C_atomic"], ref) < 1e-5 and oracle.max_abs_rel(g["C_reduce"], ref) < 1e-5
    part = oracle.partition(48, 40, 72, 16, 8, 8, 7)
    assert [part[k] for k in g["partition_keys"]] == g["partition"].tolist()
    # 15 tiles of 9 iterations on 7 CTAs: 15 % 7 + 7 = 8 Stream-K tiles = 72 iterations,
    # 10 per CTA and 2 left over; 7 data-parallel tiles
    assert (part["total_tiles"], part["streamk_tiles"], part["blocking_tiles"]) == (15, 8, 7)
    assert (part["streamk_full_tiles"], part["streamk_partial_tiles"]) == (10, 2)


def test_bad_arguments(oracle):
    A, B = _inputs(8, 8, 8)
    with pytest.raises(ValueError):
        oracle.streamk_gemm_f32(A, B, 0, 8, 8, 2)


def test_f8e4m3_decode(oracle):
    """The e4m3 decoder of the fp8 oracle against the format's definition (known values: 1.0, the largest
    finite value 448, the smallest subnormal 2^-9 and normal 2^-6, the two NaN patterns, signed zero;
    strictly increasing over the positive bytes) and against torch's own CPU conversion of all 256 bytes."""
    import torch
    d = oracle.f8e4m3_decode(np.arange(256, dtype=np.uint8))
    assert d.dtype == np.float32
    assert d[0x38] == 1.0 and d[0x7E] == 448.0 and d[0x01] == 2.0 ** -9 and d[0x08] == 2.0 ** -6 and d[0x07] == 7 * 2.0 ** -9
    assert d[0x00] == 0 and d[0x80] == 0 and np.signbit(d[0x80]) and not np.signbit(d[0x00])
    assert np.isnan(d[0x7F]) and np.isnan(d[0xFF]) and np.isnan(d).sum() == 2
    assert np.all(np.diff(d[:0x7F]) > 0) and np.array_equal(d[0x80:0xFF], -d[:0x7F])
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    assert np.array_equal(np.isnan(d), np.isnan(t)) and np.array_equal(d[~np.isnan(d)], t[~np.isnan(t)])
    # the host product is the plain sum of products
    A = np.array([[0x38, 0x40, 0xB8, 0x01]], dtype=np.uint8)   # 1, 2, -1, 2^-9
    B = np.array([[0x38, 0x38, 0x40, 0x7E], [0, 0, 0, 0]], dtype=np.uint8)   # 1, 1, 2, 448
    assert np.array_equal(oracle.f8_gemm_ref(A, B), [[1 + 2 - 2 + 448 * 2.0 ** -9, 0.0]])


def test_f8e5m2_decode(oracle):
    """e5m2 decoder: known values (1.0 = 0x3C, largest finite 57344 = 0x7B, smallest subnormal 2^-16 = 0x01,
    smallest normal 2^-14 = 0x04, infinities 0x7C / 0xFC, NaNs above them), a closed form over all finite
    bytes, and torch's CPU conversion of all 256 bytes."""
    import torch
    d = oracle.f8e5m2_decode(np.arange(256, dtype=np.uint8))
    assert d[0x3C] == 1.0 and d[0x7B] == 57344.0 and d[0x01] == 2.0 ** -16 and d[0x04] == 2.0 ** -14 and d[0xC0] == -2.0
    assert np.isposinf(d[0x7C]) and np.isneginf(d[0xFC]) and np.isnan(d[0x7D:0x80]).all() and np.isnan(d[0xFD:]).all()
    for b in range(0x7C):
        e, m = b >> 2, b & 3
        assert d[b] == (m * 2.0 ** -16 if e == 0 else (4 + m) * 2.0 ** (e - 17)) and d[b | 0x80] == -d[b]
    t = torch.arange(256, dtype=torch.uint8).view(torch.float8_e5m2).float().numpy()
    assert np.array_equal(np.isnan(d), np.isnan(t)) and np.array_equal(d[~np.isnan(d)], t[~np.isnan(t)])
    A = np.array([[0x3C, 0x40, 0xBC, 0x01]], dtype=np.uint8)   # 1, 2, -1, 2^-16
    B = np.array([[0x3C, 0x3C, 0x40, 0x7B]], dtype=np.uint8)   # 1, 1, 2, 57344
    assert np.array_equal(oracle.f8_gemm_ref(A, B, "e5m2"), [[1 + 2 - 2 + 57344 * 2.0 ** -16]])


def test_i8_gemm_ref(oracle):
    """The int8 host product: hand-worked values at the ends of the range and agreement with a Python-int loop."""
    A = np.array([[-128, 127, 1, 0], [1, 1, 1, 1]], dtype=np.int8)
    B = np.array([[-128, 127, -1, 5], [127, -128, 0, 0], [0, 0, 0, 0]], dtype=np.int8)
    assert np.array_equal(oracle.i8_gemm_ref(A, B), [[16384 + 16129 - 1, -16256 - 16256, 0], [3, -1, 0]])
    rs = np.random.RandomState(0)
    A, B = rs.randint(-128, 128, (5, 37)).astype(np.int8), rs.randint(-128, 128, (4, 37)).astype(np.int8)
    want = [[sum(int(a) * int(b) for a, b in zip(ra, rb)) for rb in B] for ra in A]
    assert np.array_equal(oracle.i8_gemm_ref(A, B), want)


def test_activation_ref(oracle):
    """The activations of the fused epilogue against torch's CPU routines (float64), the erf form of GELU (the
    tanh form stays within 1e-3 of it), and their limits: 0 at 0, the identity far right, 0 far left."""
    import torch
    from scipy.special import erf
    x = np.concatenate([np.linspace(-12, 12, 4801), [0.0, 1e-8, -1e-8, 40.0, -40.0, 700.0, -700.0]])
    t = torch.from_numpy(x)
    assert np.array_equal(oracle.activation_ref(x, "relu"), torch.relu(t).numpy())
    assert np.allclose(oracle.activation_ref(x, "gelu_tanh"), torch.nn.functional.gelu(t, approximate="tanh").numpy(),
                       rtol=1e-12, atol=1e-14)  # 1 + tanh cancels in the far left tail
    assert np.allclose(oracle.activation_ref(x, "silu"), torch.nn.functional.silu(t).numpy(), rtol=1e-12,
                       atol=1e-300)
    assert np.max(np.abs(oracle.activation_ref(x, "gelu_tanh") - 0.5 * x * (1 + erf(x / np.sqrt(2))))) < 1e-3
    for name in ("relu", "gelu_tanh", "silu"):
        y = oracle.activation_ref(np.array([0.0, 40.0, -40.0]), name)
        assert y[0] == 0 and abs(y[1] - 40.0) < 1e-12 and abs(y[2]) < 1e-12, name
    assert np.array_equal(oracle.activation_ref(x, None), x)
    with pytest.raises(ValueError):
        oracle.activation_ref(x, "tanh")

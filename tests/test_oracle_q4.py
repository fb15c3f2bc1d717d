"""Pins the oracle's Q4 dequantisation: element order from the reference
(streamk_fp16_ladder_block_reduce_q4.py:552), value w = fp16((fp16(q) - zero) * scale)."""
import os

import numpy as np


def test_reference_subset_is_plain_nibbles(oracle):
    """zero = 0, scale = 1 is exactly what the reference computes: the nibble as fp16."""
    rng = np.random.default_rng(0)
    Wq = rng.integers(0, 256, (8, 64), dtype=np.uint8)
    ones = np.ones((8, 1), dtype=np.float16)
    W = oracle.dequant_q4(Wq, ones, group=128, zero=0)
    # scalar form of thread_level_gemm_with_macro_ladder_q4_atomic.py:280-282
    for i in range(8):
        for j in range(128):
            assert W[i, j] == np.float16((int(Wq[i, j // 2]) >> (4 * (j % 2))) & 0xF)


def test_half_conversions_exhaustive(oracle):
    """The C restatement rounds in software; check it on every binary16 value and on the exact
    products the dequant forms, against numpy's float16."""
    L = oracle.lib()
    bits = np.arange(65536, dtype=np.uint16)
    as_f32 = bits.view(np.float16).astype(np.float32)
    finite = np.isfinite(as_f32)
    for b in bits[finite][::7]:
        assert L.ora_half_to_float(int(b)) == as_f32[b]
        assert L.ora_float_to_half(float(as_f32[b])) == b


def test_all_nibbles_all_scales(oracle):
    """16 nibbles x every finite fp16 scale (63 488 values incl. subnormals): C restatement ==
    numpy float16 arithmetic, bit for bit."""
    bits = np.arange(65536, dtype=np.uint16)
    scales_all = bits.view(np.float16)
    scales_all = scales_all[np.isfinite(scales_all.astype(np.float32))]
    assert scales_all.size == 63488
    # one row per scale, one 128-wide group per row holding every nibble 8 times
    N, K = scales_all.size, 128
    nib = (np.arange(K) % 16).astype(np.uint8)
    Wq_row = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8)
    Wq = np.broadcast_to(Wq_row, (N, K // 2)).copy()
    sc = scales_all.reshape(N, 1)
    for zero in (8, 0, 15):
        a = oracle.dequant_q4(Wq, sc, 128, zero).view(np.uint16)
        b = oracle.dequant_q4_np(Wq, sc, 128, zero).view(np.uint16)
        # -0.0 vs +0.0 cannot differ either: both compute (q - zero) * s with IEEE signs
        assert np.array_equal(a, b), zero


def test_golden_fixture(oracle, golden_dir):
    g = np.load(os.path.join(golden_dir, "q4_16x256.npz"))
    assert np.array_equal(oracle.unpack_q4_np(g["Wq"]), g["nibbles"])
    W = oracle.dequant_q4(g["Wq"], g["scales"], 128, 8)
    assert np.array_equal(W.view(np.uint16), g["W"].view(np.uint16))
    # closed form on a few elements, computed in exact rational-free float64 then rounded once
    for (n, k) in [(0, 0), (3, 17), (15, 255), (7, 128)]:
        q = int(g["nibbles"][n, k])
        exact = (q - 8) * float(g["scales"][n, k // 128])
        assert W[n, k] == np.float16(exact)
    ref = g["A"].astype(np.float64) @ W.astype(np.float64).T
    assert np.max(np.abs(g["C"] - ref)) / np.max(np.abs(ref)) < 1e-5

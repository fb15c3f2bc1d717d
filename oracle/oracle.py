"""CPU oracle for the Stream-K GEMM hot path.  TEST INFRASTRUCTURE ONLY.

Two independent statements of the same arithmetic live here so each can pin the other:

* ``liboracle.so`` (``streamk_oracle.c``): plain-C restatement of the reference partitioner, the
  per-CTA segment loop with both fix-up flavours, and the Q4 dequantisation.
* numpy / pure-Python twins in this file (``partition_py``, ``cta_segments_py``, ``dequant_q4_np``).

Reference lines followed (relative to the LeiWang1999/Stream-k.tvm checkout):
  partition       streamk_fp32.py:33-54
  CTA range       streamk_fp32.py:93-96
  segment loop    streamk_fp32.py:98-136, triton_impl.py:104-127
  DP loop         streamk_fp32.py:149-158
  Q4 order        streamk.fp16.breakdown/streamk_fp16_ladder_block_reduce_q4.py:552
  host check      streamk_fp32.py:204-208 (dense matmul, rtol = atol = 1e-2)

Nothing here is ever used by the product path; the product raises when its HIP library is missing.
"""
import ctypes
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


class _Partition(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int) for n in (
        "num_block_m", "num_block_n", "iters_per_tile", "total_tiles", "streamk_tiles",
        "blocking_tiles", "streamk_iters", "streamk_full_tiles", "streamk_partial_tiles",
        "sm_partition_factor")]


def build():
    """Compile liboracle.so with gcc (a second or two)."""
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.ora_partition.argtypes = [ctypes.c_int] * 7 + [ctypes.POINTER(_Partition)]
        L.ora_partition.restype = None
        L.ora_cta_range.argtypes = [ctypes.POINTER(_Partition), ctypes.c_int,
                                    ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int)]
        L.ora_cta_range.restype = None
        L.ora_streamk_gemm_f32.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 8 + [
            ctypes.c_void_p, ctypes.c_int]
        L.ora_streamk_gemm_f32.restype = ctypes.c_int
        L.ora_dequant_q4.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 4
        L.ora_dequant_q4.restype = None
        L.ora_half_to_float.argtypes = [ctypes.c_uint16]
        L.ora_half_to_float.restype = ctypes.c_float
        L.ora_float_to_half.argtypes = [ctypes.c_float]
        L.ora_float_to_half.restype = ctypes.c_uint16
        _LIB = L
    return _LIB


# ------------------------------------------------------------------ partition (C and Python twins)
def partition(M, N, K, BM, BN, BK, P):
    """C restatement of streamk_fp32.py:33-54 -> dict."""
    p = _Partition()
    lib().ora_partition(M, N, K, BM, BN, BK, P, ctypes.byref(p))
    return {n: getattr(p, n) for n, _ in _Partition._fields_}


def partition_py(M, N, K, BM, BN, BK, P):
    """Pure-Python twin of streamk_fp32.py:33-54 (factor = blocking_tiles // P, 0 allowed)."""
    nbm, nbn, ipt = math.ceil(M / BM), math.ceil(N / BN), math.ceil(K / BK)
    total = nbm * nbn
    sk = total % P
    if total - sk > P:
        sk += P
    dp = total - sk
    it = sk * ipt
    return dict(num_block_m=nbm, num_block_n=nbn, iters_per_tile=ipt, total_tiles=total,
                streamk_tiles=sk, blocking_tiles=dp, streamk_iters=it, streamk_full_tiles=it // P,
                streamk_partial_tiles=it % P, sm_partition_factor=dp // P)


def cta_range(part, pid):
    p = _Partition(**part)
    s, e = ctypes.c_int(), ctypes.c_int()
    lib().ora_cta_range(ctypes.byref(p), pid, ctypes.byref(s), ctypes.byref(e))
    return s.value, e.value


def cta_segments_py(part, pid):
    """Segments (tile, k0, n_iters, whole) a CTA walks in its Stream-K wave
    (streamk_fp32.py:93-136), pure Python."""
    full, partial, ipt = (part["streamk_full_tiles"], part["streamk_partial_tiles"],
                          part["iters_per_tile"])
    start = pid * full + min(pid, partial)
    last = (pid + 1) * full + min(pid + 1, partial)
    out = []
    while start < last:
        end = min(start + (ipt - start % ipt), last)
        k0 = start % ipt
        out.append((start // ipt, k0, end - start, k0 == 0 and end % ipt == 0))
        start = end
    return out


def dp_tiles_py(part, pid, P):
    """Tiles of the data-parallel phase for one CTA (streamk_fp32.py:149-150)."""
    return [pid + part["streamk_tiles"] + p * P for p in range(part["sm_partition_factor"])]


# ------------------------------------------------------------------ Stream-K GEMM on the CPU
def streamk_gemm_f32(A, B, BM, BN, BK, P, trans_b=False, cta_order=None, fixup="atomic"):
    """Runs the reference's persistent kernel with P simulated CTAs (C restatement).
    A [M,K] float32; B [K,N] (trans_b False) or [N,K] (trans_b True).  Returns C float32."""
    A = np.ascontiguousarray(A, dtype=np.float32)
    B = np.ascontiguousarray(B, dtype=np.float32)
    M, K = A.shape
    N = B.shape[0] if trans_b else B.shape[1]
    assert (B.shape[1] if trans_b else B.shape[0]) == K
    C = np.zeros((M, N), dtype=np.float32)  # pre-zero contract, streamk_fp32.py:200
    order = None
    if cta_order is not None:
        order = np.ascontiguousarray(cta_order, dtype=np.int32)
        assert sorted(order.tolist()) == list(range(P))
    rc = lib().ora_streamk_gemm_f32(A.ctypes.data, B.ctypes.data, C.ctypes.data, M, N, K,
                                    int(trans_b), BM, BN, BK, P,
                                    order.ctypes.data if order is not None else None,
                                    {"atomic": 0, "reduce": 1}[fixup])
    if rc:
        raise ValueError("ora_streamk_gemm_f32 rejected its arguments")
    return C


def matmul_fp32(A, B, trans_b=False):
    """The reference's dense check (streamk_fp32.py:204, streamk_fp16.py:389) on the host in fp32:
    inputs are widened to float32 first, as block_level_gemm.py:92-103 does."""
    A = np.asarray(A, dtype=np.float32)
    B = np.asarray(B, dtype=np.float32)
    return A @ (B.T if trans_b else B)


def max_abs_rel(got, ref):
    """max |got - ref| / max |ref|  (the 'max-abs-rel' figure quoted for GEMM accuracy)."""
    got = np.asarray(got, dtype=np.float64)
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.max(np.abs(got - ref)) / max(float(np.max(np.abs(ref))), 1e-30))


# ------------------------------------------------------------------ Q4
def unpack_q4_np(Wq):
    """[N, K/2] uint8 -> [N, K] uint8 nibbles; low nibble is the even k
    (streamk_fp16_ladder_block_reduce_q4.py:552)."""
    Wq = np.asarray(Wq, dtype=np.uint8)
    out = np.empty((Wq.shape[0], Wq.shape[1] * 2), dtype=np.uint8)
    out[:, 0::2] = Wq & 0xF
    out[:, 1::2] = Wq >> 4
    return out


def pack_q4_np(q):
    """[N, K] nibbles -> [N, K/2] bytes, the array streamk_fp16_ladder_block_reduce_q4.py:552 expands
    (element k in bits 4*(k&1).. of byte k/2)."""
    q = np.asarray(q, dtype=np.uint8)
    assert q.max(initial=0) <= 15
    return (q[:, 0::2] | (q[:, 1::2] << 4)).astype(np.uint8)


def quantize_q4_np(W, group=128, zero=8):
    """Group-wise quantisation rule of this build (the reference draws random nibbles and has no
    quantiser): scale = fp16(max|w| / levels), q = clamp(rint(w / scale) + zero, 0, 15), fp32
    divisions; levels = min(zero, 15 - zero) or 15 if that is 0; q = zero where scale is 0.
    Returns (Wq [N, K/2] uint8, scales [N, K/group] float16)."""
    W = np.asarray(W, dtype=np.float16)
    N, K = W.shape
    levels = min(zero, 15 - zero) or 15
    w = W.astype(np.float32).reshape(N, K // group, group)
    amax = np.abs(w).max(axis=2)
    sc = (amax / np.float32(levels)).astype(np.float16)
    s = sc.astype(np.float32)[:, :, None]
    with np.errstate(divide="ignore", invalid="ignore"):
        q = np.rint(w / s) + np.float32(zero)
    q = np.where(s == 0, np.float32(zero), np.clip(q, 0, 15)).astype(np.uint8).reshape(N, K)
    return pack_q4_np(q), sc


def dequant_q4_np(Wq, scales, group=128, zero=8):
    """numpy float16 evaluation: w = fp16((fp16(q) - fp16(zero)) * scale[n, k // group])."""
    q = unpack_q4_np(Wq).astype(np.float16)
    d = q - np.float16(zero)
    s = np.repeat(np.asarray(scales, dtype=np.float16), group, axis=1)[:, :q.shape[1]]
    return (d * s).astype(np.float16)


def dequant_q4(Wq, scales, group=128, zero=8):
    """C restatement (software binary16 rounding), returns float16 [N, K]."""
    Wq = np.ascontiguousarray(Wq, dtype=np.uint8)
    N, K = Wq.shape[0], Wq.shape[1] * 2
    sc = np.ascontiguousarray(scales, dtype=np.float16)
    assert sc.shape == (N, math.ceil(K / group)), sc.shape
    out = np.empty((N, K), dtype=np.float16)
    lib().ora_dequant_q4(Wq.ctypes.data, sc.ctypes.data, out.ctypes.data, N, K, group, zero)
    return out


def q4_gemm_ref(A, Wq, scales, group=128, zero=8):
    """fp32 host product of A [M,K] with the dequantised weights [N,K]^T."""
    W = dequant_q4(Wq, scales, group, zero).astype(np.float32)
    return np.asarray(A, dtype=np.float32) @ W.T


# ------------------------------------------------------------------ fp8 (OCP e4m3)
def f8e4m3_decode(u8):
    """Bytes -> float32 values of the OCP 8-bit floating point format E4M3 (OCP 8-bit Floating Point
    Specification (OFP8) rev 1.0, section 5: sign, 4 exponent bits with bias 7, 3 mantissa bits; no
    infinities; S.1111.111 is NaN; exponent 0 is subnormal, m * 2^-9).  Not in the reference's scripts,
    which stop at fp16; its Triton comparator takes the dtype of its inputs (triton.streamk/first_wave.py:123)."""
    u8 = np.asarray(u8, dtype=np.uint8)
    e = ((u8 >> 3) & 15).astype(np.int32)
    m = (u8 & 7).astype(np.float32)
    mag = np.where(e == 0, np.ldexp(m, -9), np.ldexp(8.0 + m, e - 10)).astype(np.float32)
    mag = np.where((e == 15) & ((u8 & 7) == 7), np.float32(np.nan), mag)
    return np.where(u8 >> 7 == 1, -mag, mag).astype(np.float32)


def f8e5m2_decode(u8):
    """Bytes -> float32 values of the OCP format E5M2 (OFP8 rev 1.0, section 5: sign, 5 exponent bits with bias 15,
    2 mantissa bits, IEEE-style infinities and NaNs): the upper byte of an IEEE binary16 number."""
    u8 = np.asarray(u8, dtype=np.uint8)
    return (u8.astype(np.uint16) << 8).view(np.float16).astype(np.float32)


def f8_gemm_ref(A_u8, B_u8, fmt="e4m3"):
    """float64 host product A [M,K] x B [N,K]^T of fp8 bytes, both e4m3 or both e5m2 (each product of two fp8
    values is exact in float32; the sum is taken in float64)."""
    dec = f8e4m3_decode if fmt == "e4m3" else f8e5m2_decode
    return dec(A_u8).astype(np.float64) @ dec(B_u8).astype(np.float64).T


def i8_gemm_ref(A_i8, B_i8):
    """Exact integer product A [M,K] x B [N,K]^T of int8 operands (int64 on the host; the device accumulates
    in int32 like the reference's Triton comparator, triton.streamk/first_wave.py:123, which is the same
    number while |sum| < 2^31)."""
    A = np.asarray(A_i8)
    B = np.asarray(B_i8)
    assert A.dtype == np.int8 and B.dtype == np.int8
    return A.astype(np.int64) @ B.astype(np.int64).T


# ------------------------------------------------------------------ Q4 with one zero point per group and row
def dequant_q4_zp_np(Wq, scales, zeros, group=128):
    """w = fp16((fp16(q) - z[n, k // group]) * scale[n, k // group]) in numpy float16 arithmetic; z holds
    integers 0..15.  With a constant z this is dequant_q4_np / ora_dequant_q4 at that zero point (tested),
    which follow streamk.fp16.breakdown/streamk_fp16_ladder_block_reduce_q4_atomic.py:280-282."""
    q = unpack_q4_np(Wq).astype(np.float16)
    z = np.repeat(np.asarray(zeros, dtype=np.float16), group, axis=1)[:, :q.shape[1]]
    s = np.repeat(np.asarray(scales, dtype=np.float16), group, axis=1)[:, :q.shape[1]]
    return ((q - z) * s).astype(np.float16)


def quantize_q4_zp_np(W, group=128):
    """Asymmetric group-wise rule of this build (the reference has no quantiser): lo = min(min w, 0),
    hi = max(max w, 0); scale = fp16((hi - lo) / 15); z = clip(rint(-lo / scale), 0, 15);
    q = clip(rint(w / scale) + z, 0, 15); scale 0: z = q = 0.  fp32 arithmetic.
    Returns (Wq [N, K/2] uint8, scales, zeros [N, K/group] float16)."""
    W = np.asarray(W, dtype=np.float16)
    N, K = W.shape
    w = W.astype(np.float32).reshape(N, K // group, group)
    lo = np.minimum(w.min(axis=2), np.float32(0))
    hi = np.maximum(w.max(axis=2), np.float32(0))
    sc = ((hi - lo) / np.float32(15)).astype(np.float16)
    s = sc.astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        z = np.where(s == 0, np.float32(0), np.clip(np.rint(-lo / s), 0, 15)).astype(np.float32)
        q = np.rint(w / s[:, :, None]) + z[:, :, None]
    q = np.where(s[:, :, None] == 0, np.float32(0), np.clip(q, 0, 15)).astype(np.uint8).reshape(N, K)
    return pack_q4_np(q), sc, z.astype(np.float16)


def q4_zp_gemm_ref(A, Wq, scales, zeros, group=128):
    """fp32 host product of A [M,K] with the dequantised weights [N,K]^T."""
    W = dequant_q4_zp_np(Wq, scales, zeros, group).astype(np.float32)
    return np.asarray(A, dtype=np.float32) @ W.T


def activation_ref(x, name):
    """Epilogue activations in float64 on a numpy array: 'relu' max(x, 0); 'gelu_tanh'
    0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) (the tanh form of GELU, Hendrycks & Gimpel 2016, eq. 2);
    'silu' x / (1 + exp(-x)); None / 'none' the identity.  No counterpart in the reference, whose kernels end
    at the store of C; pinned in tests/test_oracle_gemm.py against torch's CPU routines and the erf form."""
    x = np.asarray(x, dtype=np.float64)
    if name in (None, "none"):
        return x
    if name == "relu":
        return np.maximum(x, 0.0)
    if name == "gelu_tanh":
        return 0.5 * x * (1.0 + np.tanh(np.sqrt(2.0 / np.pi) * (x + 0.044715 * x ** 3)))
    if name == "silu":
        with np.errstate(over="ignore"):
            return x / (1.0 + np.exp(-x))
    raise ValueError(f"unknown activation {name!r}")

"""Python-facing Stream-K GEMM entry points over the C ABI.

Mirrors the reference's operator surface:
  * `streamk_fp16(A, B)` / `streamk_fp32(A, B)`: what running streamk_fp16.py / streamk_fp32.py
    computes (C = A @ B.T for the fp16 NT script, C = A @ B for the fp32 NN script);
  * `tl_matmul_streamk(M, N, K, ...)` returns a callable `kernel(A, B, C)` that writes C in place,
    the shape of the reference's `tl_mod = TL.Profiler(...)`; `tl_mod(A, B, b_c)`
    (streamk_fp16.py:382-387), including `do_bench`.
torch is used for device memory and streams only.
"""
import ctypes

import torch

from . import _lib
from .plan import make_plan

_workspaces = {}


def _stream_ptr():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _workspace(nbytes, device):
    """One self-cleaning workspace per (device, stream), grown on demand and zeroed once."""
    if nbytes == 0:
        return None
    key = (device.index if device.index is not None else torch.cuda.current_device(),
           torch.cuda.current_stream().cuda_stream)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _lib.check(_lib.lib().sk_workspace_init(ws.data_ptr(), ws.numel(), _stream_ptr()),
                   "sk_workspace_init")
        _workspaces[key] = ws
    return ws


def reset_workspaces():
    """Drops cached workspaces (needed after a StreamKError with status SK_ERR_TIMEOUT)."""
    _workspaces.clear()


def workspace_status():
    """SK_OK / raises if any fix-up wait on the current stream's workspace timed out."""
    for (dev, stream), ws in _workspaces.items():
        if stream == torch.cuda.current_stream().cuda_stream:
            _lib.check(_lib.lib().sk_workspace_status(ws.data_ptr(), _stream_ptr()), "sk_workspace_status")


def _check_matrix(t, name, dtype):
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError(f"{name} must be a CUDA/HIP tensor")
    if t.dtype != dtype:
        raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{name} must be 2-D with unit stride along its last dimension")


def _epilogue(bias, N, dtype, device, activation=None):
    """sk_epilogue for a bias vector (N values of C's type on C's device) and / or an activation
    ('relu', 'gelu_tanh', 'silu'), or None when there is neither."""
    if activation not in _lib.ACTIVATIONS:
        raise ValueError(f"activation must be one of {sorted(k for k in _lib.ACTIVATIONS if k)} or None")
    act = _lib.ACTIVATIONS[activation]
    if bias is None:
        return _lib.SkEpilogue(bias=None, activation=act) if act else None
    if not isinstance(bias, torch.Tensor) or bias.dtype != dtype or bias.dim() != 1 or bias.shape[0] != N \
            or not bias.is_contiguous() or bias.device != device:
        raise ValueError(f"bias must be a contiguous {dtype} vector of {N} elements on {device}")
    return _lib.SkEpilogue(bias=bias.data_ptr(), activation=act)


def streamk_fp16(A, B, *, Wq=None, scales=None, layout="nt", out=None, plan=None, config=None,
                 zero=8, group=128, bias=None, activation=None, **kw):
    """C = A @ B.T (layout 'nt', B is [N,K]) or A @ B (layout 'nn', B is [K,N]) in fp16 with fp32
    accumulation.

    With `Wq` (uint8 [N, K/2], low nibble = even k) and `scales` (fp16 [N, K/group]) the weights
    are dequantised on the fly, w = fp16((q - zero) * scale), and B is ignored (pass None).
    `config`/kwargs: bm, bn, bk, grid, schedule, fixup, raster (see plan.make_config).
    `bias` (fp16 [N]) is added to every row in fp32 before the rounding to fp16; `activation`
    ('relu', 'gelu_tanh', 'silu') is applied after it, also in fp32.
    """
    if Wq is not None:
        return streamk_q4(A, Wq, scales, out=out, plan=plan, config=config, zero=zero, group=group, bias=bias,
                          activation=activation, **kw)
    _check_matrix(A, "A", torch.float16)
    _check_matrix(B, "B", torch.float16)
    if layout not in ("nt", "nn"):
        raise ValueError("layout must be 'nt' (B is [N,K]) or 'nn' (B is [K,N])")
    M, K = A.shape
    N, Kb = B.shape if layout == "nt" else (B.shape[1], B.shape[0])
    if K != Kb:
        raise ValueError(f"K mismatch: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if plan is None:
        plan = make_plan(M, N, K, "float16", layout, config, **kw)
    C = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=A.device)
    _check_matrix(C, "out", torch.float16)
    if tuple(C.shape) != (M, N):
        raise ValueError("out has the wrong shape")
    ws = _workspace(plan.workspace_bytes, A.device)
    epi = _epilogue(bias, N, torch.float16, A.device, activation)
    args = (A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0), C.stride(0),
            ctypes.byref(plan), ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _stream_ptr())
    rc = _lib.lib().sk_gemm_f16(*args) if epi is None else _lib.lib().sk_gemm_f16_ex(*args, ctypes.byref(epi))
    _lib.check(rc, "sk_gemm_f16")
    return C


def streamk_bf16(A, B, *, layout="nt", out=None, plan=None, config=None, bias=None, activation=None, **kw):
    """streamk_fp16 for bfloat16 operands and output (fp32 accumulation, C rounded to nearest even).
    The reference's scripts are fp16 / fp32 only; this is the bfloat16 instance of the same tile
    kernels."""
    _check_matrix(A, "A", torch.bfloat16)
    _check_matrix(B, "B", torch.bfloat16)
    if layout not in ("nt", "nn"):
        raise ValueError("layout must be 'nt' (B is [N,K]) or 'nn' (B is [K,N])")
    M, K = A.shape
    N, Kb = B.shape if layout == "nt" else (B.shape[1], B.shape[0])
    if K != Kb:
        raise ValueError(f"K mismatch: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if plan is None:
        plan = make_plan(M, N, K, "bfloat16", layout, config, **kw)
    C = out if out is not None else torch.empty((M, N), dtype=torch.bfloat16, device=A.device)
    _check_matrix(C, "out", torch.bfloat16)
    if tuple(C.shape) != (M, N):
        raise ValueError("out has the wrong shape")
    ws = _workspace(plan.workspace_bytes, A.device)
    epi = _epilogue(bias, N, torch.bfloat16, A.device, activation)
    args = (A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0), C.stride(0),
            ctypes.byref(plan), ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _stream_ptr())
    rc = _lib.lib().sk_gemm_bf16(*args) if epi is None else _lib.lib().sk_gemm_bf16_ex(*args, ctypes.byref(epi))
    _lib.check(rc, "sk_gemm_bf16")
    return C


def streamk_fp8(A, B, *, alpha=1.0, fmt=None, out=None, plan=None, config=None, bias=None, activation=None, **kw):
    """C = activation(alpha * (A @ B.T) + bias) for fp8 operands, A [M,K], B [N,K]; fp32 accumulation, alpha applied to the
    fp32 sums, fp16 C.  Both operands are OCP e4m3 (torch.float8_e4m3fn) or both OCP e5m2
    (torch.float8_e5m2); raw uint8 bytes are taken as `fmt` ("e4m3" by default, or "e5m2").  alpha is the
    product of the per-tensor scales of a scaled-fp8 caller; bias (fp16 [N]) and activation as for
    streamk_fp16, applied after alpha.  The reference's scripts stop at fp16; this is
    the same partitioner and fix-ups over the fp8 form of the tile kernel."""
    kinds = {getattr(torch, "float8_e4m3fn", None): "e4m3", getattr(torch, "float8_e5m2", None): "e5m2"}
    for t, name in ((A, "A"), (B, "B")):
        if not isinstance(t, torch.Tensor) or (t.dtype != torch.uint8 and t.dtype not in kinds):
            raise TypeError(f"{name} must be a float8_e4m3fn / float8_e5m2 (or uint8) tensor")
        _check_matrix(t, name, t.dtype)
        if t.dtype != torch.uint8:
            if fmt not in (None, kinds[t.dtype]):
                raise TypeError("A and B must be in the same fp8 format")
            fmt = kinds[t.dtype]
    fmt = fmt or "e4m3"
    if fmt not in ("e4m3", "e5m2"):
        raise ValueError("fmt must be 'e4m3' or 'e5m2'")
    M, K = A.shape
    N, Kb = B.shape
    if K != Kb:
        raise ValueError(f"K mismatch: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if plan is None:
        plan = make_plan(M, N, K, "float8_" + fmt, "nt", config, **kw)
    elif plan.dtype != (_lib.SK_F8E5M2 if fmt == "e5m2" else _lib.SK_F8E4M3):
        raise ValueError("the plan was made for the other fp8 format")
    C = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=A.device)
    _check_matrix(C, "out", torch.float16)
    if tuple(C.shape) != (M, N):
        raise ValueError("out has the wrong shape")
    ws = _workspace(plan.workspace_bytes, A.device)
    epi = _epilogue(bias, N, torch.float16, A.device, activation)
    args = (A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0), B.stride(0), C.stride(0), float(alpha),
            ctypes.byref(plan), ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _stream_ptr())
    rc = _lib.lib().sk_gemm_f8(*args) if epi is None else _lib.lib().sk_gemm_f8_ex(*args, ctypes.byref(epi))
    _lib.check(rc, "sk_gemm_f8")
    return C


def streamk_int8(A, B, *, out=None, plan=None, config=None, **kw):
    """C = A @ B.T for int8 operands, A [M,K], B [N,K]; exact int32 accumulation, int32 C (the accumulator
    type the reference's Triton comparator picks for integer inputs, triton.streamk/first_wave.py:123).
    Every schedule and fix-up returns the same bits."""
    _check_matrix(A, "A", torch.int8)
    _check_matrix(B, "B", torch.int8)
    M, K = A.shape
    N, Kb = B.shape
    if K != Kb:
        raise ValueError(f"K mismatch: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if plan is None:
        plan = make_plan(M, N, K, "int8", "nt", config, **kw)
    C = out if out is not None else torch.empty((M, N), dtype=torch.int32, device=A.device)
    _check_matrix(C, "out", torch.int32)
    if tuple(C.shape) != (M, N):
        raise ValueError("out has the wrong shape")
    ws = _workspace(plan.workspace_bytes, A.device)
    rc = _lib.lib().sk_gemm_i8(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0),
                               B.stride(0), C.stride(0), ctypes.byref(plan),
                               ws.data_ptr() if ws is not None else None,
                               ws.numel() if ws is not None else 0, _stream_ptr())
    _lib.check(rc, "sk_gemm_i8")
    return C


Q4_MAX_M = 64  # rows of A the Q4 kernels take in one launch


def tile_q4(Wq):
    """Packed weights Wq[N, K/2] -> the tiled layout (16 rows x 64 bytes per tile, [row block][group]),
    on the device Wq lives on.  Returns a [ceil(N/16)*16, K/2] array (rows past N are zero) to pass to
    streamk_q4(..., tiled=True); the weights then stream faster and the results are the same bit
    for bit.  The counterpart of the reference's offline weight transformation
    (streamk_fp16_ladder_block_reduce_q4.py:568-580)."""
    if Wq.dtype != torch.uint8 or Wq.dim() != 2 or not Wq.is_contiguous():
        raise ValueError("Wq must be a contiguous 2-D uint8 tensor")
    N, K = Wq.shape[0], Wq.shape[1] * 2
    out = torch.empty(((N + 15) // 16 * 16, K // 2), dtype=torch.uint8, device=Wq.device)
    if Wq.is_cuda:
        _lib.check(_lib.lib().sk_q4_tile(Wq.data_ptr(), N, K, out.data_ptr(), _stream_ptr()), "sk_q4_tile")
    else:
        _lib.check(_lib.lib().sk_q4_tile_host(Wq.data_ptr(), N, K, out.data_ptr()), "sk_q4_tile_host")
    return out


def untile_q4(tiled, N):
    """Inverse of tile_q4 for host tensors: the row-major Wq[N, K/2]."""
    if tiled.dtype != torch.uint8 or tiled.dim() != 2 or tiled.is_cuda or not tiled.is_contiguous():
        raise ValueError("tiled must be a contiguous 2-D uint8 tensor in host memory")
    K = tiled.shape[1] * 2
    if tiled.shape[0] != (N + 15) // 16 * 16:
        raise ValueError("tiled has ceil(N/16)*16 rows")
    Wq = torch.empty((N, K // 2), dtype=torch.uint8)
    _lib.check(_lib.lib().sk_q4_untile_host(tiled.data_ptr(), N, K, Wq.data_ptr()), "sk_q4_untile_host")
    return Wq


def _zero_points(zeros, scales):
    """Per-group zero points as the library takes them: fp16 [N, K/group] holding integers 0..15.  Integer
    tensors are converted (an allocation per call: keep them as fp16 to avoid it)."""
    if zeros.dtype != torch.float16:
        zeros = zeros.to(torch.float16)
    _check_matrix(zeros, "zeros", torch.float16)
    if tuple(zeros.shape) != tuple(scales.shape) or not zeros.is_contiguous():
        raise ValueError(f"zeros must be contiguous and shaped like scales; got {tuple(zeros.shape)}")
    return zeros


def streamk_q4(A, Wq, scales, *, out=None, plan=None, config=None, zero=8, group=128, tiled=False, zeros=None,
               bias=None, activation=None, **kw):
    """C[M,N] fp16 = A[M,K] fp16 @ dequant(Wq)[N,K].T, weights in natural nibble order
    (streamk_fp16_ladder_block_reduce_q4.py:552).  tiled=True: Wq is the output of tile_q4 (N is
    then taken from scales).  zeros: one zero point per scale group and row ([N, K/group], integers
    0..15) instead of the scalar `zero`.  bias / activation: as for streamk_fp16."""
    if zeros is not None:
        if tiled:
            raise ValueError("per-group zero points need the row-major weights")
        zeros = _zero_points(zeros, scales)
    _check_matrix(A, "A", torch.float16)
    _check_matrix(Wq, "Wq", torch.uint8)
    _check_matrix(scales, "scales", torch.float16)
    M, K = A.shape
    N = scales.shape[0] if tiled else Wq.shape[0]
    if Wq.shape[1] * 2 != K or not Wq.is_contiguous() or (tiled and Wq.shape[0] != (N + 15) // 16 * 16):
        raise ValueError(f"Wq must be contiguous [N, K/2] (tiled: ceil(N/16)*16 rows); got {tuple(Wq.shape)} for K={K}")
    if tuple(scales.shape) != (N, K // group) or not scales.is_contiguous():
        raise ValueError(f"scales must be contiguous [N, K/group]; got {tuple(scales.shape)}")
    if plan is not None and (plan.dtype == _lib.SK_Q4_TILED) != bool(tiled):
        raise ValueError("the plan was made for the other weight layout")
    if plan is not None and (plan.dtype == _lib.SK_Q4_ZP) != (zeros is not None):
        raise ValueError("the plan was made with / without per-group zero points")
    C = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=A.device)
    _check_matrix(C, "out", torch.float16)
    if tuple(C.shape) != (M, N):
        raise ValueError("out has the wrong shape")
    if plan is None and M > Q4_MAX_M:
        # the Q4 kernels stream the weights past at most 64 rows of A.  Up to 256 rows: one launch
        # per block of 64 rows.  Beyond: dequantise once (bit-exact device function) and run the
        # fp16 tile kernels, whose time then dwarfs the extra pass over the weights.
        if M <= 4 * Q4_MAX_M:
            for m0 in range(0, M, Q4_MAX_M):
                streamk_q4(A[m0:m0 + Q4_MAX_M], Wq, scales, out=C[m0:m0 + Q4_MAX_M], config=config, zero=zero,
                           group=group, tiled=tiled, zeros=zeros, bias=bias, activation=activation, **kw)
            return C
        if tiled:
            raise ValueError("more than 256 rows of A need the row-major weights (they are dequantised once)")
        return streamk_fp16(A, dequant_q4(Wq, scales, zero=zero, group=group, zeros=zeros), out=C, bias=bias,
                            activation=activation)
    if plan is None:
        plan = make_plan(M, N, K, "q4_zp" if zeros is not None else ("q4_tiled" if tiled else "q4"), "nt", config, **kw)
    ws = _workspace(plan.workspace_bytes, A.device)
    epi = _epilogue(bias, N, torch.float16, A.device, activation)
    tail = (ctypes.byref(plan), ws.data_ptr() if ws is not None else None, ws.numel() if ws is not None else 0,
            _stream_ptr())
    L = _lib.lib()
    if epi is not None:
        rc = L.sk_gemm_q4_ex(A.data_ptr(), Wq.data_ptr(), scales.data_ptr(), zeros.data_ptr() if zeros is not None else None,
                             C.data_ptr(), M, N, K, A.stride(0), C.stride(0), group, zero, *tail, ctypes.byref(epi))
    elif zeros is not None:
        rc = L.sk_gemm_q4_zp(A.data_ptr(), Wq.data_ptr(), scales.data_ptr(), zeros.data_ptr(), C.data_ptr(), M, N, K,
                             A.stride(0), C.stride(0), group, *tail)
    else:
        rc = L.sk_gemm_q4(A.data_ptr(), Wq.data_ptr(), scales.data_ptr(), C.data_ptr(), M, N, K, A.stride(0),
                          C.stride(0), group, zero, *tail)
    _lib.check(rc, "sk_gemm_q4")
    return C


def dequant_q4(Wq, scales, *, zero=8, group=128, zeros=None):
    """fp16 W[N,K] from packed nibbles, by the same device function the Q4 GEMM uses."""
    _check_matrix(Wq, "Wq", torch.uint8)
    _check_matrix(scales, "scales", torch.float16)
    N, K = Wq.shape[0], Wq.shape[1] * 2
    if not Wq.is_contiguous() or not scales.is_contiguous():
        raise ValueError("Wq and scales must be contiguous")
    W = torch.empty((N, K), dtype=torch.float16, device=Wq.device)
    if zeros is not None:
        zeros = _zero_points(zeros, scales)
        rc = _lib.lib().sk_dequant_q4_zp(Wq.data_ptr(), scales.data_ptr(), zeros.data_ptr(), W.data_ptr(), N, K,
                                         group, _stream_ptr())
        _lib.check(rc, "sk_dequant_q4_zp")
        return W
    rc = _lib.lib().sk_dequant_q4(Wq.data_ptr(), scales.data_ptr(), W.data_ptr(), N, K, group, zero,
                                  _stream_ptr())
    _lib.check(rc, "sk_dequant_q4")
    return W


def pack_q4(q):
    """Wq[N, K/2] from q[N, K] (uint8 values 0..15, host memory): element k of a row goes to nibble
    k & 1 of byte k / 2, the order streamk_fp16_ladder_block_reduce_q4.py:552 expands.  This is the
    array the kernels read: there is no further permutation step (the reference's :568-595)."""
    if q.dtype != torch.uint8 or q.dim() != 2 or q.is_cuda or not q.is_contiguous():
        raise ValueError("q must be a contiguous 2-D uint8 tensor in host memory")
    N, K = q.shape
    Wq = torch.empty((N, K // 2), dtype=torch.uint8)
    _lib.check(_lib.lib().sk_q4_pack_host(q.data_ptr(), N, K, Wq.data_ptr()), "sk_q4_pack_host")
    return Wq


def unpack_q4(Wq):
    """Inverse of pack_q4 (host memory)."""
    if Wq.dtype != torch.uint8 or Wq.dim() != 2 or Wq.is_cuda or not Wq.is_contiguous():
        raise ValueError("Wq must be a contiguous 2-D uint8 tensor in host memory")
    N, K = Wq.shape[0], Wq.shape[1] * 2
    q = torch.empty((N, K), dtype=torch.uint8)
    _lib.check(_lib.lib().sk_q4_unpack_host(Wq.data_ptr(), N, K, q.data_ptr()), "sk_q4_unpack_host")
    return q


def quantize_q4(W, *, group=128, zero=8, asymmetric=False):
    """(Wq[N, K/2] uint8, scales[N, K/group] fp16) from fp16 W[N, K], on the device W lives on.
    scale = fp16(max|w| / levels) per group, q = clamp(rint(w / scale) + zero, 0, 15).
    asymmetric=True: each group's range [min(w, 0), max(w, 0)] is mapped onto 0..15 with its own zero
    point; returns (Wq, scales, zeros[N, K/group] fp16) for streamk_q4(..., zeros=zeros)."""
    if W.dtype != torch.float16 or W.dim() != 2 or W.stride(1) != 1:
        raise ValueError("W must be a 2-D fp16 tensor with unit stride along K")
    N, K = W.shape
    ldw = W.stride(0) if N > 1 else K  # the stride of a single row is arbitrary
    Wq = torch.empty((N, K // 2), dtype=torch.uint8, device=W.device)
    sc = torch.empty((N, K // max(group, 1)), dtype=torch.float16, device=W.device)
    if asymmetric:
        zp = torch.empty_like(sc)
        if W.is_cuda:
            rc = _lib.lib().sk_q4_quantize_zp(W.data_ptr(), N, K, ldw, group, Wq.data_ptr(), sc.data_ptr(),
                                              zp.data_ptr(), _stream_ptr())
        else:
            rc = _lib.lib().sk_q4_quantize_zp_host(W.data_ptr(), N, K, ldw, group, Wq.data_ptr(), sc.data_ptr(),
                                                   zp.data_ptr())
        _lib.check(rc, "sk_q4_quantize_zp")
        return Wq, sc, zp
    if W.is_cuda:
        rc = _lib.lib().sk_q4_quantize(W.data_ptr(), N, K, ldw, group, zero, Wq.data_ptr(), sc.data_ptr(),
                                       _stream_ptr())
        _lib.check(rc, "sk_q4_quantize")
    else:
        rc = _lib.lib().sk_q4_quantize_host(W.data_ptr(), N, K, ldw, group, zero, Wq.data_ptr(),
                                            sc.data_ptr())
        _lib.check(rc, "sk_q4_quantize_host")
    return Wq, sc


def streamk_fp32(A, B, *, layout="nn", out=None, plan=None, config=None, **kw):
    """C = A @ B in fp32 (layout 'nn', B is [K,N]: streamk_fp32.py:65-76)."""
    _check_matrix(A, "A", torch.float32)
    _check_matrix(B, "B", torch.float32)
    if layout not in ("nt", "nn"):
        raise ValueError("layout must be 'nn' (B is [K,N]) or 'nt' (B is [N,K])")
    M, K = A.shape
    N, Kb = (B.shape[1], B.shape[0]) if layout == "nn" else B.shape
    if K != Kb:
        raise ValueError(f"K mismatch: A is {tuple(A.shape)}, B is {tuple(B.shape)}")
    if plan is None:
        plan = make_plan(M, N, K, "float32", layout, config, **kw)
    C = out if out is not None else torch.empty((M, N), dtype=torch.float32, device=A.device)
    _check_matrix(C, "out", torch.float32)
    ws = _workspace(plan.workspace_bytes, A.device)
    rc = _lib.lib().sk_gemm_f32(A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, A.stride(0),
                                B.stride(0), C.stride(0), ctypes.byref(plan),
                                ws.data_ptr() if ws is not None else None,
                                ws.numel() if ws is not None else 0, _stream_ptr())
    _lib.check(rc, "sk_gemm_f32")
    return C


class StreamKKernel:
    """A planned GEMM, callable as `kernel(A, B, C)` (C written in place), the role of the
    reference's compiled `tl_mod` (streamk_fp32.py:197-202)."""

    def __init__(self, M, N, K, dtype, layout, plan):
        self.M, self.N, self.K, self.dtype, self.layout, self.plan = M, N, K, dtype, layout, plan

    def __call__(self, A, B, C):
        if self.dtype == "float16":
            return streamk_fp16(A, B, layout=self.layout, out=C, plan=self.plan)
        return streamk_fp32(A, B, layout=self.layout, out=C, plan=self.plan)

    def do_bench(self, fn=None, warmup=25, rep=100):
        """Mean milliseconds per call over `rep` back-to-back launches after `warmup`
        (streamk_fp16.py:394)."""
        if fn is None:
            dt = torch.float16 if self.dtype == "float16" else torch.float32
            A = torch.randn(self.M, self.K, device="cuda", dtype=dt)
            bshape = (self.N, self.K) if self.layout == "nt" else (self.K, self.N)
            B = torch.randn(*bshape, device="cuda", dtype=dt)
            C = torch.empty(self.M, self.N, device="cuda", dtype=dt)
            fn = lambda: self(A, B, C)  # noqa: E731
        return bench_ms(fn, warmup, rep)


def bench_ms(fn, warmup=25, rep=100):
    for _ in range(warmup):
        fn()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(rep):
        fn()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) / rep


def tl_matmul_streamk(M, N, K, *, dtypeAB="float16", layout=None, block_M=None, block_N=None,
                      block_K=None, streamk_programs=None, schedule="auto", fixup="auto", raster=0):
    """Factory with the reference's name and role (streamk_fp32.py:57-72, streamk_fp16.py:116-124):
    fixes shape, tile and partition, returns the in-place kernel callable."""
    if layout is None:
        layout = "nt" if dtypeAB == "float16" else "nn"
    plan = make_plan(M, N, K, dtypeAB, layout, bm=block_M, bn=block_N, bk=block_K,
                     grid=streamk_programs, schedule=schedule, fixup=fixup, raster=raster)
    return StreamKKernel(M, N, K, dtypeAB, layout, plan)

"""ctypes binding of libstreamk.so (the C ABI declared in include/streamk.h).

The library is mandatory: there is no Python or CPU fallback for any GEMM entry point.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libstreamk.so")

SK_F16, SK_F32, SK_Q4, SK_BF16, SK_Q4_TILED, SK_F8E4M3, SK_I8, SK_Q4_ZP, SK_F8E5M2, SK_Q4_ZP_TILED = 0, 1, 2, 3, 4, 5, 6, 7, 8, 9
LAYOUT_NT, LAYOUT_NN = 0, 1
SCHEDULES = {"auto": 0, "dp": 1, "sk2": 2, "sk1": 3, "basic": 4, "splitk": 5}
FIXUPS = {"auto": 0, "atomic": 1, "reduce": 2, "atomic_c": 3, "reduce16": 4}


class SkConfig(ctypes.Structure):
    _fields_ = [("bm", ctypes.c_int32), ("bn", ctypes.c_int32), ("bk", ctypes.c_int32),
                ("grid", ctypes.c_int32), ("schedule", ctypes.c_int32), ("fixup", ctypes.c_int32),
                ("raster", ctypes.c_int32), ("spin_limit", ctypes.c_int32),
                ("reserved", ctypes.c_int32 * 4)]


class SkPlan(ctypes.Structure):
    _fields_ = [(n, ctypes.c_int32) for n in (
        "bm", "bn", "bk", "grid", "schedule", "fixup", "raster", "dtype", "layout",
        "num_block_m", "num_block_n", "iters_per_tile", "total_tiles", "streamk_tiles",
        "blocking_tiles", "streamk_iters", "streamk_full_tiles", "streamk_partial_tiles",
        "dp_waves", "kernel_id", "threads", "lds_bytes", "spin_limit", "interleave")] + [
        ("workspace_bytes", ctypes.c_int64), ("M", ctypes.c_int64), ("N", ctypes.c_int64),
        ("K", ctypes.c_int64)]

    def as_dict(self):
        return {n: getattr(self, n) for n, _ in self._fields_}


# sk_activation
ACTIVATIONS = {None: 0, "none": 0, "relu": 1, "gelu_tanh": 2, "silu": 3}


class SkEpilogue(ctypes.Structure):
    """sk_epilogue: optional operands of the *_ex entry points."""
    _fields_ = [("bias", ctypes.c_void_p), ("activation", ctypes.c_int64), ("reserved", ctypes.c_int64 * 2)]


class StreamKError(RuntimeError):
    def __init__(self, status, where):
        self.status = status
        super().__init__(f"{where}: {strerror(status)} (status {status})")


_lib = None


def lib():
    """Loads libstreamk.so.  torch is imported first so that the library binds to the HIP runtime
    torch already carries (one runtime per process: streams and pointers are shared)."""
    global _lib
    if _lib is not None:
        return _lib
    import torch  # noqa: F401  (must precede the dlopen)
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `make -C stream-k.tvm_amd/csrc` "
            "(or __graft_entry__.build()); there is no fallback path")
    L = ctypes.CDLL(LIB_PATH)
    i64, vp, ci, sz = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    P = ctypes.POINTER
    L.sk_version.restype = ci
    L.sk_strerror.argtypes = [ci]
    L.sk_strerror.restype = ctypes.c_char_p
    L.sk_kernel_name.argtypes = [ci]
    L.sk_kernel_name.restype = ctypes.c_char_p
    L.sk_device_info.argtypes = [P(ci), P(ci), P(ci)]
    L.sk_make_plan.argtypes = [i64, i64, i64, ci, ci, P(SkConfig), ci, P(SkPlan)]
    L.sk_plan_cta_range.argtypes = [P(SkPlan), ci, P(ctypes.c_int32), P(ctypes.c_int32)]
    L.sk_plan_tile_coords.argtypes = [P(SkPlan), ci, P(ctypes.c_int32), P(ctypes.c_int32)]
    L.sk_workspace_bytes.argtypes = [P(SkPlan)]
    L.sk_workspace_bytes.restype = sz
    L.sk_workspace_init.argtypes = [vp, sz, vp]
    L.sk_workspace_status.argtypes = [vp, vp]
    L.sk_workspace_release.argtypes = [vp]
    L.sk_workspace_release.restype = ci
    L.sk_gemm_f16.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp, sz, vp]
    L.sk_gemm_f32.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp, sz, vp]
    L.sk_gemm_f16_static.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp]
    L.sk_gemm_f16_static.restype = ci
    L.sk_static_init.argtypes = []
    L.sk_static_init.restype = ci
    L.sk_gemm_bf16.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp, sz, vp]
    L.sk_gemm_bf16.restype = ci
    L.sk_gemm_q4_zp.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, ci, P(SkPlan), vp, sz, vp]
    L.sk_gemm_q4_zp.restype = ci
    L.sk_dequant_q4_zp.argtypes = [vp, vp, vp, vp, i64, i64, ci, vp]
    L.sk_dequant_q4_zp.restype = ci
    L.sk_q4_quantize_zp_host.argtypes = [vp, i64, i64, i64, ci, vp, vp, vp]
    L.sk_q4_quantize_zp_host.restype = ci
    L.sk_q4_quantize_zp.argtypes = [vp, i64, i64, i64, ci, vp, vp, vp, vp]
    L.sk_q4_quantize_zp.restype = ci
    L.sk_gemm_f16_ex.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp, sz, vp, P(SkEpilogue)]
    L.sk_gemm_f16_ex.restype = ci
    L.sk_gemm_bf16_ex.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp, sz, vp, P(SkEpilogue)]
    L.sk_gemm_bf16_ex.restype = ci
    L.sk_gemm_q4_ex.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, ci, ci, P(SkPlan), vp, sz, vp, P(SkEpilogue)]
    L.sk_gemm_q4_ex.restype = ci
    L.sk_gemm_f8.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ctypes.c_float, P(SkPlan), vp, sz, vp]
    L.sk_gemm_f8.restype = ci
    L.sk_gemm_f8_ex.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, ctypes.c_float, P(SkPlan), vp, sz, vp, P(SkEpilogue)]
    L.sk_gemm_f8_ex.restype = ci
    L.sk_gemm_i8.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, P(SkPlan), vp, sz, vp]
    L.sk_gemm_i8.restype = ci
    L.sk_gemm_q4.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i64, ci, ci, P(SkPlan), vp, sz, vp]
    L.sk_dequant_q4.argtypes = [vp, vp, vp, i64, i64, ci, ci, vp]
    L.sk_q4_pack_host.argtypes = [vp, i64, i64, vp]
    L.sk_q4_unpack_host.argtypes = [vp, i64, i64, vp]
    L.sk_q4_quantize_host.argtypes = [vp, i64, i64, i64, ci, ci, vp, vp]
    L.sk_q4_quantize.argtypes = [vp, i64, i64, i64, ci, ci, vp, vp, vp]
    L.sk_q4_tile_host.argtypes = [vp, i64, i64, vp]
    L.sk_q4_untile_host.argtypes = [vp, i64, i64, vp]
    L.sk_q4_tile.argtypes = [vp, i64, i64, vp, vp]
    for f in ("sk_q4_pack_host", "sk_q4_unpack_host", "sk_q4_quantize_host", "sk_q4_quantize", "sk_q4_tile_host",
              "sk_q4_untile_host", "sk_q4_tile"):
        getattr(L, f).restype = ci
    for f in ("sk_device_info", "sk_make_plan", "sk_plan_cta_range", "sk_plan_tile_coords",
              "sk_workspace_init", "sk_workspace_status", "sk_gemm_f16", "sk_gemm_f32",
              "sk_gemm_q4", "sk_dequant_q4"):
        getattr(L, f).restype = ci
    _lib = L
    return L


def kernel_name(kernel_id):
    name = lib().sk_kernel_name(kernel_id)
    return name.decode() if name else None


def strerror(status):
    return lib().sk_strerror(status).decode()


def check(status, where):
    if status != 0:
        raise StreamKError(status, where)

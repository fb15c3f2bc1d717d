"""Host partitioner front-end: the integers of streamk_fp32.py:30-54 for a run-time shape."""
import ctypes

from . import _lib
from ._lib import SkConfig, SkPlan

_DTYPES = {"float16": _lib.SK_F16, "float32": _lib.SK_F32, "q4": _lib.SK_Q4, "bfloat16": _lib.SK_BF16,
           "q4_tiled": _lib.SK_Q4_TILED, "float8_e4m3": _lib.SK_F8E4M3, "float8_e5m2": _lib.SK_F8E5M2,
           "int8": _lib.SK_I8, "q4_zp": _lib.SK_Q4_ZP, "q4_zp_tiled": _lib.SK_Q4_ZP_TILED}
_LAYOUTS = {"nt": _lib.LAYOUT_NT, "nn": _lib.LAYOUT_NN}
_num_cus = None


def num_cus():
    """Compute units of the current device (the reference hard-codes total_sm = 108,
    streamk_fp32.py:17)."""
    global _num_cus
    if _num_cus is None:
        n = ctypes.c_int()
        _lib.check(_lib.lib().sk_device_info(ctypes.byref(n), None, None), "sk_device_info")
        _num_cus = n.value
    return _num_cus


def make_config(config=None, **kw):
    """dict / kwargs -> SkConfig.  Keys: bm, bn, bk, grid, schedule ('auto'|'dp'|'sk2'|'sk1'|
    'basic'|'splitk'), split, fixup ('auto'|'atomic'|'reduce'|'atomic_c'|'reduce16'), raster, spin_limit, variant, interleave."""
    d = dict(config or {})
    d.update(kw)
    c = SkConfig()
    for k, v in d.items():
        if v is None:
            continue
        if k == "schedule":
            v = _lib.SCHEDULES[v] if isinstance(v, str) else int(v)
        elif k == "fixup":
            v = _lib.FIXUPS[v] if isinstance(v, str) else int(v)
        if k == "variant":  # 0 = newest kernel variant of the tile, v > 0 = variant v - 1
            c.reserved[0] = int(v)
            continue
        if k == "split":  # factor of schedule 'splitk'; 0 = choose
            c.reserved[1] = int(v)
            continue
        if k == "interleave":  # 1: interleaved order of the Stream-K tiles (sk_plan.interleave)
            c.reserved[2] = int(v)
            continue
        if k not in ("bm", "bn", "bk", "grid", "schedule", "fixup", "raster", "spin_limit"):
            raise KeyError(f"unknown Stream-K config key {k!r}")
        setattr(c, k, int(v))
    return c


_tuned = None


_tuned_generation = 0


def invalidate_tuned_cache():
    """Forget the loaded tuned cache (the autotuner calls this when it has written an entry).  Plans that other
    layers made from the old cache are told apart by tuned_generation()."""
    global _tuned, _tuned_generation
    _tuned = None
    _tuned_generation += 1


def tuned_generation():
    """Counts the invalidations of the tuned cache: part of the key of every cache of plans made from it."""
    return _tuned_generation


def tuned_config(M, N, K, dtype="float16", layout="nt"):
    """Configuration the autotuner recorded for exactly this problem, or None."""
    global _tuned
    if _tuned is None:
        from .autotune import load_cache
        _tuned = load_cache()
    hit = _tuned.get(f"gfx950/{dtype}/{layout}/{M}x{N}x{K}")
    if not hit:
        return None
    cfg = dict(hit["config"])
    if cfg.get("raster") == 0:   # recorded as "row-major was fastest"; 0 now means "library default"
        cfg["raster"] = 1
    return cfg


_TWIN_OF = {"bfloat16": "float16", "float8_e5m2": "float8_e4m3"}


def make_plan(M, N, K, dtype="float16", layout="nt", config=None, cus=None, use_tuned=True, **kw):
    """Partition an M x N x K GEMM.  `cus` overrides the device's CU count (lets the partitioner
    run without a GPU).  With no configuration given, a tuned one from the autotune cache is used
    when there is one for this exact problem, else the library heuristic."""
    kw = {k: v for k, v in kw.items() if v is not None}
    if use_tuned and not config and not kw and cus is None:
        config = tuned_config(M, N, K, dtype, layout)
        if config is None and dtype in _TWIN_OF:
            # the bfloat16 kernels are twins of the fp16 ones, the e5m2 kernels of the e4m3 ones (same data
            # movement, same MFMA rate): a shape tuned for the other type only takes that entry, where the kernel
            # it names has a twin
            borrowed = tuned_config(M, N, K, _TWIN_OF[dtype], layout)
            if borrowed is not None:
                try:
                    return make_plan(M, N, K, dtype, layout, borrowed)
                except _lib.StreamKError:
                    pass
    cfg = make_config(config, **kw)
    plan = SkPlan()
    rc = _lib.lib().sk_make_plan(M, N, K, _DTYPES[dtype], _LAYOUTS[layout], ctypes.byref(cfg),
                                 cus if cus is not None else num_cus(), ctypes.byref(plan))
    _lib.check(rc, f"sk_make_plan({M},{N},{K},{dtype},{layout},{kw or config})")
    return plan


def cta_range(plan, pid):
    s, e = ctypes.c_int32(), ctypes.c_int32()
    _lib.check(_lib.lib().sk_plan_cta_range(ctypes.byref(plan), pid, ctypes.byref(s), ctypes.byref(e)),
               "sk_plan_cta_range")
    return s.value, e.value


def tile_coords(plan, tile):
    m, n = ctypes.c_int32(), ctypes.c_int32()
    _lib.check(_lib.lib().sk_plan_tile_coords(ctypes.byref(plan), tile, ctypes.byref(m), ctypes.byref(n)),
               "sk_plan_tile_coords")
    return m.value, n.value

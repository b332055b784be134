"""ctypes binding of libfp8bs.so (C ABI declared in include/fp8bs.h).

There is no fallback: if the library has not been built the import of the entry points fails
loudly, so a GPU run can never silently take another path.
"""
import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libfp8bs.so")

# Every symbol include/fp8bs.h declares.
EXPORTS = (
    "fp8bs_version", "fp8bs_strerror", "fp8bs_plan", "fp8bs_workspace_bytes",
    "fp8bs_gemm", "fp8bs_gemm_ex", "fp8bs_gemm_noalloc", "fp8bs_gemm_grouped", "fp8bs_gemm_grouped_ex",
    "fp8bs_quantize_a", "fp8bs_quantize_b", "fp8bs_gather_a",
    "fp8bs_moe_topk", "fp8bs_moe_route_workspace_bytes", "fp8bs_moe_route",
    "fp8bs_gemm_silu_mul", "fp8bs_moe_combine", "fp8bs_convert_fnuz_to_fn", "fp8bs_diag_mfma_mix",
)

VARIANT_NAMES = {0: "auto", 1: "generic", 2: "t256x256", 3: "t128x128", 4: "t64x128", 5: "t256x128", 6: "skinny64x144", 7: "skinny64x256", 8: "skinny64x288", 9: "t256x192", 10: "t256x128s3", 11: "t192x192s3", 12: "t64x256s3"}


class Plan(ctypes.Structure):
    """Mirror of fp8bs_plan_t."""
    _fields_ = [
        ("variant", ctypes.c_int32), ("tile_m", ctypes.c_int32), ("tile_n", ctypes.c_int32),
        ("split_k", ctypes.c_int32), ("grid_x", ctypes.c_int32), ("grid_y", ctypes.c_int32),
        ("grid_z", ctypes.c_int32), ("block_threads", ctypes.c_int32), ("lds_bytes", ctypes.c_int32),
        ("stream_k", ctypes.c_int32), ("sum_in_kernel", ctypes.c_int32), ("reserved", ctypes.c_int32),
        ("workspace_bytes", ctypes.c_uint64),
    ]


SPLIT_SUM_IN_KERNEL = 1 << 30        # FP8BS_SPLIT_SUM_IN_KERNEL
MIN_VERSION = 300                    # fp8bs_version() of the first library whose fp8bs_plan_t has sum_in_kernel


_lib = None


def load() -> ctypes.CDLL:
    """Load the library once; raise RuntimeError if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            "libfp8bs.so is not built (%s missing): run `python __graft_entry__.py` or "
            "`python amd-developer-challenge-2025_amd/build.py`; there is no fallback path" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    vp, i32, sz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    lib.fp8bs_version.restype = i32
    lib.fp8bs_version.argtypes = []
    if lib.fp8bs_version() < MIN_VERSION:
        # an older build fills a shorter fp8bs_plan_t than the Plan mirrored here
        raise RuntimeError("%s is version %d, this package needs %d or later: rebuild it with "
                           "`python amd-developer-challenge-2025_amd/build.py`" % (LIB_PATH, lib.fp8bs_version(), MIN_VERSION))
    lib.fp8bs_strerror.restype = ctypes.c_char_p
    lib.fp8bs_strerror.argtypes = [i32]
    lib.fp8bs_plan.restype = i32
    lib.fp8bs_plan.argtypes = [i32, i32, i32, i32, ctypes.POINTER(Plan)]
    lib.fp8bs_workspace_bytes.restype = sz
    lib.fp8bs_workspace_bytes.argtypes = [i32, i32, i32]
    lib.fp8bs_gemm.restype = i32
    lib.fp8bs_gemm.argtypes = [vp, vp, vp, vp, vp, vp, sz, i32, i32, i32, vp]
    lib.fp8bs_gemm_noalloc.restype = i32
    lib.fp8bs_gemm_noalloc.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32, vp]
    lib.fp8bs_gemm_ex.restype = i32
    lib.fp8bs_gemm_ex.argtypes = [vp, vp, vp, vp, vp, vp, sz, i32, i32, i32, i32, i32, vp]
    lib.fp8bs_gemm_grouped.restype = i32
    lib.fp8bs_gemm_grouped.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]
    lib.fp8bs_gemm_grouped_ex.restype = i32
    lib.fp8bs_gemm_grouped_ex.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]
    i64 = ctypes.c_int64
    lib.fp8bs_quantize_a.restype = i32
    lib.fp8bs_quantize_a.argtypes = [vp, i32, i64, vp, i32, vp, vp, i32, i32, vp]
    lib.fp8bs_quantize_b.restype = i32
    lib.fp8bs_quantize_b.argtypes = [vp, i32, i64, vp, vp, i32, i32, vp]
    lib.fp8bs_gather_a.restype = i32
    lib.fp8bs_gather_a.argtypes = [vp, vp, i32, vp, vp, vp, i32, i32, vp]
    lib.fp8bs_moe_topk.restype = i32
    lib.fp8bs_moe_topk.argtypes = [vp, i32, i32, i32, vp, vp]
    lib.fp8bs_moe_route_workspace_bytes.restype = sz
    lib.fp8bs_moe_route_workspace_bytes.argtypes = [i32, i32]
    lib.fp8bs_moe_route.restype = i32
    lib.fp8bs_moe_route.argtypes = [vp, i32, i32, i32, vp, vp, vp, vp, sz, vp]
    lib.fp8bs_gemm_silu_mul.restype = i32
    lib.fp8bs_gemm_silu_mul.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, vp]
    lib.fp8bs_moe_combine.restype = i32
    lib.fp8bs_moe_combine.argtypes = [vp, i32, vp, vp, vp, i32, i32, i32, vp]
    lib.fp8bs_convert_fnuz_to_fn.restype = i32
    lib.fp8bs_convert_fnuz_to_fn.argtypes = [vp, vp, sz, vp]
    lib.fp8bs_diag_mfma_mix.restype = i32
    lib.fp8bs_diag_mfma_mix.argtypes = [i32, i32, i32, vp, sz, vp, vp]
    _lib = lib
    return lib


_pycall = False


def pycall():
    """The CPython binding of fp8bs_gemm_ex / fp8bs_gemm_grouped_ex (csrc/fp8bs_pycall.c: the same library
    functions without ctypes' per-argument marshalling), or None where it has not been built or cannot be
    imported (one warning); callers then use the ctypes functions of load().  Either way the work is done by libfp8bs.so, which has no substitute."""
    global _pycall
    if _pycall is False:
        load()                                        # the library must be there first; raises if it is not
        path = os.path.join(HERE, "_fp8bs_pycall.so")
        _pycall = None
        if os.path.exists(path):
            import importlib.machinery
            import importlib.util
            try:
                loader = importlib.machinery.ExtensionFileLoader("_fp8bs_pycall", path)
                spec = importlib.util.spec_from_file_location("_fp8bs_pycall", path, loader=loader)
                mod = importlib.util.module_from_spec(spec)
                loader.exec_module(mod)
                _pycall = mod
            except (ImportError, OSError) as ex:      # built for another Python, or its libfp8bs.so cannot be resolved
                import warnings
                warnings.warn("_fp8bs_pycall.so cannot be imported (%s); binding libfp8bs.so through ctypes instead" % ex)
    return _pycall


def check(status: int) -> None:
    """Raise RuntimeError with the library's message for a non-zero status."""
    if status != 0:
        raise RuntimeError("fp8bs: %s (status %d)" % (load().fp8bs_strerror(status).decode(), status))

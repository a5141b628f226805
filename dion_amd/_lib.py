"""ctypes binding of libdion_hip.so (the C ABI declared in include/dion_hip.h).

The library is loaded lazily and never built here: `python -m dion_amd._build` (or
`__graft_entry__.build()`) produces it.  A missing library is a hard error -- there is no
fallback implementation behind these entry points.
"""
import ctypes  # noqa: F401  (re-exported for callers building C arrays)
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libdion_hip.so")

DION_BF16 = 0
DION_F32 = 1
DION_NS_GRAM = 1
DION_NS_STATIC_SCRATCH_BYTES = 64 << 20
ABI_VERSION = 12  # dion_abi_version() of the library these signatures describe

_u64p = ctypes.POINTER(ctypes.c_uint64)
_i64p = ctypes.POINTER(ctypes.c_int64)
_f32p = ctypes.POINTER(c_float)

# name -> (restype, argtypes); mirrors include/dion_hip.h one to one.
SIGNATURES = {
    "dion_last_error": (c_char_p, []),
    "dion_abi_version": (c_int, []),
    "dion_ns_line_1": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "dion_ns_line_2": (c_int, [c_void_p, c_void_p, c_int, c_int, c_float, c_float, c_void_p]),
    "dion_ns_line_3": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_void_p]),
    "dion_ns_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "dion_ns_orthogonalize": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, _f32p, c_int,
                                      c_float, c_float, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "dion_ns_orthogonalize_static": (c_int, [c_void_p, c_int, c_void_p, c_int, c_int, c_int, _f32p, c_int,
                                             c_float, c_float, c_int, c_int, c_void_p]),
    "dion_ns_plan_audit": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_size_t]),
    "dion_ns_update_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "dion_ns_orthogonalize_update": (c_int, [c_void_p, c_int, _u64p, c_int, c_int, c_int, c_int, c_int, _f32p,
                                             c_int, c_float, c_float, c_int, c_int, c_void_p, c_float, c_void_p,
                                             c_float, c_int, c_void_p, c_size_t, c_void_p]),
    "dion_ns_accepts_prepared": (c_int, [c_int, c_int, c_int, c_int, c_int]),
    "dion_ns_orthogonalize_prepared": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, _f32p,
                                               c_int, c_float, c_float, c_int, c_int, c_void_p, c_size_t,
                                               c_void_p]),
    "dion_ns_orthogonalize_update_prepared": (c_int, [c_void_p, c_void_p, c_int, _u64p, c_int, c_int, c_int, c_int,
                                                      c_int, _f32p, c_int, c_float, c_float, c_int, c_int, c_void_p,
                                                      c_float, c_void_p, c_float, c_int, c_void_p, c_size_t,
                                                      c_void_p]),
    "dion_ns_plan_audit_prepared": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                            c_size_t]),
    "dion_gemm_tile_edge": (c_int, [c_int, c_int, c_int, c_int]),
    "dion_muon_pre_sumsq_blocks": (c_int, [c_int, c_int]),
    "dion_muon_pre_prepared": (c_int, [_u64p, c_int, _u64p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                       c_float, c_int, c_void_p]),
    "dion_muon_pre": (c_int, [_u64p, c_int, _u64p, c_int, c_void_p, c_int, c_int64, c_float, c_int, c_void_p]),
    "dion_scale_rows": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int, c_void_p]),
    "dion_muon_post": (c_int, [_u64p, c_int, c_void_p, c_int, c_int, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                               c_float, c_void_p, c_float, c_int, c_void_p]),
    "dion_normuon_stats": (c_int, [c_void_p, _u64p, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p,
                                   c_void_p]),
    "dion_normuon_stats_selected": (c_int, [c_void_p, _u64p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                            c_float, c_void_p, c_void_p]),
    "dion_dion2_accumulate_scratch_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "dion_dion2_accumulate": (c_int, [_u64p, c_int, _u64p, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_void_p, c_void_p, c_size_t, c_void_p]),
    "dion_dion2_topk": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "dion_dion2_gather": (c_int, [_u64p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float,
                                  c_void_p, c_void_p]),
    "dion_dion2_gather_sumsq_blocks": (c_int, [c_int, c_int, c_int, c_int]),
    "dion_dion2_gather_prepared": (c_int, [_u64p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_float,
                                           c_void_p, c_void_p, c_void_p]),
    "dion_dion2_post": (c_int, [_u64p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_void_p,
                                c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_float, c_void_p]),
    "dion_dion2_index_map": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "dion_slice_l1": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "dion_gather_slices": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p,
                                   c_void_p]),
    "dion_scatter_slices": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p,
                                    c_void_p]),
    "dion_mask_index": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "dion_dion2_post_masked": (c_int, [_u64p, _u64p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                       c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_float, c_float,
                                       c_void_p]),
    "dion_adamw_step": (c_int, [_u64p, _u64p, c_int, _u64p, _u64p, c_int, _u64p, _i64p, c_int, c_void_p, c_float,
                                c_float, c_float, c_void_p, c_float, c_int, c_void_p]),
    "dion_lion_step": (c_int, [_u64p, _u64p, c_int, _u64p, c_int, _i64p, c_int, c_void_p, c_float, c_float,
                               c_void_p, c_float, c_int, c_void_p]),
}

_lib = None


class DionHipError(RuntimeError):
    """A libdion_hip.so entry point returned a failure code."""


def load() -> ctypes.CDLL:
    """Load the shared library and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is missing: the HIP extension has not been built. "
            "Run `python -m dion_amd._build` (needs hipcc)."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    built = lib.dion_abi_version()
    if built != ABI_VERSION:
        raise ImportError(
            f"{LIB_PATH} was built with ABI version {built}, this binding describes version {ABI_VERSION}: "
            "rebuild it with `python -m dion_amd._build`."
        )
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().dion_last_error().decode("utf-8", "replace")
        if rc == -1:
            raise ValueError(f"{what}: {msg}")
        raise DionHipError(f"{what} failed ({rc}): {msg}")


def ptr_table(ptrs):
    """Host array of device pointers for the *_ptrs arguments."""
    return (ctypes.c_uint64 * len(ptrs))(*ptrs)

"""ctypes binding of libfastmoe_hip.so (the C ABI declared in include/fast_moe_amd.h).

The library is loaded from the package directory; there is no fallback: if it is
missing or a symbol cannot be resolved, importing an operator fails loudly.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_size_t, c_uint8, c_void_p

_PKG_DIR = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
# (FMOE_LIB_PATH: another build of the same library, e.g. the -DFMOE_TRACE debug build)
LIB_PATH = os.environ.get("FMOE_LIB_PATH") or os.path.join(_PKG_DIR, "libfastmoe_hip.so")

FMOE_F32, FMOE_BF16, FMOE_E4M3 = 0, 1, 2
EPI_NONE, EPI_SILU, EPI_SWIGLU, EPI_GATED = 0, 1, 2, 3
PLAN_NONE, PLAN_RING, PLAN_STAGED, PLAN_STAGED_SHORT, PLAN_ELEMENT = -1, 0, 1, 2, 3

# every symbol include/fast_moe_amd.h declares
EXPORTED_SYMBOLS = (
    "fmoe_version", "fmoe_last_error", "fmoe_route_workspace_bytes", "fmoe_route_topk",
    "fmoe_route_from_topk", "fmoe_quant_rows_e4m3", "fmoe_grouped_gemm", "fmoe_grouped_gemm_plan",
    "fmoe_combine",
    "fmoe_silu_mul", "fmoe_transpose_last2", "fmoe_jagged_transpose", "fmoe_segment_colsum",
    "fmoe_swiglu_bwd", "fmoe_combine_bwd", "fmoe_gather_rows", "fmoe_route_topk_static", "fmoe_hbm_probe",
)
ROUTE_STATIC_MAX_POSITIONS, ROUTE_STATIC_MAX_EXPERTS = 1 << 20, 512


class GemmDesc(ctypes.Structure):
    """struct fmoe_gemm_desc, field for field."""
    _fields_ = [
        ("num_experts", c_int32), ("n", c_int32), ("k", c_int32), ("index_div", c_int32),
        ("total_rows", c_int64), ("a_rows", c_int64),
        ("offsets", c_void_p), ("row_index", c_void_p),
        ("a", c_void_p), ("a_dtype", c_int32), ("a_silu", c_int32),
        ("a_stride_row", c_int64), ("a_stride_e", c_int64), ("a_scale", c_void_p),
        ("b", c_void_p), ("b2", c_void_p),
        ("b_stride_e", c_int64), ("b_stride_k", c_int64), ("b_stride_n", c_int64),
        ("b_scale", c_void_p), ("b2_scale", c_void_p),
        ("bias", c_void_p), ("bias2", c_void_p), ("bias_stride_e", c_int64),
        ("epilogue", c_int32), ("out_dtype", c_int32),
        ("out", c_void_p), ("out_stride_row", c_int64),
        ("k_window", c_void_p),
        ("k_window_multiple", c_int32),
        ("k_slack_rows", c_int32),
        ("aux", c_void_p),
        ("aux2", c_void_p),
        ("aux_stride_row", c_int64),
        ("a_stride_k", c_int64),
        ("a2", c_void_p), ("k2", c_int32), ("scale_pow2", c_int32), ("out2", c_void_p),
    ]


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m fast_moe_amd.build` "
            f"(hipcc --offload-arch=gfx950); fast_moe_amd has no fallback path")
    lib = ctypes.CDLL(LIB_PATH)
    lib.fmoe_version.restype = c_int
    lib.fmoe_version.argtypes = []
    lib.fmoe_last_error.restype = c_char_p
    lib.fmoe_last_error.argtypes = []
    lib.fmoe_route_workspace_bytes.restype = c_size_t
    lib.fmoe_route_workspace_bytes.argtypes = [c_int64, c_int, c_int]
    lib.fmoe_route_topk.restype = c_int
    lib.fmoe_route_topk.argtypes = [c_void_p, c_int, c_int64, c_int, c_int, c_int] + [c_void_p] * 7 + [
        c_void_p, c_size_t, c_void_p]
    lib.fmoe_route_topk_static.restype = c_int
    lib.fmoe_route_topk_static.argtypes = [c_void_p, c_int, c_int64, c_int, c_int, c_int] + [c_void_p] * 7 + [c_void_p]
    lib.fmoe_route_from_topk.restype = c_int
    lib.fmoe_route_from_topk.argtypes = [c_void_p, c_int64, c_int, c_int] + [c_void_p] * 6 + [
        c_void_p, c_size_t, c_void_p]
    lib.fmoe_quant_rows_e4m3.restype = c_int
    lib.fmoe_quant_rows_e4m3.argtypes = [c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64,
                                         c_int64, c_int, c_void_p, c_int64, c_int64, c_int64, c_void_p,
                                         c_int, c_void_p]
    lib.fmoe_grouped_gemm.restype = c_int
    lib.fmoe_grouped_gemm.argtypes = [POINTER(GemmDesc), c_void_p]
    lib.fmoe_grouped_gemm_plan.restype = c_int
    lib.fmoe_grouped_gemm_plan.argtypes = [POINTER(GemmDesc), POINTER(c_int)]
    lib.fmoe_combine.restype = c_int
    lib.fmoe_combine.argtypes = [c_void_p, c_int, c_int64, c_int, c_int64, c_int64, c_void_p, c_void_p,
                                 c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p]
    lib.fmoe_silu_mul.restype = c_int
    lib.fmoe_silu_mul.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_void_p]
    lib.fmoe_transpose_last2.restype = c_int
    lib.fmoe_transpose_last2.argtypes = [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_int64,
                                         c_void_p]
    lib.fmoe_jagged_transpose.restype = c_int
    lib.fmoe_jagged_transpose.argtypes = [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p,
                                          c_void_p, c_int, c_void_p, c_int64, c_int64, c_int, c_void_p]
    lib.fmoe_segment_colsum.restype = c_int
    lib.fmoe_segment_colsum.argtypes = [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p,
                                        c_void_p]
    lib.fmoe_gather_rows.restype = c_int
    lib.fmoe_gather_rows.argtypes = [c_void_p, c_int64, c_int64, c_int64, c_void_p, c_int, c_int64, c_void_p,
                                     c_int64, c_void_p]
    lib.fmoe_swiglu_bwd.restype = c_int
    lib.fmoe_swiglu_bwd.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64,
                                    c_int64, c_void_p]
    lib.fmoe_combine_bwd.restype = c_int
    lib.fmoe_combine_bwd.argtypes = [c_void_p, c_void_p, c_int, c_int64, c_int, c_int64, c_int64, c_void_p,
                                     c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
                                     c_void_p]
    lib.fmoe_hbm_probe.restype = c_int
    lib.fmoe_hbm_probe.argtypes = [c_void_p, c_int64, c_int, c_int, c_void_p]
    _lib = lib
    return lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().fmoe_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (status {rc}): {msg}")

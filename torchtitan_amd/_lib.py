"""ctypes binding of the C ABI declared in include/mxfp8.h.

The library is built in-tree by torchtitan_amd._build (hipcc, gfx950).  There is no CPU
fallback: if the shared object is missing, loading raises.
"""
from __future__ import annotations

import ctypes
from ctypes import c_int, c_int64, c_void_p, c_char_p
from pathlib import Path

import os

# MXFP8_LIBRARY names another build of the same library (a measurement variant made by
# `python -m torchtitan_amd._build --define ... --out ...`); unset, the in-tree product library.
LIB_PATH = Path(os.environ.get("MXFP8_LIBRARY") or Path(__file__).resolve().parent / "libmxfp8_gfx950.so").resolve()

MX_SCALE_FLOOR = 0
MX_SCALE_RCEIL = 1
MX_SCALES_ROWMAJOR = 0
MX_SCALES_MFMA = 1

_P = c_void_p
_I = c_int64

# name -> (restype, argtypes); mirrors include/mxfp8.h one to one
SIGNATURES = {
    "mx_version": (c_int, []),
    "mx_status_string": (c_char_p, [c_int]),
    "mx_scales_mfma_bytes": (_I, [_I, _I]),
    "mx_cast_dim0": (c_int, [_P, _I, _I, _I, _P, _P, c_int, c_int, _P]),
    "mx_cast_dim1": (c_int, [_P, _I, _I, _I, _P, _P, c_int, c_int, _P]),
    "mx_cast_dim0_dim1": (c_int, [_P, _I, _I, _I, _P, _P, _P, _P, c_int, c_int, _P]),
    "mx_cast_dim0_dim1_ld": (c_int, [_P, _I, _I, _I, _P, _I, _P, _P, _I, _P, c_int, c_int, _P]),
    "mx_cast_dim1_batched": (c_int, [_P, _I, _I, _I, _I, _P, _P, c_int, c_int, _P]),
    "mx_cast_dim0_dim1_batched": (c_int, [_P, _I, _I, _I, _I, _P, _P, _P, _P, c_int, c_int, _P]),
    "mx_cast_rows_gathered": (c_int, [_P, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, c_int, c_int, _P]),
    "mx_dequant": (c_int, [_P, _P, _I, _I, c_int, _P, _I, _P]),
    "mx_token_logprob_fwd": (c_int, [_P, _I, _I, _I, _P, _P, _P, _P]),
    "mx_token_logprob_bwd": (c_int, [_P, _I, _I, _I, _P, _P, _P, _P, _I, _P]),
    "mx_moe_route_plan": (c_int, [_P, _I, _P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P]),
    "mx_moe_combine": (c_int, [_P, _P, _I, _I, _P, _P, _I, _I, _I, _P, _I, _P]),
    "mx_moe_row_dot": (c_int, [_P, _P, _I, _I, _P, _P, _I, _I, _P, _I, _I, _P, _P]),
    "mx_rmsnorm_cast_dim0_dim1": (c_int, [_P, _P, ctypes.c_float, _I, _I, _I, _P, _P, _P, _P, _P, _P, c_int, c_int, _P]),
    "mx_rmsnorm_cast_dim0_dim1_ld": (c_int, [_P, _P, ctypes.c_float, _I, _I, _I, _P, _P, _P, _I, _P, _P, _I, _P, c_int, c_int, _P]),
    "mx_swiglu_cast_dim0_dim1_ld": (c_int, [_P, _P, _I, _I, _I, _I, _P, _I, _P, _P, _I, _P, _P, c_int, c_int, _P]),
    "mx_swiglu_bwd_cast_dim0_dim1_ld": (c_int, [_P, _P, _P, _I, _I, _I, _I, _I, _P, _I, _P, _P, _I, _P, _P, c_int, c_int, _P]),
    "mx_swiglu_cast_dim0_dim1": (c_int, [_P, _P, _I, _I, _I, _I, _P, _P, _P, _P, _P, c_int, c_int, _P]),
    "mx_swiglu_bwd_cast_dim0_dim1": (c_int, [_P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _P, _P, _P, c_int, c_int, _P]),
    "mx_scale_layout": (c_int, [_P, _I, _I, _P, _P]),
    "mx_scale_unlayout": (c_int, [_P, _I, _I, _P, _P]),
    "mx_gemm_nt": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_workspace_bytes": (_I, [_I, _I, _I]),
    "mx_gemm_nt_ws": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P, _I, _P]),
    "mx_gemm_nt_ld": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _I, _P]),
    "mx_gemm_nt_static_max_bytes": (_I, []),
    "mx_gemm_nt_static": (c_int, [_P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_pair": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_pair_ld": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_shared_a_ld": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_shared_b_ld": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_shared_a": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mx_gemm_nt_shared_b": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mx_grouped_gemm_2d3d_shared_a": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mx_grouped_gemm_2d2d_shared_b": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P]),
    "mx_grouped_gemm_2d3d_rows_out": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _P]),
    "mx_grouped_gemm_2d3d_pair": (c_int, [_P, _P, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P]),
    "mx_grouped_gemm_2d3d": (c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, c_int, _P]),
    "mx_grouped_gemm_2d2d": (c_int, [_P, _P, _P, _P, _P, _P, _I, _I, _I, _I, c_int, _P]),
    "mx_group_offsets_pad": (c_int, [_P, _I, _I, _I, _I, _P, _P, _P, _P]),
}

_lib = None


class MXLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Load libmxfp8_gfx950.so (once) and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise MXLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m torchtitan_amd._build` "
            "(the MXFP8 path has no fallback implementation)"
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().mx_status_string(status).decode()
        raise MXLibraryError(f"{what}: {msg} (status {status})")

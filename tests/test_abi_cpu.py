"""The C-ABI library loads and exports every symbol include/mxfp8.h declares (no GPU calls)."""
import ctypes
import re
from pathlib import Path

from torchtitan_amd import _lib

HEADER = Path(__file__).resolve().parent.parent / "include" / "mxfp8.h"


def declared_functions():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return re.findall(r"\b(mx_[a-z0-9_]+)\s*\(", text)


def test_header_declares_the_path():
    names = set(declared_functions())
    for must in ("mx_cast_dim0", "mx_cast_dim1", "mx_cast_dim0_dim1", "mx_scale_layout", "mx_gemm_nt",
                 "mx_grouped_gemm_2d3d", "mx_grouped_gemm_2d2d", "mx_group_offsets_pad"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in declared_functions():
        assert hasattr(lib, name), name
        assert name in _lib.SIGNATURES, f"{name} has no ctypes prototype"
    assert set(_lib.SIGNATURES) == set(declared_functions())


def test_host_side_entry_points_answer_without_a_gpu():
    lib = _lib.load()
    assert lib.mx_version() >= 100
    assert lib.mx_status_string(0) == b"ok" and b"align" in lib.mx_status_string(2)
    assert lib.mx_scales_mfma_bytes(16384, 128) == 16384 * 128
    assert lib.mx_scales_mfma_bytes(100, 7) == 1 * 4 * 256
    # argument validation happens before any launch
    assert lib.mx_cast_dim0(None, 4, 48, 48, None, None, 0, 0, None) != 0
    assert lib.mx_cast_dim0(None, 0, 64, 64, None, None, 0, 0, None) == 0  # empty is a no-op
    assert lib.mx_gemm_nt(None, None, None, None, None, 16, 16, 33, 16, None) != 0
    assert lib.mx_group_offsets_pad(None, 0, 1, 0, 32, None, None, None, None) == 1


def test_ctypes_prototypes_have_the_declared_number_of_arguments():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    for name, args in re.findall(r"\b(mx_[a-z0-9_]+)\s*\(([^)]*)\)\s*;", text):
        args = args.strip()
        n = 0 if args in ("", "void") else len(args.split(","))
        assert len(_lib.SIGNATURES[name][1]) == n, name
    # the grouped forms take the scale order just before the stream
    assert lib_arg_kinds("mx_grouped_gemm_2d3d")[-2:] == [ctypes.c_int, ctypes.c_void_p]
    assert lib_arg_kinds("mx_grouped_gemm_2d2d")[-2:] == [ctypes.c_int, ctypes.c_void_p]


def lib_arg_kinds(name):
    return list(_lib.SIGNATURES[name][1])


def test_new_entry_points_validate_arguments_before_any_launch():
    """Status 1 (invalid argument) for null pointers / negative sizes, 2 (alignment) for shapes or
    pointers the kernels cannot take, 0 for empty problems: decided on the host, no GPU needed."""
    lib = _lib.load()
    P = ctypes.c_void_p
    a16, odd = P(0x1000), P(0x1004)
    # gate-fused casts
    assert lib.mx_swiglu_cast_dim0_dim1(None, None, 0, 64, 64, 64, None, None, None, None, None, 1, 1, None) == 0
    assert lib.mx_swiglu_cast_dim0_dim1(None, a16, 32, 64, 64, 64, a16, a16, a16, a16, None, 1, 1, None) == 1
    assert lib.mx_swiglu_cast_dim0_dim1(a16, a16, 33, 64, 64, 64, a16, a16, a16, a16, None, 1, 1, None) == 2
    assert lib.mx_swiglu_cast_dim0_dim1(a16, odd, 32, 64, 64, 64, a16, a16, a16, a16, None, 1, 1, None) == 2
    assert lib.mx_swiglu_cast_dim0_dim1(a16, a16, 32, 64, 64, 64, a16, a16, a16, a16, None, 7, 1, None) == 1
    assert lib.mx_swiglu_bwd_cast_dim0_dim1(a16, a16, None, 32, 64, 64, 64, 64, a16, a16, a16, a16, None, 1, 1, None) == 1
    assert lib.mx_swiglu_bwd_cast_dim0_dim1(a16, a16, a16, 32, 64, 60, 64, 64, a16, a16, a16, a16, None, 1, 1, None) == 1
    assert lib.mx_swiglu_bwd_cast_dim0_dim1(a16, a16, a16, 32, 48, 64, 64, 64, a16, a16, a16, a16, None, 1, 1, None) == 2
    # gathered cast: the column-wise outputs come as a pair or not at all
    assert lib.mx_cast_rows_gathered(a16, a16, None, 10, 0, 64, 64, a16, a16, None, None, 1, 1, None) == 0
    assert lib.mx_cast_rows_gathered(a16, None, None, 10, 32, 64, 64, a16, a16, None, None, 1, 1, None) == 1
    assert lib.mx_cast_rows_gathered(a16, a16, None, 10, 32, 64, 64, a16, a16, a16, None, 1, 1, None) == 1
    assert lib.mx_cast_rows_gathered(a16, a16, None, 10, 40, 64, 64, a16, a16, a16, a16, 1, 1, None) == 2
    assert lib.mx_cast_rows_gathered(a16, a16, None, 10, 32, 72, 72, a16, a16, None, None, 1, 1, None) == 2
    # combine / row dot
    assert lib.mx_moe_combine(a16, None, 8, 64, a16, None, 0, 2, 64, a16, 64, None) == 0
    assert lib.mx_moe_combine(a16, None, 8, 64, None, None, 4, 2, 64, a16, 64, None) == 1
    assert lib.mx_moe_combine(a16, None, 8, 60, a16, None, 4, 2, 64, a16, 64, None) == 1
    assert lib.mx_moe_combine(a16, None, 8, 68, a16, None, 4, 2, 68, a16, 68, None) == 2
    assert lib.mx_moe_combine(a16, odd, 8, 64, a16, None, 4, 2, 64, a16, 64, None) == 2
    assert lib.mx_moe_row_dot(a16, None, 8, 64, a16, a16, 8, 64, None, 4, 64, a16, None) == 1
    assert lib.mx_moe_row_dot(a16, None, 8, 64, a16, odd, 8, 64, a16, 4, 64, a16, None) == 2
    # dequantization and token log-probabilities
    assert lib.mx_dequant(a16, a16, 4, 48, 0, a16, 48, None) == 2
    assert lib.mx_dequant(a16, None, 4, 64, 0, a16, 64, None) == 1
    assert lib.mx_dequant(a16, a16, 4, 64, 5, a16, 64, None) == 1
    assert lib.mx_token_logprob_fwd(a16, 0, 100, 104, a16, a16, a16, None) == 0
    assert lib.mx_token_logprob_fwd(a16, 4, 0, 104, a16, a16, a16, None) == 1
    assert lib.mx_token_logprob_fwd(a16, 4, 100, 100, a16, a16, a16, None) == 2
    assert lib.mx_token_logprob_bwd(a16, 70000, 104, 104, a16, a16, a16, a16, 104, None) == 4
    assert lib.mx_token_logprob_bwd(a16, 4, 104, 104, a16, a16, None, a16, 104, None) == 1
    # the GEMM that may split its contraction: same checks as mx_gemm_nt, decided before any launch
    assert lib.mx_gemm_nt_ws(a16, a16, a16, a16, a16, 0, 64, 64, 64, None, 0, None) == 0
    assert lib.mx_gemm_nt_ws(None, a16, a16, a16, a16, 64, 64, 64, 64, None, 0, None) == 1
    assert lib.mx_gemm_nt_ws(a16, a16, a16, a16, a16, 64, 64, 64, 32, None, 0, None) == 1   # ldd < N
    assert lib.mx_gemm_nt_ws(a16, a16, a16, a16, a16, 64, 64, 48, 64, None, 0, None) == 2   # K % 32
    assert lib.mx_gemm_nt_ws(odd, a16, a16, a16, a16, 64, 64, 64, 64, None, 0, None) == 2
    # shapes that are never split need no device to say so
    assert lib.mx_gemm_nt_workspace_bytes(64, 64, 4096) == 0
    assert lib.mx_gemm_nt_workspace_bytes(4096, 4096, 0) == 0


def test_library_exports_the_test_hooks_of_the_debug_header():
    """include/mxfp8_debug.h: every hook is exported, except the one that exists in timing builds
    only; the yardsticks check their arguments before any launch."""
    debug = HEADER.with_name("mxfp8_debug.h")
    text = re.sub(r"/\*.*?\*/", "", debug.read_text(), flags=re.S)
    names = set(re.findall(r"\b(mx_debug_[a-z0-9_]+)\s*\(", text))
    assert {"mx_debug_force_kernel", "mx_debug_set_grid", "mx_debug_stream", "mx_debug_mfma_only"} <= names
    lib = ctypes.CDLL(str(_lib.LIB_PATH))
    for name in names - {"mx_debug_set_prof"}:
        assert hasattr(lib, name), name
    assert not hasattr(lib, "mx_debug_set_prof"), "the product build carries no timing instances"
    lib.mx_debug_mfma_only.restype = ctypes.c_int
    lib.mx_debug_mfma_only.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int,
                                       ctypes.c_void_p]
    assert lib.mx_debug_mfma_only(8, None, None, 1, 1, None) == 1      # no such MFMA shape
    assert lib.mx_debug_mfma_only(16, None, None, 256, 10, None) == 1  # null operands
    lib.mx_debug_stream.restype = ctypes.c_int
    lib.mx_debug_stream.argtypes = [ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
    assert lib.mx_debug_stream(0, None, None, 24, None) == 1           # not a multiple of 16 bytes

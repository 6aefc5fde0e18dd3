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

"""ctypes loader for oracle/libmx_oracle.so (the C restatement).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB = HERE / "libmx_oracle.so"


def build() -> Path:
    subprocess.run(["make", "-C", str(HERE), "-B", "libmx_oracle.so"], check=True, capture_output=True)
    return LIB


def load():
    if not LIB.exists():
        build()
    lib = ctypes.CDLL(str(LIB))
    P, I = ctypes.c_void_p, ctypes.c_int64
    lib.mxo_cast_dim0.argtypes = [P, I, I, ctypes.c_int, P, P]
    lib.mxo_cast_dim1.argtypes = [P, I, I, ctypes.c_int, P, P]
    lib.mxo_dequant.argtypes = [P, P, I, I, P]
    return lib


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def cast_dim0(x_bits: np.ndarray, mode: int):
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    R, C = x.shape
    codes = np.empty((R, C), np.uint8)
    scales = np.empty((R, C // 32), np.uint8)
    load().mxo_cast_dim0(_p(x), R, C, mode, _p(codes), _p(scales))
    return codes, scales


def cast_dim1(x_bits: np.ndarray, mode: int):
    x = np.ascontiguousarray(x_bits, dtype=np.uint16)
    R, C = x.shape
    codes = np.empty((C, R), np.uint8)
    scales = np.empty((C, R // 32), np.uint8)
    load().mxo_cast_dim1(_p(x), R, C, mode, _p(codes), _p(scales))
    return codes, scales


def dequant(codes: np.ndarray, scales: np.ndarray) -> np.ndarray:
    codes = np.ascontiguousarray(codes, dtype=np.uint8)
    scales = np.ascontiguousarray(scales, dtype=np.uint8)
    R, C = codes.shape
    out = np.empty((R, C), np.float32)
    load().mxo_dequant(_p(codes), _p(scales), R, C, _p(out))
    return out

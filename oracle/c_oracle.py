"""ctypes binding of the bit-level C oracle (oracle/fp8_cast_ref.c).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_DIR = Path(__file__).resolve().parent
_LIB = None

E4M3, E5M2 = 0, 1


def build() -> Path:
    subprocess.run(["make", "-s", "-C", str(_DIR), "liboracle.so"], check=True)
    return _DIR / "liboracle.so"


def lib() -> ctypes.CDLL:
    global _LIB
    if _LIB is None:
        path = _DIR / "liboracle.so"
        if not path.exists():
            build()
        L = ctypes.CDLL(str(path))
        L.orc_f32_to_fp8.restype = ctypes.c_uint8
        L.orc_f32_to_fp8.argtypes = [ctypes.c_float, ctypes.c_int]
        L.orc_fp8_to_f32.restype = ctypes.c_float
        L.orc_fp8_to_f32.argtypes = [ctypes.c_uint8, ctypes.c_int]
        L.orc_scale_from_amax.restype = ctypes.c_float
        L.orc_scale_from_amax.argtypes = [ctypes.c_float, ctypes.c_int, ctypes.c_int]
        L.orc_amax_bf16.restype = ctypes.c_float
        L.orc_amax_bf16.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        L.orc_amax_f32.restype = ctypes.c_float
        L.orc_amax_f32.argtypes = [ctypes.c_void_p, ctypes.c_size_t]
        L.orc_cast_bf16.restype = None
        L.orc_cast_bf16.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_int, ctypes.c_void_p]
        L.orc_cast_f32.restype = None
        L.orc_cast_f32.argtypes = [ctypes.c_void_p, ctypes.c_size_t, ctypes.c_float, ctypes.c_int, ctypes.c_void_p]
        L.orc_emulated_mm.restype = None
        L.orc_emulated_mm.argtypes = [
            ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
            ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_int,
            ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
        ]
        _LIB = L
    return _LIB


def cast_bf16_bits(bits_u16: np.ndarray, scale: float, dtype: int) -> np.ndarray:
    """bits_u16: bf16 bit patterns (uint16). Returns fp8 bytes (uint8)."""
    x = np.ascontiguousarray(bits_u16, dtype=np.uint16)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_cast_bf16(x.ctypes.data, x.size, ctypes.c_float(scale), dtype, out.ctypes.data)
    return out


def cast_f32(x: np.ndarray, scale: float, dtype: int) -> np.ndarray:
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_cast_f32(x.ctypes.data, x.size, ctypes.c_float(scale), dtype, out.ctypes.data)
    return out


def amax_bf16_bits(bits_u16: np.ndarray) -> float:
    x = np.ascontiguousarray(bits_u16, dtype=np.uint16)
    return float(lib().orc_amax_bf16(x.ctypes.data, x.size))


def scale_from_amax(amax: float, dtype: int, pow2: bool) -> float:
    return float(lib().orc_scale_from_amax(ctypes.c_float(amax), dtype, int(pow2)))


def fp8_to_f32(byte: int, dtype: int) -> float:
    return float(lib().orc_fp8_to_f32(byte, dtype))


def emulated_mm(a: np.ndarray, a_dtype: int, sa: np.ndarray, b: np.ndarray, b_dtype: int, sb: np.ndarray) -> np.ndarray:
    """a [M,K] uint8, b [N,K] uint8; sa/sb float32 arrays of size 1 (scalar) or M / N."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    sa = np.ascontiguousarray(sa, dtype=np.float32).reshape(-1)
    sb = np.ascontiguousarray(sb, dtype=np.float32).reshape(-1)
    M, K = a.shape
    N = b.shape[0]
    out = np.empty((M, N), dtype=np.float64)
    lib().orc_emulated_mm(
        a.ctypes.data, a_dtype, sa.ctypes.data, int(sa.size > 1),
        b.ctypes.data, b_dtype, sb.ctypes.data, int(sb.size > 1),
        M, N, K, out.ctypes.data,
    )
    return out

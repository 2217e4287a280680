"""
ctypes binding of libmi8.so (the C ABI declared in include/mi8.h).

The library is loaded once; it is never built from here and there is no fallback path: if the shared
object is missing, every operator raises ``MI8LibraryMissing`` with the build command.
"""

from __future__ import annotations

import ctypes
from ctypes import c_char_p, c_float, c_int, c_int32, c_int64, c_uint32, c_void_p, POINTER
from pathlib import Path
from typing import Optional

from .exceptions import MI8KernelError

import os

# MI8_LIBRARY overrides the in-tree location (e.g. to try a differently built library)
LIB_PATH = Path(os.environ.get("MI8_LIBRARY") or (Path(__file__).resolve().parent / "lib" / "libmi8.so"))

MI8_E4M3, MI8_E5M2 = 0, 1
MI8_BF16, MI8_F32, MI8_F16, MI8_RAW8 = 0, 1, 2, 3
FLAG_POW2_SCALE = 1
FLAG_SW_CVT = 2
FLAG_AMAX_READY = 4
AMAX_SLOTS = 2048

# name -> (restype, argtypes); mirrors include/mi8.h one to one
_SIGNATURES = {
    "mi8_version": (c_int, []),
    "mi8_last_error": (c_char_p, []),
    "mi8_amax_partials": (c_int, [c_void_p, c_int, c_int64, c_void_p, POINTER(c_int32), c_void_p]),
    "mi8_amax_partials_batch": (c_int, [POINTER(c_void_p), POINTER(c_int64), c_int32, c_int, c_void_p, POINTER(c_int32), c_void_p]),
    "mi8_amax_slots_for": (c_int32, [c_int64]),
    "mi8_scale_from_partials": (c_int, [c_void_p, c_int32, c_int, c_uint32, c_void_p, c_void_p]),
    "mi8_multi_tensor_scales": (
        c_int,
        [c_void_p, c_void_p, c_int32, c_int, c_int, c_uint32, c_void_p, c_void_p, c_void_p],
    ),
    "mi8_cast_tensorwise": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_void_p, c_int, c_uint32, c_void_p, c_int64,
         c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "mi8_cast_tensorwise_static": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int, c_uint32, c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "mi8_cast_rowwise": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int, c_uint32, c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "mi8_colamax_workspace_slots": (c_int64, [c_int64, c_int64]),
    "mi8_cast_colwise_t": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_int, c_uint32, c_void_p, c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "mi8_gemm_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p,
         c_int, c_void_p, c_int, c_int64, c_int, c_void_p],
    ),
    "mi8_gemm_fp8_accumulate": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p,
         c_int, c_void_p, c_int, c_int64, c_void_p],
    ),
    "mi8_gemm_fp8_swiglu_matches_separate": (c_int, [c_int64, c_int64, c_int64]),
    "mi8_gemm_fp8_swiglu": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, POINTER(c_int32), c_void_p, c_void_p],
    ),
    "mi8_gemm_fp8_splitk": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p,
         c_int, c_void_p, c_int, c_int64, c_int, c_void_p, c_int64, c_void_p],
    ),
    "mi8_gemm_splitk_suggest": (c_int, [c_int64, c_int64, c_int64]),
    "mi8_gemm_splitk_workspace_bytes": (c_int64, [c_int64, c_int64, c_int]),
    "mi8_gemm_num_variants": (c_int, []),
    "mi8_gemm_variant_name": (c_char_p, [c_int]),
    "mi8_swiglu_fwd": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "mi8_swiglu_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "mi8_swiglu_bwd_cast": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_int32, c_int, c_uint32, c_void_p, c_void_p,
         c_int64, c_void_p, c_void_p, c_int64, c_void_p, c_void_p, c_void_p],
    ),
    "mi8_rowseg_code_count": (c_int64, [c_int64, c_int64]),
    "mi8_swiglu_amax_state_words": (c_int64, [c_int64, c_int64]),
    "mi8_rowseg_max_codes": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "mi8_swiglu_bwd_amax_from_codes": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "mi8_gemm_fp8_codes_supported": (c_int, [c_int64, c_int64, c_int64]),
    "mi8_gemm_fp8_codes": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p,
         c_int64, c_void_p, c_void_p],
    ),
    "mi8_moe_gather": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int32, c_void_p, c_void_p],
    ),
    "mi8_moe_binned_gather": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_int32, c_int64, c_int32, c_void_p,
         c_void_p],
    ),
    "mi8_moe_scatter": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int, c_int32, c_void_p, c_void_p, c_void_p],
    ),
    "mi8_moe_binned_scatter": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int, c_void_p, c_int32, c_int64, c_int32, c_void_p,
         c_void_p, c_void_p],
    ),
    "mi8_moe_scatter_wgrad": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_void_p, c_void_p],
    ),
    "mi8_moe_binned_scatter_wgrad": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int32, c_int64, c_int32, c_void_p, c_void_p],
    ),
    "mi8_grouped_padded_rows": (c_int64, [c_int64, c_int32]),
    "mi8_grouped_cast_colwise_t": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_int, c_uint32, c_void_p, c_void_p, c_int64, c_void_p,
         c_void_p],
    ),
    "mi8_grouped_swiglu_fwd": (
        c_int,
        [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p],
    ),
    "mi8_grouped_swiglu_bwd": (
        c_int,
        [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_int32, c_void_p, c_void_p, c_void_p, c_void_p,
         c_void_p, c_void_p, c_void_p],
    ),
    "mi8_grouped_cast_rows_and_colwise_t": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_int, c_uint32, c_void_p, c_void_p, c_int64, c_void_p,
         c_void_p, c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "mi8_moe_gather_cast_rows_and_colwise_t": (
        c_int,
        [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_void_p, c_int, c_void_p, c_int32, c_int, c_uint32, c_void_p,
         c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p],
    ),
    "mi8_grouped_gemm_fp8": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_int64, c_int64, c_int64,
         c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int64, c_void_p],
    ),
    "mi8_grouped_gemm_fp8_accumulate": (
        c_int,
        [c_void_p, c_int, c_int64, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_int64, c_int64, c_int64,
         c_void_p, c_void_p, c_int64, c_void_p, c_int, c_int64, c_void_p],
    ),
    "mi8_grouped_gemm_fp8_dual_supported": (c_int, [c_int64, c_int64, c_int64, c_int64]),
    "mi8_grouped_gemm_fp8_dual": (
        c_int,
        [c_void_p, c_void_p, c_int, c_int64, c_void_p, c_void_p, c_int, c_int64, c_int64, c_void_p, c_int32, c_int64, c_int64,
         c_int64, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_int64, c_void_p],
    ),
    "mi8_grouped_wgrad_fp8": (
        c_int,
        [c_void_p, c_int, c_void_p, c_int, c_int64, c_void_p, c_int32, c_int64, c_int64, c_int64, c_void_p, c_void_p,
         c_void_p, c_int, c_void_p],
    ),
}

EXPORTED_SYMBOLS = tuple(_SIGNATURES)

# libmi8_diag.so (include/mi8_diag.h): measurement kernels, loaded by bench.py only
DIAG_LIB_PATH = LIB_PATH.parent / "libmi8_diag.so"
_DIAG_SIGNATURES = {
    "mi8_diag_last_error": (c_char_p, []),
    "mi8_probe_mfma_loop": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mi8_probe_mfma_feed": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "mi8_probe_store_rate": (c_int, [c_int, c_int, c_int, c_int, c_void_p, c_int64, c_void_p, c_void_p]),
    "mi8_diag_gemm_tile_timeline": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_int, c_void_p, c_void_p]),
}
DIAG_EXPORTED_SYMBOLS = tuple(_DIAG_SIGNATURES)


class MI8LibraryMissing(RuntimeError):
    pass


_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """The loaded library (loads on first use)."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise MI8LibraryMissing(
                f"{LIB_PATH} is not built. Build it with `python -m olmo_core_amd.build` (needs hipcc); "
                "there is no fallback implementation."
            )
        handle = ctypes.CDLL(str(LIB_PATH))
        for name, (res, args) in _SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _lib = handle
    return _lib


_diag: Optional[ctypes.CDLL] = None


def diag() -> ctypes.CDLL:
    """The diagnostics library (loads on first use)."""
    global _diag
    if _diag is None:
        if not DIAG_LIB_PATH.exists():
            raise MI8LibraryMissing(f"{DIAG_LIB_PATH} is not built. Build it with `python -m olmo_core_amd.build`.")
        handle = ctypes.CDLL(str(DIAG_LIB_PATH))
        for name, (res, args) in _DIAG_SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = res
            fn.argtypes = args
        _diag = handle
    return _diag


def check_diag(status: int, what: str = "") -> None:
    if status != 0:
        msg = diag().mi8_diag_last_error()
        raise MI8KernelError(f"{what or 'libmi8_diag'}: error {status}: {msg.decode() if msg else ''}")


def is_built() -> bool:
    return LIB_PATH.exists()


def last_error() -> str:
    msg = lib().mi8_last_error()
    return msg.decode() if msg else ""


def check(status: int, what: str = "") -> None:
    """Raise on a non-zero status from the library."""
    if status != 0:
        kind = {-1: "bad argument", -2: "unsupported shape/alignment", -3: "launch failure"}.get(status, "error")
        raise MI8KernelError(f"{what or 'libmi8'}: {kind} ({status}): {last_error()}")

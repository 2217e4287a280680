"""The C-ABI library loads and exports every symbol include/mi8.h declares (no GPU work is launched)."""

import ctypes
import re
from pathlib import Path

import pytest

from olmo_core_amd import _C

ROOT = Path(__file__).resolve().parent.parent


def _declared_symbols(header="mi8.h"):
    text = (ROOT / "include" / header).read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mi8_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_agree():
    assert _declared_symbols() == sorted(_C.EXPORTED_SYMBOLS)


def test_library_exports_every_declared_symbol():
    assert _C.is_built(), "libmi8.so is not built: run `python -m olmo_core_amd.build`"
    handle = ctypes.CDLL(str(_C.LIB_PATH))
    for name in _declared_symbols():
        assert hasattr(handle, name), f"libmi8.so does not export {name}"


def test_diagnostics_live_in_their_own_library():
    """The measurement kernels are no part of the drop-in boundary: mi8.h / libmi8.so do not carry them,
    mi8_diag.h / libmi8_diag.so do."""
    diag_syms = _declared_symbols("mi8_diag.h")
    assert diag_syms == sorted(_C.DIAG_EXPORTED_SYMBOLS)
    assert not set(diag_syms) & set(_declared_symbols())
    assert _C.DIAG_LIB_PATH.exists(), "libmi8_diag.so is not built: run `python -m olmo_core_amd.build`"
    main, diag = ctypes.CDLL(str(_C.LIB_PATH)), ctypes.CDLL(str(_C.DIAG_LIB_PATH))
    for name in diag_syms:
        assert hasattr(diag, name), f"libmi8_diag.so does not export {name}"
        assert not hasattr(main, name), f"libmi8.so exports the diagnostic {name}"
    assert _C.diag().mi8_probe_mfma_loop(7, 0, 1, 1, None, None) == -1  # argument check, nothing launched
    assert b"sink" in _C.diag().mi8_diag_last_error()


def test_host_only_entry_points():
    L = _C.lib()
    assert L.mi8_version() == 100
    assert L.mi8_gemm_num_variants() >= 1
    assert L.mi8_gemm_variant_name(0)
    assert L.mi8_gemm_variant_name(999) is None
    assert L.mi8_amax_slots_for(1) == 1
    assert L.mi8_amax_slots_for(1 << 40) == _C.AMAX_SLOTS
    assert L.mi8_colamax_workspace_slots(16384, 4096) % 4096 == 0
    # split-K planning: large problems are not split, a few rows go to the kernel that streams the weight once,
    # few output tiles with a long K are cut so that no slice is empty and each keeps at least four K steps
    assert L.mi8_gemm_splitk_suggest(16384, 11008, 4096) == 1
    assert L.mi8_gemm_splitk_suggest(16, 4096, 4096) == 1
    assert L.mi8_gemm_splitk_suggest(256, 256, 512) == 1
    for (m, n, k) in ((256, 4096, 11008), (100, 200, 1040), (384, 1024, 4096), (64, 11008, 4096)):
        s = L.mi8_gemm_splitk_suggest(m, n, k)
        steps = -(-k // 128)
        per = -(-steps // s)
        assert 2 <= s <= 32 and per >= 4 - 1 and (s - 1) * per < steps, (m, n, k, s)
    assert L.mi8_gemm_splitk_workspace_bytes(100, 30, 4) == 4 * 100 * 32 * 4
    assert L.mi8_gemm_splitk_workspace_bytes(0, 30, 4) == 0


def test_host_only_shape_helpers():
    """Sizes and shape predicates the callers plan with (no GPU work)."""
    L = _C.lib()
    # one code per 64 columns of a row, ragged last segment included
    assert L.mi8_rowseg_code_count(16384, 11008) == 16384 * 172
    assert L.mi8_rowseg_code_count(3, 65) == 6 and L.mi8_rowseg_code_count(0, 64) == 0
    assert L.mi8_swiglu_amax_state_words(16384, 11008) >= 4 and L.mi8_swiglu_amax_state_words(0, 0) == 0
    # the GEMM that records codes is the persistent tile kernel: full tiles, K in 128-byte steps, whole segments
    assert L.mi8_gemm_fp8_codes_supported(16384, 11008, 4096) == 1
    for shape in ((128, 11008, 4096), (16384, 11008, 4000), (16384, 11000, 4096)):
        assert L.mi8_gemm_fp8_codes_supported(*shape) == 0, shape
    # the fused SwiGLU launch replaces the separate GEMMs only where both run on that kernel
    assert L.mi8_gemm_fp8_swiglu_matches_separate(16384, 11008, 4096) == 1
    assert L.mi8_gemm_fp8_swiglu_matches_separate(64, 11008, 4096) == 0
    # the padded token axis of the grouped transposed copies: groups whose sizes sum to T fill at most
    # ceil(T / 128) + groups - 1 tiles of 128 rows
    assert L.mi8_grouped_padded_rows(131072, 64) == 131072 + 63 * 128
    assert L.mi8_grouped_padded_rows(5, 2) == 2 * 128


def test_argument_validation_happens_before_any_gpu_call():
    L = _C.lib()
    assert L.mi8_cast_rowwise(None, 0, 4, 16, 0, 0, None, 16, None, None) == -1
    assert "null" in _C.last_error()
    assert L.mi8_gemm_fp8(None, 0, 16, None, 0, 16, 1, 1, 16, None, 0, None, 0, None, 0, 16, -1, None) == -1
    assert L.mi8_gemm_fp8_splitk(None, 0, 16, None, 0, 16, 1, 1, 16, None, 0, None, 0, None, 0, 16, 2, None, 0, None) == -1
    assert L.mi8_amax_partials_batch(None, None, 1, 0, None, None, None) == -1
    ptrs, ns = (ctypes.c_void_p * 9)(), (ctypes.c_int64 * 9)()
    assert L.mi8_amax_partials_batch(ptrs, ns, 9, 0, ctypes.c_void_p(16), None, None) == -1 and "9 tensors" in _C.last_error()
    assert L.mi8_amax_partials_batch(ptrs, ns, 2, 0, ctypes.c_void_p(16), None, None) == -1 and "tensor 0 is null" in _C.last_error()
    with pytest.raises(Exception):
        _C.check(-2, "x")

"""
Torch-level wrappers over the C ABI: quantised operands and the scaled GEMM.

torch is used here for device memory and streams only: every wrapper allocates its outputs with
``torch.empty`` on the input's device, passes raw pointers plus the current HIP stream to
``libmi8.so``, and returns tensors.  Nothing in this file computes on the host or falls back to PyTorch
arithmetic.  (What the callers in ``linear.py`` leave to torch is what the reference leaves in high precision
too: a GEMM whose two cast configs are DISABLED - ``rowwise_with_gw_hp``'s grad_weight - is a bf16 ``torch.mm``,
and the bias is added by ``+``.)
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch

from .. import _C

_FP8_CODE = {torch.float8_e4m3fn: _C.MI8_E4M3, torch.float8_e5m2: _C.MI8_E5M2}
_HP_CODE = {torch.bfloat16: _C.MI8_BF16, torch.float32: _C.MI8_F32}

# Debug/testing switch: convert with the integer-arithmetic path instead of v_cvt_pk_*.
FORCE_SW_CVT = False

# Measurement hook: when set to a list, every GEMM launch appends (start_event, end_event, (M, N, K)) recorded
# on the launch stream.
GEMM_EVENT_SINK = None


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """Handle of torch's current stream on ``t``'s device (the direct query costs a fifth of building a
    ``torch.cuda.Stream`` object, which shows in calls on a few rows)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


def _flags(pow2: bool) -> int:
    return (_C.FLAG_POW2_SCALE if pow2 else 0) | (_C.FLAG_SW_CVT if FORCE_SW_CVT else 0)


def _require_gpu(t: torch.Tensor, what: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{what}: expected a tensor on the GPU, got device '{t.device}' (there is no CPU path)")


def _hp2d(x: torch.Tensor, what: str) -> torch.Tensor:
    _require_gpu(x, what)
    if x.dim() != 2:
        raise ValueError(f"{what}: expected a 2-D tensor, got shape {tuple(x.shape)}")
    if x.dtype not in _HP_CODE:
        raise TypeError(f"{what}: unsupported dtype {x.dtype} (bfloat16 or float32)")
    if not x.is_contiguous() or x.data_ptr() % 16:
        x = x.contiguous()
        if x.data_ptr() % 16:
            x = x.clone()
    return x


_SMALL_CAST = 65536  # elements up to which mi8_cast_tensorwise takes the amax itself


def pad16(n: int) -> int:
    return (n + 15) // 16 * 16


def amax_partials(x: torch.Tensor) -> Tuple[torch.Tensor, int]:
    """Per-workgroup partial maxima of |x| (as float32 bit patterns); returns (slots, n_used)."""
    _require_gpu(x, "amax_partials")
    xc = x if x.is_contiguous() else x.contiguous()
    slots = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=x.device)
    used = _C.c_int32(0)
    _C.check(
        _C.lib().mi8_amax_partials(xc.data_ptr(), _HP_CODE[xc.dtype], xc.numel(), slots.data_ptr(), used, _stream(x)),
        "mi8_amax_partials",
    )
    return slots, used.value


AMAX_BATCH = 8


def amax_partials_batch(tensors) -> list:
    """:func:`amax_partials` of up to ``AMAX_BATCH`` contiguous GPU tensors of one dtype in one launch: a list of
    ``(slots, n_used)`` in the order given (same values as separate calls)."""
    n = len(tensors)
    if not 0 < n <= AMAX_BATCH:
        raise ValueError(f"amax_partials_batch: {n} tensors (1..{AMAX_BATCH})")
    t0 = tensors[0]
    _require_gpu(t0, "amax_partials_batch")
    for t in tensors:
        if t.dtype != t0.dtype or t.device != t0.device or not t.is_contiguous():
            raise ValueError("amax_partials_batch: tensors must be contiguous, on one GPU and of one dtype")
    slots = torch.empty((n, _C.AMAX_SLOTS), dtype=torch.int32, device=t0.device)
    ptrs = (_C.c_void_p * n)(*[t.data_ptr() for t in tensors])
    numels = (_C.c_int64 * n)(*[t.numel() for t in tensors])
    used = (_C.c_int32 * n)()
    _C.check(
        _C.lib().mi8_amax_partials_batch(ptrs, numels, n, _HP_CODE[t0.dtype], slots.data_ptr(), used, _stream(t0)),
        "mi8_amax_partials_batch",
    )
    return [(slots[i], int(used[i])) for i in range(n)]


def scale_from_partials(slots: torch.Tensor, n_slots: int, fp8_dtype: torch.dtype, pow2: bool = False) -> torch.Tensor:
    """Returns a float32 tensor [2] = (scale, amax)."""
    out = torch.empty(2, dtype=torch.float32, device=slots.device)
    _C.check(
        _C.lib().mi8_scale_from_partials(
            slots.data_ptr(), n_slots, _FP8_CODE[fp8_dtype], _flags(pow2), out.data_ptr(), _stream(slots)
        ),
        "mi8_scale_from_partials",
    )
    return out


def tensor_to_scale(x: torch.Tensor, fp8_dtype: torch.dtype, pow2: bool = False) -> torch.Tensor:
    """Tensorwise dynamic scale of ``x`` (0-d float32 tensor on x's device)."""
    slots, used = amax_partials(x)
    return scale_from_partials(slots, used, fp8_dtype, pow2)[0]


def multi_tensor_scales(tensors, fp8_dtype: torch.dtype, pow2: bool = False) -> torch.Tensor:
    """Tensorwise dynamic scales of a list of same-dtype GPU tensors in one batch of launches: float32 ``[n]``."""
    if not tensors:
        raise ValueError("multi_tensor_scales: no tensors")
    t0 = tensors[0]
    _require_gpu(t0, "multi_tensor_scales")
    step = 8 if t0.dtype == torch.bfloat16 else 4
    for t in tensors:
        if t.dtype != t0.dtype or t.dtype not in _HP_CODE or t.device != t0.device or not t.is_contiguous():
            raise ValueError("multi_tensor_scales: tensors must be contiguous, on one GPU and of one dtype (bf16 or fp32)")
        if t.numel() % step or t.data_ptr() % 16:
            raise ValueError("multi_tensor_scales: every tensor needs 16-byte alignment and a multiple of 16 bytes")
    n = len(tensors)
    table = torch.tensor([[t.data_ptr() for t in tensors], [t.numel() for t in tensors]], dtype=torch.int64).to(t0.device)
    ws = torch.empty(n, dtype=torch.int32, device=t0.device)
    out = torch.empty(n, dtype=torch.float32, device=t0.device)
    _C.check(
        _C.lib().mi8_multi_tensor_scales(
            table[0].data_ptr(), table[1].data_ptr(), n, _HP_CODE[t0.dtype], _FP8_CODE[fp8_dtype], _flags(pow2),
            ws.data_ptr(), out.data_ptr(), _stream(t0),
        ),
        "mi8_multi_tensor_scales",
    )
    return out


def _operand(shape: Tuple[int, int], fp8_dtype: torch.dtype, device, pitch: Optional[int] = None) -> torch.Tensor:
    """Uninitialised fp8 ``[rows, k]`` GEMM operand; with ``pitch > k`` a view of a wider buffer (the kernels take
    any row pitch that is a multiple of 16)."""
    rows, k = shape
    if pitch is None or pitch == k:
        return torch.empty((rows, k), dtype=fp8_dtype, device=device)
    if pitch < k or pitch % 16:
        raise ValueError(f"operand pitch {pitch} must be a multiple of 16 and at least {k}")
    return torch.empty((rows, pitch), dtype=fp8_dtype, device=device)[:, :k]


def cast_tensorwise(
    x: torch.Tensor,
    fp8_dtype: torch.dtype,
    *,
    pow2: bool = False,
    want_rowmajor: bool = True,
    want_transposed: bool = False,
    slots: Optional[Tuple[torch.Tensor, int]] = None,
    scale: Optional[torch.Tensor] = None,
    pitch: Optional[int] = None,
    pitch_t: Optional[int] = None,
) -> Tuple[Optional[torch.Tensor], Optional[torch.Tensor], torch.Tensor]:
    """
    Quantise ``x [rows, cols]`` with one scale.  Returns ``(q, q_t, scale)``: ``q`` fp8 ``[rows, cols]``,
    ``q_t`` fp8 ``[cols, pad16(rows)]`` (zero padded), ``scale`` float32 ``[1]``.  The scale comes from
    ``scale`` if given, else from amax partials (``slots`` if already computed by a producer kernel).
    """
    x = _hp2d(x, "cast_tensorwise")
    rows, cols = x.shape
    dev = x.device
    # small tensors with only the row-major copy: the cast kernel takes the amax itself (one launch)
    fused_amax = scale is None and slots is None and want_rowmajor and not want_transposed and x.numel() <= _SMALL_CAST
    if scale is None and slots is None and not fused_amax:
        slots = amax_partials(x)
    q = _operand((rows, cols), fp8_dtype, dev, pitch) if want_rowmajor else None
    q_t = _operand((cols, pad16(rows)), fp8_dtype, dev, pitch_t) if want_transposed else None
    scale_out = torch.empty(1, dtype=torch.float32, device=dev)
    if scale is not None:
        scale = scale.reshape(1).to(torch.float32)
    _C.check(
        _C.lib().mi8_cast_tensorwise(
            x.data_ptr(), _HP_CODE[x.dtype], rows, cols,
            slots[0].data_ptr() if slots is not None and scale is None else None,
            slots[1] if slots is not None and scale is None else 0,
            scale.data_ptr() if scale is not None else None,
            _FP8_CODE[fp8_dtype], _flags(pow2),
            q.data_ptr() if q is not None else None, q.stride(0) if q is not None else 0,
            q_t.data_ptr() if q_t is not None else None, q_t.stride(0) if q_t is not None else 0,
            scale_out.data_ptr(), _stream(x),
        ),
        "mi8_cast_tensorwise",
    )
    return q, q_t, scale_out


def cast_rowwise(
    x: torch.Tensor, fp8_dtype: torch.dtype, *, pow2: bool = False, pitch: Optional[int] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One scale per row: returns (q fp8 [rows, cols], scale float32 [rows])."""
    x = _hp2d(x, "cast_rowwise")
    rows, cols = x.shape
    q = _operand((rows, cols), fp8_dtype, x.device, pitch)
    s = torch.empty(rows, dtype=torch.float32, device=x.device)
    _C.check(
        _C.lib().mi8_cast_rowwise(
            x.data_ptr(), _HP_CODE[x.dtype], rows, cols, _FP8_CODE[fp8_dtype], _flags(pow2), q.data_ptr(),
            q.stride(0), s.data_ptr(), _stream(x),
        ),
        "mi8_cast_rowwise",
    )
    return q, s


def cast_colwise_t(
    x: torch.Tensor, fp8_dtype: torch.dtype, *, pow2: bool = False, pitch_t: Optional[int] = None
) -> Tuple[torch.Tensor, torch.Tensor]:
    """One scale per column, transposed output: returns (q_t fp8 [cols, pad16(rows)], scale float32 [cols])."""
    x = _hp2d(x, "cast_colwise_t")
    rows, cols = x.shape
    q_t = _operand((cols, pad16(rows)), fp8_dtype, x.device, pitch_t)
    s = torch.empty(cols, dtype=torch.float32, device=x.device)
    ws = torch.empty(_C.lib().mi8_colamax_workspace_slots(rows, cols), dtype=torch.int32, device=x.device)
    _C.check(
        _C.lib().mi8_cast_colwise_t(
            x.data_ptr(), _HP_CODE[x.dtype], rows, cols, _FP8_CODE[fp8_dtype], _flags(pow2), ws.data_ptr(),
            q_t.data_ptr(), q_t.stride(0), s.data_ptr(), _stream(x),
        ),
        "mi8_cast_colwise_t",
    )
    return q_t, s


def gemm_fp8(
    a: torch.Tensor,
    sa: torch.Tensor,
    b: torch.Tensor,
    sb: torch.Tensor,
    *,
    k: Optional[int] = None,
    out_dtype: torch.dtype = torch.bfloat16,
    variant: int = -1,
    out: Optional[torch.Tensor] = None,
    splits: int = -1,
    accumulate: bool = False,
) -> torch.Tensor:
    """
    ``out[M, N] = (a[M, :k] @ b[N, :k].T) / sa / sb`` with fp32 accumulation on the fp8 matrix cores.
    ``accumulate`` (needs ``out``): ``out += product`` with the bits of ``out + gemm_fp8(...)`` on ``out_dtype`` tensors.
    ``a`` and ``b`` are fp8 tensors whose rows are K-contiguous; ``sa`` / ``sb`` hold one scale or one per row.
    ``out``: an ``[M, N]`` tensor of ``out_dtype`` with contiguous rows (any row pitch) to write into.
    ``splits``: slices of K summed separately and added afterwards (for problems with few output tiles);
    -1 lets the library decide from the shape, 1 forbids splitting; a forced ``variant`` is never split.
    """
    _require_gpu(a, "gemm_fp8")
    if a.dim() != 2 or b.dim() != 2 or a.stride(1) != 1 or b.stride(1) != 1:
        raise ValueError("gemm_fp8: operands must be 2-D with contiguous rows")
    if a.dtype not in _FP8_CODE or b.dtype not in _FP8_CODE:
        raise TypeError(f"gemm_fp8: operands must be float8, got {a.dtype} and {b.dtype}")
    if out_dtype not in _HP_CODE:
        raise TypeError(f"gemm_fp8: unsupported output dtype {out_dtype}")
    M, N = a.shape[0], b.shape[0]
    K = min(a.shape[1], b.shape[1]) if k is None else k
    if sa.numel() not in (1, M) or sb.numel() not in (1, N):
        raise ValueError(f"gemm_fp8: scale sizes {sa.numel()}, {sb.numel()} do not match M={M}, N={N}")
    if accumulate and out is None:
        raise ValueError("gemm_fp8: accumulate needs the tensor to add into (out=)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype, device=a.device)
    elif tuple(out.shape) != (M, N) or out.dtype != out_dtype or out.stride(1) != 1 or out.device != a.device:
        raise ValueError(f"gemm_fp8: out must be a [{M}, {N}] {out_dtype} tensor with contiguous rows on {a.device}")
    elif not out.is_inference():
        # the kernels write through the raw pointer: tell autograd and any cache keyed on the version counter
        torch._C._increment_version((out,))
    sink = GEMM_EVENT_SINK
    if sink is not None:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
    L = _C.lib()
    if accumulate and variant < 0 and splits != 1 and L.mi8_gemm_splitk_suggest(M, N, K) > 1:
        # few output tiles: the plain call cuts K into slices (another summation order); the sum keeps its bits
        return out.add_(gemm_fp8(a, sa, b, sb, k=K, out_dtype=out_dtype, splits=splits))
    if accumulate:
        _C.check(
            L.mi8_gemm_fp8_accumulate(
                a.data_ptr(), _FP8_CODE[a.dtype], a.stride(0), b.data_ptr(), _FP8_CODE[b.dtype], b.stride(0), M, N, K,
                sa.data_ptr(), int(sa.numel() != 1), sb.data_ptr(), int(sb.numel() != 1),
                out.data_ptr(), _HP_CODE[out_dtype], out.stride(0), _stream(a),
            ),
            "mi8_gemm_fp8_accumulate",
        )
        if sink is not None:
            ev1.record()
            sink.append((ev0, ev1, (M, N, K)))
        return out
    if variant >= 0:
        splits = 1
    elif splits < 0:
        splits = L.mi8_gemm_splitk_suggest(M, N, K)
    if splits > 1:
        # the planes come from torch's caching allocator: reuse is ordered on the stream like any other tensor
        planes = torch.empty(L.mi8_gemm_splitk_workspace_bytes(M, N, splits), dtype=torch.uint8, device=a.device)
        _C.check(
            L.mi8_gemm_fp8_splitk(
                a.data_ptr(), _FP8_CODE[a.dtype], a.stride(0), b.data_ptr(), _FP8_CODE[b.dtype], b.stride(0), M, N, K,
                sa.data_ptr(), int(sa.numel() != 1),
                sb.data_ptr(), int(sb.numel() != 1),
                out.data_ptr(), _HP_CODE[out_dtype], out.stride(0), splits, planes.data_ptr(), planes.numel(),
                _stream(a),
            ),
            "mi8_gemm_fp8_splitk",
        )
    else:
        _C.check(
            L.mi8_gemm_fp8(
                a.data_ptr(), _FP8_CODE[a.dtype], a.stride(0), b.data_ptr(), _FP8_CODE[b.dtype], b.stride(0), M, N, K,
                sa.data_ptr(), int(sa.numel() != 1),
                sb.data_ptr(), int(sb.numel() != 1),
                out.data_ptr(), _HP_CODE[out_dtype], out.stride(0), variant, _stream(a),
            ),
            "mi8_gemm_fp8",
        )
    if sink is not None:
        ev1.record()
        sink.append((ev0, ev1, (M, N, K)))
    return out


def swiglu_gemm_supported(M: int, H: int, K: int) -> bool:
    """Shapes :func:`gemm_fp8_swiglu` takes (otherwise: two :func:`gemm_fp8` calls and :func:`swiglu_fwd`)."""
    return M >= 256 and H >= 128 and H % 8 == 0 and K % 128 == 0


def swiglu_gemm_matches_separate(M: int, H: int, K: int) -> bool:
    """Shapes for which :func:`gemm_fp8_swiglu` gives the bits of the three separate launches as the library
    dispatches them (large problems: both routes run the persistent tile kernel)."""
    return bool(_C.lib().mi8_gemm_fp8_swiglu_matches_separate(M, H, K))


def gemm_fp8_swiglu(a: torch.Tensor, sa: torch.Tensor, b1: torch.Tensor, sb1: torch.Tensor, b3: torch.Tensor,
                    sb3: torch.Tensor, *, k: Optional[int] = None, want_codes: bool = False):
    """
    ``x1 = a @ b1.T``, ``x3 = a @ b3.T`` (scaled, bf16) and ``h = silu(x1) * x3`` from one launch, with the amax
    partials of ``h``: ``(x1, x3, h, (slots, n_slots))``, each bit-identical to :func:`gemm_fp8` / :func:`swiglu_fwd`.
    Single scales only (the tensorwise recipe).  ``want_codes`` (H % 64 == 0): a fifth result, the row-segment codes
    of the larger of ``x1`` and ``x3`` (:func:`rowseg_max_codes`), which the backward pass's
    :func:`swiglu_bwd_cast` takes.
    """
    _require_gpu(a, "gemm_fp8_swiglu")
    if a.dim() != 2 or b1.dim() != 2 or b1.shape != b3.shape or b1.dtype != b3.dtype or b1.stride(0) != b3.stride(0):
        raise ValueError("gemm_fp8_swiglu: b1 and b3 must be matrices of one shape, type and row pitch")
    if a.stride(1) != 1 or b1.stride(1) != 1 or b3.stride(1) != 1:
        raise ValueError("gemm_fp8_swiglu: operands must have contiguous rows")
    if a.dtype not in _FP8_CODE or b1.dtype not in _FP8_CODE:
        raise TypeError("gemm_fp8_swiglu: operands must be float8")
    if sa.numel() != 1 or sb1.numel() != 1 or sb3.numel() != 1:
        raise ValueError("gemm_fp8_swiglu: single scales only")
    M, H = a.shape[0], b1.shape[0]
    K = min(a.shape[1], b1.shape[1]) if k is None else k
    x1, x3, h = (torch.empty((M, H), dtype=torch.bfloat16, device=a.device) for _ in range(3))
    slots = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=a.device)
    used = _C.c_int32(0)
    codes = torch.empty(_C.lib().mi8_rowseg_code_count(M, H), dtype=torch.int16, device=a.device) if want_codes else None
    sink = GEMM_EVENT_SINK
    if sink is not None:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
    _C.check(
        _C.lib().mi8_gemm_fp8_swiglu(
            a.data_ptr(), _FP8_CODE[a.dtype], a.stride(0), b1.data_ptr(), b3.data_ptr(), _FP8_CODE[b1.dtype],
            b1.stride(0), M, H, K, sa.data_ptr(), sb1.data_ptr(), sb3.data_ptr(), x1.data_ptr(), x3.data_ptr(),
            h.data_ptr(), H, slots.data_ptr(), used, codes.data_ptr() if want_codes else None, _stream(a),
        ),
        "mi8_gemm_fp8_swiglu",
    )
    if sink is not None:
        ev1.record()
        sink.append((ev0, ev1, (M, 2 * H, K)))
    if want_codes:
        return x1, x3, h, (slots, used.value), codes
    return x1, x3, h, (slots, used.value)


def gemm_codes_supported(M: int, N: int, K: int) -> bool:
    """Shapes :func:`gemm_fp8_codes` takes (the result then has the bits of :func:`gemm_fp8`)."""
    return bool(_C.lib().mi8_gemm_fp8_codes_supported(M, N, K))


def gemm_fp8_codes(a: torch.Tensor, sa: torch.Tensor, b: torch.Tensor, sb: torch.Tensor, *, k: Optional[int] = None):
    """
    ``out = gemm_fp8(a, sa, b, sb)`` (single scales, bf16) together with the row-segment codes of ``out``
    (:func:`rowseg_max_codes`), written by the GEMM's epilogue.  Returns ``(out, codes)``.
    """
    _require_gpu(a, "gemm_fp8_codes")
    if a.dim() != 2 or b.dim() != 2 or a.stride(1) != 1 or b.stride(1) != 1:
        raise ValueError("gemm_fp8_codes: operands must be 2-D with contiguous rows")
    if a.dtype not in _FP8_CODE or b.dtype not in _FP8_CODE:
        raise TypeError("gemm_fp8_codes: operands must be float8")
    if sa.numel() != 1 or sb.numel() != 1:
        raise ValueError("gemm_fp8_codes: single scales only")
    M, N = a.shape[0], b.shape[0]
    K = min(a.shape[1], b.shape[1]) if k is None else k
    out = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    codes = torch.empty(_C.lib().mi8_rowseg_code_count(M, N), dtype=torch.int16, device=a.device)
    sink = GEMM_EVENT_SINK
    if sink is not None:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
    _C.check(
        _C.lib().mi8_gemm_fp8_codes(
            a.data_ptr(), _FP8_CODE[a.dtype], a.stride(0), b.data_ptr(), _FP8_CODE[b.dtype], b.stride(0), M, N, K,
            sa.data_ptr(), sb.data_ptr(), out.data_ptr(), N, codes.data_ptr(), _stream(a),
        ),
        "mi8_gemm_fp8_codes",
    )
    if sink is not None:
        ev1.record()
        sink.append((ev0, ev1, (M, N, K)))
    return out, codes


def gemm_variants() -> list:
    L = _C.lib()
    return [L.mi8_gemm_variant_name(i).decode() for i in range(L.mi8_gemm_num_variants())]


def swiglu_fwd(x1: torch.Tensor, x3: torch.Tensor, want_amax: bool = True):
    """h = silu(x1) * x3 (bf16); optionally the amax partials of h for the cast that follows."""
    _require_gpu(x1, "swiglu_fwd")
    if x1.dtype != torch.bfloat16 or x3.dtype != torch.bfloat16 or x1.shape != x3.shape:
        raise TypeError("swiglu_fwd: expects two bfloat16 tensors of the same shape")
    x1, x3 = x1.contiguous(), x3.contiguous()
    h = torch.empty_like(x1)
    slots = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=x1.device) if want_amax else None
    n = x1.numel()
    _C.check(
        _C.lib().mi8_swiglu_fwd(
            x1.data_ptr(), x3.data_ptr(), h.data_ptr(), n, slots.data_ptr() if want_amax else None, _stream(x1)
        ),
        "mi8_swiglu_fwd",
    )
    return h, ((slots, _C.lib().mi8_amax_slots_for(n)) if want_amax else None)


def swiglu_bwd(x1: torch.Tensor, x3: torch.Tensor, gh: torch.Tensor, want_amax: bool = True):
    """Gradients of h = silu(x1) * x3 w.r.t. x1 and x3 (bf16) and optionally their amax partials."""
    _require_gpu(x1, "swiglu_bwd")
    x1, x3, gh = x1.contiguous(), x3.contiguous(), gh.contiguous()
    g1, g3 = torch.empty_like(x1), torch.empty_like(x1)
    n = x1.numel()
    s1 = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=x1.device) if want_amax else None
    s3 = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=x1.device) if want_amax else None
    _C.check(
        _C.lib().mi8_swiglu_bwd(
            x1.data_ptr(), x3.data_ptr(), gh.data_ptr(), g1.data_ptr(), g3.data_ptr(), n,
            s1.data_ptr() if want_amax else None, s3.data_ptr() if want_amax else None, _stream(x1),
        ),
        "mi8_swiglu_bwd",
    )
    used = _C.lib().mi8_amax_slots_for(n)
    return g1, g3, ((s1, used) if want_amax else None), ((s3, used) if want_amax else None)


def rowseg_max_codes(a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One 16-bit code per row segment (64 consecutive columns of a row) of a bf16 matrix: the largest magnitude in
    it (of ``a``, or of ``a`` and ``b``), as the integer formed by the exponent and mantissa bits; int16
    ``[ceil(cols / 64) * rows]``, the codes of one column block contiguous over the rows."""
    _require_gpu(a, "rowseg_max_codes")
    if a.dtype != torch.bfloat16 or a.dim() != 2 or (b is not None and (b.dtype != a.dtype or b.shape != a.shape)):
        raise ValueError("rowseg_max_codes expects one or two bfloat16 matrices of one shape")
    a = a.contiguous()
    b = b.contiguous() if b is not None else None
    rows, cols = a.shape
    codes = torch.empty(_C.lib().mi8_rowseg_code_count(rows, cols), dtype=torch.int16, device=a.device)
    _C.check(
        _C.lib().mi8_rowseg_max_codes(a.data_ptr(), b.data_ptr() if b is not None else None, rows, cols, codes.data_ptr(),
                                      _stream(a)),
        "mi8_rowseg_max_codes",
    )
    return codes


def swiglu_bwd_amax_from_codes(x1: torch.Tensor, x3: torch.Tensor, gh: torch.Tensor, gh_codes: torch.Tensor,
                               x_codes: torch.Tensor) -> torch.Tensor:
    """The amax of g1 and g3 (float32 bit patterns in words 0 and 1 of the returned int32 array), computing only the
    row segments whose codes say they could raise it; equal to the maxima of :func:`swiglu_bwd`'s partials."""
    _require_gpu(x1, "swiglu_bwd_amax_from_codes")
    rows, cols = x1.shape
    n = _C.lib().mi8_rowseg_code_count(rows, cols)
    for c in (gh_codes, x_codes):
        if c.dtype != torch.int16 or c.numel() != n or not c.is_contiguous() or c.device != x1.device:
            raise ValueError("swiglu_bwd_amax_from_codes: codes must be the int16 arrays of rowseg_max_codes for this shape")
    state = torch.empty(_C.lib().mi8_swiglu_amax_state_words(rows, cols), dtype=torch.int32, device=x1.device)
    _C.check(
        _C.lib().mi8_swiglu_bwd_amax_from_codes(x1.data_ptr(), x3.data_ptr(), gh.data_ptr(), rows, cols, gh_codes.data_ptr(),
                                                x_codes.data_ptr(), state.data_ptr(), _stream(x1)),
        "mi8_swiglu_bwd_amax_from_codes",
    )
    return state


def swiglu_bwd_cast(
    x1: torch.Tensor, x3: torch.Tensor, gh: torch.Tensor, fp8_dtype: torch.dtype, *, pow2: bool = False,
    want_rowmajor: bool = True, want_transposed: bool = False, codes: Optional[tuple] = None,
):
    """
    ``swiglu_bwd`` followed by ``cast_tensorwise`` of both gradients, without ever writing them in bf16: a first
    pass takes only their amax, a second recomputes them tile by tile and writes the fp8 copies.  Returns
    ``(g1q, g1q_t, scale1, g3q, g3q_t, scale3)`` with the bytes and scales of the two-step route.
    ``codes`` = ``(gh_codes, x_codes)`` (from :func:`gemm_fp8_codes` / :func:`gemm_fp8_swiglu`, or
    :func:`rowseg_max_codes`): the amax is then found by computing only the row segments that can hold it, instead
    of by the pass over all three tensors.
    """
    _require_gpu(x1, "swiglu_bwd_cast")
    if not (x1.dtype == x3.dtype == gh.dtype == torch.bfloat16) or not (x1.shape == x3.shape == gh.shape) or x1.dim() != 2:
        raise ValueError("swiglu_bwd_cast expects three bfloat16 matrices of one shape")
    if not (want_rowmajor or want_transposed):
        raise ValueError("swiglu_bwd_cast: no output requested")
    x1, x3, gh = x1.contiguous(), x3.contiguous(), gh.contiguous()
    rows, cols = x1.shape
    dev = x1.device
    n = x1.numel()
    if codes is not None:
        state = swiglu_bwd_amax_from_codes(x1, x3, gh, codes[0], codes[1])
        s1, s3, used = state[0:1], state[1:2], 1
    else:
        s1 = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=dev)
        s3 = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=dev)
        _C.check(
            _C.lib().mi8_swiglu_bwd(x1.data_ptr(), x3.data_ptr(), gh.data_ptr(), None, None, n, s1.data_ptr(), s3.data_ptr(),
                                    _stream(x1)),
            "mi8_swiglu_bwd",
        )
        used = _C.lib().mi8_amax_slots_for(n)
    q = [_operand((rows, cols), fp8_dtype, dev) if want_rowmajor else None for _ in range(2)]
    q_t = [_operand((cols, pad16(rows)), fp8_dtype, dev) if want_transposed else None for _ in range(2)]
    scales = [torch.empty(1, dtype=torch.float32, device=dev) for _ in range(2)]
    ptr = lambda t: t.data_ptr() if t is not None else None  # noqa: E731
    _C.check(
        _C.lib().mi8_swiglu_bwd_cast(
            x1.data_ptr(), x3.data_ptr(), gh.data_ptr(), rows, cols, s1.data_ptr(), s3.data_ptr(), used,
            _FP8_CODE[fp8_dtype], _flags(pow2), ptr(q[0]), ptr(q[1]), q[0].stride(0) if want_rowmajor else 0,
            ptr(q_t[0]), ptr(q_t[1]), q_t[0].stride(0) if want_transposed else 0,
            scales[0].data_ptr(), scales[1].data_ptr(), _stream(x1),
        ),
        "mi8_swiglu_bwd_cast",
    )
    return q[0], q_t[0], scales[0], q[1], q_t[1], scales[1]


# ---- ragged grouped operations (dropless-MoE expert layer) -------------------------------------------


def grouped_padded_rows(T: int, num_groups: int) -> int:
    return _C.lib().mi8_grouped_padded_rows(T, num_groups)


def _sizes_i64(group_sizes: torch.Tensor, dev) -> torch.Tensor:
    if group_sizes.dim() != 1:
        raise ValueError("group sizes must be a 1-D tensor")
    if group_sizes.device != dev or group_sizes.dtype != torch.int64 or not group_sizes.is_contiguous():
        group_sizes = group_sizes.to(device=dev, dtype=torch.int64).contiguous()
    return group_sizes


def grouped_cast_colwise_t(
    x: torch.Tensor, group_sizes: torch.Tensor, fp8_dtype: torch.dtype, *, pow2: bool = False
) -> Tuple[torch.Tensor, torch.Tensor]:
    """
    Per-group, per-column cast with transposed output.  ``x [T, cols]``, rows grouped consecutively by
    ``group_sizes [E]`` (int64, on the device).  Returns ``(q_t [cols, ld_t], scale [E, cols])`` where group e's
    bytes start at column ``128 * (number of 128-row tiles of the groups before it)`` and the padding is zero.
    """
    x = _hp2d(x, "grouped_cast_colwise_t")
    T, cols = x.shape
    sizes = _sizes_i64(group_sizes, x.device)
    E = sizes.numel()
    ld_t = grouped_padded_rows(T, E)
    q_t = torch.empty((cols, ld_t), dtype=fp8_dtype, device=x.device)
    scale = torch.empty((E, cols), dtype=torch.float32, device=x.device)
    ws = torch.zeros(E * cols, dtype=torch.int32, device=x.device)
    _C.check(
        _C.lib().mi8_grouped_cast_colwise_t(
            x.data_ptr(), _HP_CODE[x.dtype], T, cols, sizes.data_ptr(), E, _FP8_CODE[fp8_dtype], _flags(pow2),
            ws.data_ptr(), q_t.data_ptr(), ld_t, scale.data_ptr(), _stream(x),
        ),
        "mi8_grouped_cast_colwise_t",
    )
    return q_t, scale


def _grouped_amax_workspace(T: int, cols: int, E: int, device) -> torch.Tensor:
    """Zeroed ``uint32[E * cols + T]``: the per-(group, column) amax table followed by the per-row one."""
    return torch.zeros(E * cols + T, dtype=torch.int32, device=device)


def grouped_swiglu_fwd(x1: torch.Tensor, x2: torch.Tensor, group_sizes: torch.Tensor):
    """``h = silu(x1) * x2`` (bf16, ``[T, cols]``, rows grouped by ``group_sizes``) plus the amax workspace of ``h``
    that :func:`grouped_cast_rows_and_colwise_t` takes as ``amax``: the cast then needs one pass instead of two."""
    _require_gpu(x1, "grouped_swiglu_fwd")
    if x1.dtype != torch.bfloat16 or x2.dtype != torch.bfloat16 or x1.shape != x2.shape or x1.dim() != 2:
        raise ValueError("grouped_swiglu_fwd expects two bfloat16 matrices of one shape")
    x1, x2 = x1.contiguous(), x2.contiguous()
    T, cols = x1.shape
    sizes = _sizes_i64(group_sizes, x1.device)
    E = sizes.numel()
    h = torch.empty_like(x1)
    ws = _grouped_amax_workspace(T, cols, E, x1.device)
    _C.check(
        _C.lib().mi8_grouped_swiglu_fwd(x1.data_ptr(), x2.data_ptr(), T, cols, sizes.data_ptr(), E, h.data_ptr(),
                                        ws.data_ptr(), ws.data_ptr() + 4 * E * cols, _stream(x1)),
        "mi8_grouped_swiglu_fwd",
    )
    return h, ws


def grouped_swiglu_bwd(x1: torch.Tensor, x2: torch.Tensor, gh: torch.Tensor, group_sizes: torch.Tensor):
    """Gradients ``(g1, g2)`` of ``silu(x1) * x2`` for the incoming ``gh`` plus one amax workspace each (see
    :func:`grouped_swiglu_fwd`)."""
    _require_gpu(x1, "grouped_swiglu_bwd")
    if not (x1.dtype == x2.dtype == gh.dtype == torch.bfloat16) or not (x1.shape == x2.shape == gh.shape) or x1.dim() != 2:
        raise ValueError("grouped_swiglu_bwd expects three bfloat16 matrices of one shape")
    x1, x2, gh = x1.contiguous(), x2.contiguous(), gh.contiguous()
    T, cols = x1.shape
    sizes = _sizes_i64(group_sizes, x1.device)
    E = sizes.numel()
    g1, g2 = torch.empty_like(x1), torch.empty_like(x1)
    ws1 = _grouped_amax_workspace(T, cols, E, x1.device)
    ws2 = _grouped_amax_workspace(T, cols, E, x1.device)
    _C.check(
        _C.lib().mi8_grouped_swiglu_bwd(x1.data_ptr(), x2.data_ptr(), gh.data_ptr(), T, cols, sizes.data_ptr(), E,
                                        g1.data_ptr(), g2.data_ptr(), ws1.data_ptr(), ws1.data_ptr() + 4 * E * cols,
                                        ws2.data_ptr(), ws2.data_ptr() + 4 * E * cols, _stream(x1)),
        "mi8_grouped_swiglu_bwd",
    )
    return g1, g2, ws1, ws2


def grouped_cast_rows_and_colwise_t(
    x: torch.Tensor, group_sizes: torch.Tensor, fp8_dtype: torch.dtype, *, pow2: bool = False,
    amax: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """
    :func:`cast_rowwise` and :func:`grouped_cast_colwise_t` of the same tensor in one pair of passes:
    ``(q [T, cols], row_scale [T], q_t [cols, ld_t], col_scale [E, cols])``.  The group sizes must sum to ``T``
    (rows after the last group are left unwritten).  ``amax``: the workspace returned with ``x`` by
    :func:`grouped_swiglu_fwd` / :func:`grouped_swiglu_bwd`; the amax pass is then skipped.
    """
    x = _hp2d(x, "grouped_cast_rows_and_colwise_t")
    T, cols = x.shape
    sizes = _sizes_i64(group_sizes, x.device)
    E = sizes.numel()
    ld_t = grouped_padded_rows(T, E)
    q_t = torch.empty((cols, ld_t), dtype=fp8_dtype, device=x.device)
    scale = torch.empty((E, cols), dtype=torch.float32, device=x.device)
    q = torch.empty((T, cols), dtype=fp8_dtype, device=x.device)
    row_scale = torch.empty(T, dtype=torch.float32, device=x.device)
    flags = _flags(pow2)
    if amax is None:
        ws = _grouped_amax_workspace(T, cols, E, x.device)
    else:
        if amax.numel() != E * cols + T or amax.dtype != torch.int32 or amax.device != x.device:
            raise ValueError("amax must be the workspace returned by grouped_swiglu_fwd/bwd for this tensor")
        ws = amax
        flags |= _C.FLAG_AMAX_READY
    _C.check(
        _C.lib().mi8_grouped_cast_rows_and_colwise_t(
            x.data_ptr(), _HP_CODE[x.dtype], T, cols, sizes.data_ptr(), E, _FP8_CODE[fp8_dtype], flags,
            ws.data_ptr(), q_t.data_ptr(), ld_t, scale.data_ptr(), ws.data_ptr() + 4 * E * cols, q.data_ptr(), cols,
            row_scale.data_ptr(), _stream(x),
        ),
        "mi8_grouped_cast_rows_and_colwise_t",
    )
    return q, row_scale, q_t, scale


def gather_cast_rows_and_colwise_t(
    x: torch.Tensor, indices: torch.Tensor, top_k: int, group_sizes: torch.Tensor, fp8_dtype: torch.dtype, *,
    pow2: bool = False, weights: Optional[torch.Tensor] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """
    The token gather of a dropless-MoE layer (``weights``, one per slot: every gathered row times its slot's weight,
    rounded to the element type - the backward of the weighted scatter) (row ``i`` of the expert-sorted side is token
    ``indices[i] // top_k`` of ``x [tokens, cols]``) fused with :func:`grouped_cast_rows_and_colwise_t`: the gathered
    bf16 tensor is never written.  Returns ``(q [tokens * top_k, cols], row_scale, q_t [cols, ld_t], col_scale [E, cols])``
    with the bytes and scales of the two-step route.
    """
    x = _hp2d(x, "gather_cast_rows_and_colwise_t")
    tokens, cols = x.shape
    T = tokens * top_k
    if indices.dim() != 1 or indices.shape[0] != T or indices.device != x.device:
        raise ValueError(f"gather_cast_rows_and_colwise_t: expected {T} indices on {x.device}")
    if indices.dtype != torch.int32 or not indices.is_contiguous():
        indices = indices.to(torch.int32).contiguous()
    sizes = _sizes_i64(group_sizes, x.device)
    E = sizes.numel()
    ld_t = grouped_padded_rows(T, E)
    q_t = torch.empty((cols, ld_t), dtype=fp8_dtype, device=x.device)
    scale = torch.empty((E, cols), dtype=torch.float32, device=x.device)
    q = torch.empty((T, cols), dtype=fp8_dtype, device=x.device)
    row_scale = torch.empty(T, dtype=torch.float32, device=x.device)
    ws = _grouped_amax_workspace(T, cols, E, x.device)
    wp, wd = None, 0
    if weights is not None:
        if weights.dim() != 1 or weights.shape[0] != T or weights.device != x.device:
            raise ValueError(f"gather_cast_rows_and_colwise_t: expected {T} weights on {x.device}")
        weights = weights.contiguous()
        wd = {torch.bfloat16: _C.MI8_BF16, torch.float32: _C.MI8_F32, torch.float16: _C.MI8_F16}[weights.dtype]
        wp = weights.data_ptr()
    _C.check(
        _C.lib().mi8_moe_gather_cast_rows_and_colwise_t(
            x.data_ptr(), _HP_CODE[x.dtype], tokens, cols, indices.data_ptr(), top_k, wp, wd, sizes.data_ptr(), E,
            _FP8_CODE[fp8_dtype], _flags(pow2), ws.data_ptr(), q_t.data_ptr(), ld_t, scale.data_ptr(),
            ws.data_ptr() + 4 * E * cols, q.data_ptr(), cols, row_scale.data_ptr(), _stream(x),
        ),
        "mi8_moe_gather_cast_rows_and_colwise_t",
    )
    return q, row_scale, q_t, scale


_ONE_GROUP: dict = {}


def cast_rows_and_colwise_t(
    x: torch.Tensor, fp8_dtype: torch.dtype, *, pow2: bool = False
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """
    :func:`cast_rowwise` and :func:`cast_colwise_t` of one tensor from one pair of passes (the grouped two-product
    cast with a single group): ``(q [rows, cols], row_scale [rows], q_t [cols, rows rounded up to 128], col_scale
    [cols])``; ``q_t`` is zero beyond ``rows``.  Bytes and scales are those of the two separate casts.
    """
    x = _hp2d(x, "cast_rows_and_colwise_t")
    # one group that takes every row: the kernels clamp group sizes to the rows that exist, so one device-resident
    # "all of them" serves every shape (no host-to-device copy per call, none at all after the first)
    sizes = _ONE_GROUP.get(x.device)
    if sizes is None:
        sizes = _ONE_GROUP[x.device] = torch.tensor([1 << 62], dtype=torch.int64, device=x.device)
    q, row_scale, q_t, col_scale = grouped_cast_rows_and_colwise_t(x, sizes, fp8_dtype, pow2=pow2)
    return q, row_scale, q_t, col_scale.reshape(-1)


def grouped_gemm_fp8(
    a: torch.Tensor,
    sa: torch.Tensor,
    b: torch.Tensor,
    sb: torch.Tensor,
    group_sizes: torch.Tensor,
    *,
    n: int,
    k: int,
    b_group_stride: int,
    sb_group_stride: int,
    out_dtype: torch.dtype = torch.bfloat16,
    accumulate_into: Optional[torch.Tensor] = None,
) -> torch.Tensor:
    """
    ``out[rows of group e] = a[rows of group e, :k] @ B_e[:n, :k].T / sa / sb_e`` where ``B_e`` starts
    ``e * b_group_stride`` bytes into ``b`` (row pitch ``b.stride(0)``) and its scales ``e * sb_group_stride``
    floats into ``sb``.  ``accumulate_into``: a ``[T, n]`` tensor of ``out_dtype`` that the product is added to (the
    bits of ``accumulate_into + grouped_gemm_fp8(...)``) and that is returned.
    """
    _require_gpu(a, "grouped_gemm_fp8")
    T = a.shape[0]
    sizes = _sizes_i64(group_sizes, a.device)
    if accumulate_into is not None:
        out = accumulate_into
        if tuple(out.shape) != (T, n) or out.dtype != out_dtype or out.stride(1) != 1 or out.device != a.device:
            raise ValueError(f"grouped_gemm_fp8: accumulate_into must be a [{T}, {n}] {out_dtype} tensor on {a.device}")
        if not out.is_inference():
            torch._C._increment_version((out,))
        fn, what = _C.lib().mi8_grouped_gemm_fp8_accumulate, "mi8_grouped_gemm_fp8_accumulate"
    else:
        out = torch.empty((T, n), dtype=out_dtype, device=a.device)
        fn, what = _C.lib().mi8_grouped_gemm_fp8, "mi8_grouped_gemm_fp8"
    _C.check(
        fn(
            a.data_ptr(), _FP8_CODE[a.dtype], a.stride(0), b.data_ptr(), _FP8_CODE[b.dtype], b.stride(0),
            b_group_stride, sizes.data_ptr(), sizes.numel(), T, n, k, sa.data_ptr(), sb.data_ptr(), sb_group_stride,
            out.data_ptr(), _HP_CODE[out_dtype], out.stride(0), _stream(a),
        ),
        what,
    )
    return out


def grouped_gemm_dual_supported(T: int, n: int, k1: int, k2: int) -> bool:
    """Shapes :func:`grouped_gemm_fp8_dual` takes."""
    return bool(_C.lib().mi8_grouped_gemm_fp8_dual_supported(T, n, k1, k2))


def grouped_gemm_fp8_dual(
    a1: torch.Tensor, sa1: torch.Tensor, b1: torch.Tensor, sb1: torch.Tensor,
    a2: torch.Tensor, sa2: torch.Tensor, b2: torch.Tensor, sb2: torch.Tensor,
    group_sizes: torch.Tensor, *, n: int, k1: int, k2: int, b_group_stride: int, sb_group_stride: int,
) -> torch.Tensor:
    """
    ``out[rows of group e] = a1 @ B1_e.T / sa1 / sb1_e + a2 @ B2_e.T / sa2 / sb2_e`` (bf16), both products in one
    float32 accumulation: one launch in place of :func:`grouped_gemm_fp8` followed by its accumulating form.  All scales
    must be exact powers of two (casts made with ``pow2=True``).  ``a1`` / ``a2`` and ``b1`` / ``b2`` must share their
    row pitches; ``B_e`` starts ``e * b_group_stride`` bytes into ``b``, its scales ``e * sb_group_stride`` floats into
    ``sb``.
    """
    _require_gpu(a1, "grouped_gemm_fp8_dual")
    T = a1.shape[0]
    if a2.shape[0] != T or a1.stride(0) != a2.stride(0) or b1.stride(0) != b2.stride(0) or a1.dtype != a2.dtype or b1.dtype != b2.dtype:
        raise ValueError("grouped_gemm_fp8_dual: the two left operands and the two right operands must share rows, pitch and type")
    if a1.stride(1) != 1 or a2.stride(1) != 1 or b1.stride(1) != 1 or b2.stride(1) != 1:
        raise ValueError("grouped_gemm_fp8_dual: operands must have contiguous rows")
    if sa1.numel() != T or sa2.numel() != T or sb1.shape != sb2.shape:
        raise ValueError("grouped_gemm_fp8_dual: one scale per row of a1 / a2, column scales of one shape")
    sizes = _sizes_i64(group_sizes, a1.device)
    out = torch.empty((T, n), dtype=torch.bfloat16, device=a1.device)
    _C.check(
        _C.lib().mi8_grouped_gemm_fp8_dual(
            a1.data_ptr(), a2.data_ptr(), _FP8_CODE[a1.dtype], a1.stride(0), b1.data_ptr(), b2.data_ptr(), _FP8_CODE[b1.dtype],
            b1.stride(0), b_group_stride, sizes.data_ptr(), sizes.numel(), T, n, k1, k2, sa1.data_ptr(), sa2.data_ptr(),
            sb1.data_ptr(), sb2.data_ptr(), sb_group_stride, out.data_ptr(), out.stride(0), _stream(a1),
        ),
        "mi8_grouped_gemm_fp8_dual",
    )
    return out


def grouped_wgrad_fp8(
    a_t: torch.Tensor,
    sa: torch.Tensor,
    b_t: torch.Tensor,
    sb: torch.Tensor,
    group_sizes: torch.Tensor,
    *,
    tokens: int,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """``out[e] = a_t[:, seg_e] @ b_t[:, seg_e].T / sa[e] / sb[e]`` -> ``[E, a_t.shape[0], b_t.shape[0]]``."""
    _require_gpu(a_t, "grouped_wgrad_fp8")
    sizes = _sizes_i64(group_sizes, a_t.device)
    E, N, Kl = sizes.numel(), a_t.shape[0], b_t.shape[0]
    if a_t.stride(0) != b_t.stride(0):
        raise ValueError("grouped_wgrad_fp8: both operands must share the padded token pitch")
    out = torch.empty((E, N, Kl), dtype=out_dtype, device=a_t.device)
    _C.check(
        _C.lib().mi8_grouped_wgrad_fp8(
            a_t.data_ptr(), _FP8_CODE[a_t.dtype], b_t.data_ptr(), _FP8_CODE[b_t.dtype], a_t.stride(0),
            sizes.data_ptr(), E, tokens, N, Kl, sa.data_ptr(), sb.data_ptr(), out.data_ptr(), _HP_CODE[out_dtype],
            _stream(a_t),
        ),
        "mi8_grouped_wgrad_fp8",
    )
    return out

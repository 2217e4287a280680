"""
MoE token-permutation ops: the interface of ``olmo_core.ops.moe`` (reference ``src/olmo_core/ops/moe.py:26-205``,
``:289-304``) on the HIP kernels of ``csrc/mi8_permute.hip`` (which replace the Triton kernels of
``src/olmo_core/kernels/moe.py``).

Same functions, argument order and gradients as the reference:

* ``gather(x, indices, bin_ids, bins, top_k)``            -> ``[tokens * top_k, hidden]`` rows sorted by expert
* ``scatter(x, indices, bin_ids, weights, bins, top_k)``  -> ``[tokens, hidden]`` weighted sum over a token's slots
* ``binned_gather(x, indices, bins, bin_size, top_k)``    -> ``[experts, bin_size, hidden]``
* ``binned_scatter(x, indices, weights, bins, top_k)``    -> ``[tokens, hidden]``
* ``batched_histc(x, num_classes)``, ``histc(x, num_classes)``

``bin_ids`` is accepted for signature compatibility; the dropless kernels do not need it (row ``i`` of the sorted
side is row ``i`` of ``indices``).  Tensors must live on the GPU; there is no CPU path.
"""

from __future__ import annotations

from typing import Any, Optional

import torch

from .. import _C

_DT = {torch.bfloat16: _C.MI8_BF16, torch.float32: _C.MI8_F32, torch.float16: _C.MI8_F16}
_RAW = (torch.float8_e4m3fn, torch.float8_e5m2, torch.uint8, torch.int8)


def _stream(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _dt(x: torch.Tensor, what: str, allow_raw: bool = False) -> int:
    if not x.is_cuda:
        raise RuntimeError(f"{what}: tensors must live on the GPU (the permutation ops have no CPU implementation)")
    if x.dtype in _DT:
        return _DT[x.dtype]
    if allow_raw and x.dtype in _RAW:
        return _C.MI8_RAW8
    raise TypeError(f"{what}: unsupported element type {x.dtype}")


def _i32(t: torch.Tensor, what: str) -> torch.Tensor:
    if t.dim() != 1:
        raise ValueError(f"{what}: expected a vector, got {t.dim()} dimensions")
    return t if (t.dtype == torch.int32 and t.is_contiguous()) else t.to(torch.int32).contiguous()


def _weights(w: Optional[torch.Tensor], n: int, what: str):
    if w is None:
        return None, None, 0
    if w.dim() != 1 or w.shape[0] != n:
        raise ValueError(f"{what}: expected {n} weights, got {tuple(w.shape)}")
    w = w.contiguous()
    return w, w.data_ptr(), _dt(w, what)


# ---- kernels (no autograd) -----------------------------------------------------------------------------------


def _gather(x, indices, weights, top_k: int) -> torch.Tensor:
    if x.dim() != 2:
        raise ValueError(f"gather: expected a matrix, got {x.dim()} dimensions")
    x = x.contiguous()
    tokens, hidden = x.shape
    indices = _i32(indices, "gather")
    if indices.shape[0] != tokens * top_k:
        raise ValueError(f"gather: expected {tokens * top_k} indices, got {indices.shape[0]}")
    w, wp, wd = _weights(weights, tokens * top_k, "gather")
    out = torch.empty((tokens * top_k, hidden), dtype=x.dtype, device=x.device)
    if out.numel():
        _C.check(
            _C.lib().mi8_moe_gather(x.data_ptr(), _dt(x, "gather", allow_raw=w is None), tokens, hidden,
                                    indices.data_ptr(), wp, wd, top_k, out.data_ptr(), _stream(x)),
            "mi8_moe_gather",
        )
    return out


def _scatter(x, indices, weights, top_k: int) -> torch.Tensor:
    if x.dim() != 2:
        raise ValueError(f"scatter: expected a matrix, got {x.dim()} dimensions")
    x = x.contiguous()
    n, hidden = x.shape
    indices = _i32(indices, "scatter")
    if indices.shape[0] != n or n % top_k:
        raise ValueError(f"scatter: {n} rows, {indices.shape[0]} indices, top_k {top_k} do not fit together")
    tokens = n // top_k
    w, wp, wd = _weights(weights, n, "scatter")
    out = torch.empty((tokens, hidden), dtype=x.dtype, device=x.device)
    if out.numel():
        inverse = torch.empty(n, dtype=torch.int32, device=x.device)
        _C.check(
            _C.lib().mi8_moe_scatter(x.data_ptr(), _dt(x, "scatter"), tokens, hidden, indices.data_ptr(), wp, wd, top_k,
                                     inverse.data_ptr(), out.data_ptr(), _stream(x)),
            "mi8_moe_scatter",
        )
    return out


def _scatter_wgrad(x, grad, indices, top_k: int) -> torch.Tensor:
    x, grad = x.contiguous(), grad.contiguous()
    n, hidden = x.shape
    indices = _i32(indices, "scatter_wgrad")
    tokens = n // top_k
    if grad.shape != (tokens, hidden) or grad.dtype != x.dtype:
        raise ValueError(f"scatter_wgrad: grad {tuple(grad.shape)} {grad.dtype} does not match x {tuple(x.shape)} {x.dtype}")
    out = torch.empty(n, dtype=x.dtype, device=x.device)
    if n and hidden:
        _C.check(
            _C.lib().mi8_moe_scatter_wgrad(x.data_ptr(), grad.data_ptr(), _dt(x, "scatter_wgrad"), tokens, hidden,
                                           indices.data_ptr(), top_k, out.data_ptr(), _stream(x)),
            "mi8_moe_scatter_wgrad",
        )
    return out


def _binned_gather(x, indices, weights, bins, bin_size: int, top_k: int) -> torch.Tensor:
    if x.dim() != 2:
        raise ValueError(f"binned_gather: expected a matrix, got {x.dim()} dimensions")
    x = x.contiguous()
    tokens, hidden = x.shape
    indices, bins = _i32(indices, "binned_gather"), _i32(bins, "binned_gather")
    if indices.shape[0] != tokens * top_k:
        raise ValueError(f"binned_gather: expected {tokens * top_k} indices, got {indices.shape[0]}")
    w, wp, wd = _weights(weights, tokens * top_k, "binned_gather")
    experts = bins.shape[0]
    out = torch.empty((experts, bin_size, hidden), dtype=x.dtype, device=x.device)
    if out.numel():
        _C.check(
            _C.lib().mi8_moe_binned_gather(x.data_ptr(), _dt(x, "binned_gather", allow_raw=w is None), tokens, hidden,
                                           indices.data_ptr(), wp, wd, bins.data_ptr(), experts, bin_size, top_k,
                                           out.data_ptr(), _stream(x)),
            "mi8_moe_binned_gather",
        )
    return out


def _binned_scatter(x, indices, weights, bins, top_k: int) -> torch.Tensor:
    if x.dim() != 3:
        raise ValueError(f"binned_scatter: expected a 3-tensor, got {x.dim()} dimensions")
    x = x.contiguous()
    experts, bin_size, hidden = x.shape
    indices, bins = _i32(indices, "binned_scatter"), _i32(bins, "binned_scatter")
    if bins.shape[0] != experts or indices.shape[0] % top_k:
        raise ValueError("binned_scatter: bins / indices do not match x and top_k")
    n = indices.shape[0]
    tokens = n // top_k
    w, wp, wd = _weights(weights, n, "binned_scatter")
    out = torch.empty((tokens, hidden), dtype=x.dtype, device=x.device)
    if out.numel():
        inverse = torch.empty(n, dtype=torch.int32, device=x.device)
        _C.check(
            _C.lib().mi8_moe_binned_scatter(x.data_ptr(), _dt(x, "binned_scatter"), tokens, hidden, indices.data_ptr(),
                                            wp, wd, bins.data_ptr(), experts, bin_size, top_k, inverse.data_ptr(),
                                            out.data_ptr(), _stream(x)),
            "mi8_moe_binned_scatter",
        )
    return out


def _binned_scatter_wgrad(x, grad, indices, bins, top_k: int) -> torch.Tensor:
    x, grad = x.contiguous(), grad.contiguous()
    experts, bin_size, hidden = x.shape
    indices, bins = _i32(indices, "binned_scatter_wgrad"), _i32(bins, "binned_scatter_wgrad")
    n = indices.shape[0]
    tokens = n // top_k
    if grad.shape != (tokens, hidden) or grad.dtype != x.dtype:
        raise ValueError("binned_scatter_wgrad: grad does not match x")
    out = torch.empty(n, dtype=x.dtype, device=x.device)
    if n:
        _C.check(
            _C.lib().mi8_moe_binned_scatter_wgrad(x.data_ptr(), grad.data_ptr(), _dt(x, "binned_scatter_wgrad"), tokens,
                                                  hidden, indices.data_ptr(), bins.data_ptr(), experts, bin_size, top_k,
                                                  out.data_ptr(), _stream(x)),
            "mi8_moe_binned_scatter_wgrad",
        )
    return out


# ---- autograd functions (reference: src/olmo_core/ops/moe.py:26-205) -------------------------------------------


class GatherOp(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx: Any, x, indices, bin_ids, bins, top_k: int):
        ctx.save_for_backward(indices)
        ctx.top_k = top_k
        return _gather(x, indices, None, top_k)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad):
        (indices,) = ctx.saved_tensors
        return _scatter(grad.contiguous(), indices, None, ctx.top_k), None, None, None, None


@torch.compiler.disable
def gather(x, indices, bin_ids, bins, top_k: int) -> torch.Tensor:
    return GatherOp.apply(x, indices, bin_ids, bins, top_k)


class ScatterOp(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx: Any, x, indices, bin_ids, weights, bins, top_k: int):
        maybe_x = [x] if ctx.needs_input_grad[3] else []
        ctx.save_for_backward(indices, weights, *maybe_x)
        ctx.top_k = top_k
        return _scatter(x, indices, weights, top_k)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad):
        grad = grad.contiguous()
        indices, weights = ctx.saved_tensors[:2]
        dgrad = _gather(grad, indices, weights, ctx.top_k) if ctx.needs_input_grad[0] else None
        wgrad = None
        if ctx.needs_input_grad[3]:
            wgrad = _scatter_wgrad(ctx.saved_tensors[-1], grad, indices, ctx.top_k)
        return dgrad, None, None, wgrad, None, None


@torch.compiler.disable
def scatter(x, indices, bin_ids, weights, bins, top_k: int) -> torch.Tensor:
    return ScatterOp.apply(x, indices, bin_ids, weights, bins, top_k)


class BinnedGatherOp(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx: Any, x, indices, bins, bin_size: int, top_k: int):
        ctx.save_for_backward(indices, bins)
        ctx.top_k = top_k
        return _binned_gather(x, indices, None, bins, bin_size, top_k)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad):
        indices, bins = ctx.saved_tensors
        return _binned_scatter(grad.contiguous(), indices, None, bins, ctx.top_k), None, None, None, None


@torch.compiler.disable
def binned_gather(x, indices, bins, bin_size: int, top_k: int) -> torch.Tensor:
    return BinnedGatherOp.apply(x, indices, bins, bin_size, top_k)


class BinnedScatterOp(torch.autograd.Function):
    @staticmethod
    @torch.amp.custom_fwd(device_type="cuda")
    def forward(ctx: Any, x, indices, weights, bins, top_k: int):
        if x.dim() != 3:
            raise ValueError("binned_scatter: expected a 3-tensor")
        ctx.bin_size = x.size(1)
        ctx.top_k = top_k
        ctx.save_for_backward(x, indices, weights, bins)
        return _binned_scatter(x, indices, weights, bins, top_k)

    @staticmethod
    @torch.amp.custom_bwd(device_type="cuda")
    def backward(ctx: Any, grad):
        grad = grad.contiguous()
        x, indices, weights, bins = ctx.saved_tensors
        out = _binned_gather(grad, indices, weights, bins, ctx.bin_size, ctx.top_k)
        wgrad = _binned_scatter_wgrad(x, grad, indices, bins, ctx.top_k) if ctx.needs_input_grad[2] else None
        return out, None, wgrad, None, None


@torch.compiler.disable
def binned_scatter(x, indices, weights, bins, top_k: int) -> torch.Tensor:
    return BinnedScatterOp.apply(x, indices, weights, bins, top_k)


def batched_histc(x: torch.Tensor, num_classes: int) -> torch.Tensor:
    """A batched ``torch.histc`` over the last axis (integer class ids in ``[0, num_classes)``)."""
    hist = torch.zeros((*x.shape[:-1], num_classes), dtype=x.dtype, device=x.device)
    hist.scatter_add_(-1, x, torch.ones_like(x))
    return hist


def histc(x: torch.Tensor, num_classes: int) -> torch.Tensor:
    return batched_histc(x.reshape(1, -1), num_classes).reshape(num_classes)

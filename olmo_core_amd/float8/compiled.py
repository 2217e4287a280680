"""
The float8 linear and the fused SwiGLU feed-forward block as registered custom operators, for ``torch.compile``.

A ctypes call is opaque to Dynamo; wrapped in ``torch.library.custom_op`` with a shape function it becomes one
node of the traced graph, so that compiled blocks (the reference compiles every transformer block,
``src/olmo_core/nn/transformer/block.py:78-79``) keep a single graph around their float8 linears.  The operators
call the same forward / backward routines as the eager ``autograd.Function``.
"""

from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from . import ops
from .linear import (_COMPILED_CONFIGS, _backward_impl, _forward_impl, _is_axiswise, _kept_weight_state,
                     _saves_quantised)

_CONFIGS = _COMPILED_CONFIGS  # configs travel through the operators as indices into this list


@torch.library.custom_op("olmo_core_amd::float8_linear_fwd", mutates_args=())
def _linear_fwd(
    x2: torch.Tensor, weight: torch.Tensor, weight_scale: Optional[torch.Tensor], cfg: int, need_gx: bool, need_gw: bool,
    module_id: int,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    # (module_id: the calling module, -1 for none; what it keeps for its weight - a scale refreshed after the optimizer
    # step, float8 copies - is used if still valid: same bytes and scales as quantising here)
    kept_scale, kept_ops = _kept_weight_state(module_id, weight)
    if weight_scale is None:
        weight_scale = kept_scale
    y, x_saved, w_saved = _forward_impl(x2, weight, _CONFIGS[cfg], weight_scale, need_gx, need_gw, kept_ops)
    xa, xb = x_saved if x_saved is not None else (x2.new_empty(0), x2.new_empty(0))
    wa, wb = w_saved if w_saved is not None else (x2.new_empty(0), x2.new_empty(0))
    return y, xa, xb, wa, wb


@_linear_fwd.register_fake
def _(x2, weight, weight_scale, cfg, need_gx, need_gw, module_id):
    c = _CONFIGS[cfg]
    M, K = x2.shape
    N = weight.shape[0]
    x_is_q, w_is_q = _saves_quantised(c, need_gx, need_gw)

    def saved(is_q, rows, cols, cast):
        if not is_q:
            return x2.new_empty(0), x2.new_empty(0)
        if _is_axiswise(cast):  # transposed copy padded to 128 rows, one scale per column
            return (x2.new_empty((cols, (rows + 127) // 128 * 128), dtype=cast.target_dtype),
                    x2.new_empty(cols, dtype=torch.float32))
        return x2.new_empty((cols, (rows + 15) // 16 * 16), dtype=cast.target_dtype), x2.new_empty(1, dtype=torch.float32)

    xa, xb = saved(x_is_q, M, K, c.cast_config_input)
    wa, wb = saved(w_is_q, N, K, c.cast_config_weight)
    return x2.new_empty((M, N)), xa, xb, wa, wb


@torch.library.custom_op("olmo_core_amd::float8_linear_bwd", mutates_args=())
def _linear_bwd(
    go: torch.Tensor, xa: torch.Tensor, xb: torch.Tensor, wa: torch.Tensor, wb: torch.Tensor, cfg: int, n: int,
    x_is_q: bool, w_is_q: bool, need_gx: bool, need_gw: bool, x_dtype: torch.dtype, w_dtype: torch.dtype,
) -> Tuple[torch.Tensor, torch.Tensor]:
    gx, gw = _backward_impl(go, _CONFIGS[cfg], n, x_dtype, w_dtype, (xa, xb), (wa, wb), x_is_q, w_is_q, need_gx, need_gw)
    return (gx if gx is not None else go.new_empty(0)), (gw if gw is not None else go.new_empty(0))


@_linear_bwd.register_fake
def _(go, xa, xb, wa, wb, cfg, n, x_is_q, w_is_q, need_gx, need_gw, x_dtype, w_dtype):
    M = go.shape[0]
    if x_is_q:
        K = xa.shape[0]
    elif need_gw:
        K = xa.shape[1]
    elif w_is_q:
        K = wa.shape[0]
    else:
        K = wa.shape[1]
    gx = go.new_empty((M, K), dtype=x_dtype) if need_gx else go.new_empty(0)
    gw = go.new_empty((n, K), dtype=w_dtype) if need_gw else go.new_empty(0)
    return gx, gw


def _setup_context(ctx, inputs, output):
    x2, weight, _, cfg, need_gx, need_gw, _ = inputs
    _, xa, xb, wa, wb = output
    x_is_q, w_is_q = _saves_quantised(_CONFIGS[cfg], need_gx, need_gw)
    ctx.meta = (cfg, weight.shape[0], x_is_q, w_is_q, need_gx, need_gw, x2.dtype, weight.dtype)
    empty = xb  # a tensor to fill unused slots with
    x_part = (xa, xb) if x_is_q else ((x2, empty) if need_gw else (empty, empty))
    w_part = (wa, wb) if w_is_q else ((weight, empty) if need_gx else (empty, empty))
    ctx.save_for_backward(*x_part, *w_part)


def _backward(ctx, gy, *unused):
    cfg, n, x_is_q, w_is_q, need_gx, need_gw, x_dtype, w_dtype = ctx.meta
    xa, xb, wa, wb = ctx.saved_tensors
    gx, gw = _linear_bwd(gy.contiguous(), xa, xb, wa, wb, cfg, n, x_is_q, w_is_q, need_gx, need_gw, x_dtype, w_dtype)
    return (gx if need_gx else None), (gw if need_gw else None), None, None, None, None, None


_linear_fwd.register_autograd(_backward, setup_context=_setup_context)


def linear(x2: torch.Tensor, weight: torch.Tensor, cfg_id: int, weight_scale: Optional[torch.Tensor], module_id: int = -1):
    """``x2 [M, K] @ weight[N, K].T`` as a traceable operator call; ``cfg_id`` indexes the registered configs,
    ``module_id`` the registered modules (-1: none)."""
    out = _linear_fwd(x2, weight, weight_scale, cfg_id, x2.requires_grad, weight.requires_grad, module_id)
    return out[0]


# ---- the fused SwiGLU feed-forward block (olmo_core_amd.nn.feed_forward) ------------------------------------------
# One operator forward, one backward: a compiled transformer block keeps the launches the eager block makes (both
# input projections and the activation in one GEMM launch, the amax of the gate gradients from row-segment codes, the
# accumulating grad_x epilogue), bit for bit.  The forward returns y and the 13 tensors the backward takes.

_N_SAVED = 13


def _ff():
    from ..nn import feed_forward

    return feed_forward


@torch.library.custom_op("olmo_core_amd::float8_swiglu_mlp_fwd", mutates_args=())
def _mlp_fwd(x: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor, cfg: int, need_x: bool, need_w1: bool,
             need_w2: bool, need_w3: bool, id1: int, id2: int, id3: int) -> List[torch.Tensor]:
    # (id1..3: the three projection modules, for their precomputed scales and kept float8 weights)
    state = [_kept_weight_state(i, w) for i, w in ((id1, w1), (id2, w2), (id3, w3))]
    y, saved = _ff()._mlp_forward(x, w1, w2, w3, _CONFIGS[cfg], (need_x, need_w1, need_w2, need_w3),
                                  tuple(s[0] for s in state), tuple(s[1] for s in state))
    return [y, *saved]


@_mlp_fwd.register_fake
def _(x, w1, w2, w3, cfg, need_x, need_w1, need_w2, need_w3, id1, id2, id3):
    c = _CONFIGS[cfg]
    ff = _ff()
    M, D = x.shape
    H = w1.shape[0]
    any_grad = need_x or need_w1 or need_w2 or need_w3
    in_dt, w_dt = c.cast_config_input.target_dtype, c.cast_config_weight.target_dtype
    pad16 = lambda n: (n + 15) // 16 * 16  # noqa: E731
    none = lambda: x.new_empty(0, dtype=torch.bfloat16)  # noqa: E731
    f32 = lambda: x.new_empty(1, dtype=torch.float32)  # noqa: E731
    q_t = lambda rows, cols, dt, wanted: x.new_empty((cols, pad16(rows)), dtype=dt) if wanted else none()  # noqa: E731
    codes = none()
    if ff._fused_launch_ok(M, D, H) and ff._use_codes(M, D, H, any_grad):
        codes = x.new_empty(((H + 63) // 64) * M, dtype=torch.int16)
    bf16 = torch.bfloat16
    return [
        x.new_empty((M, w2.shape[0]), dtype=bf16),
        q_t(M, D, in_dt, need_w1 or need_w3), f32(), x.new_empty((M, H), dtype=bf16), x.new_empty((M, H), dtype=bf16),
        q_t(M, H, in_dt, need_w2), f32(),
        q_t(H, D, w_dt, need_x), f32(), q_t(w2.shape[0], H, w_dt, any_grad), f32(), q_t(H, D, w_dt, need_x), f32(),
        codes,
    ]


@torch.library.custom_op("olmo_core_amd::float8_swiglu_mlp_bwd", mutates_args=())
def _mlp_bwd(gy: torch.Tensor, saved: List[torch.Tensor], cfg: int, m: int, d: int, h: int, need_x: bool, need_w1: bool,
             need_w2: bool, need_w3: bool, x_dtype: torch.dtype, w1_dtype: torch.dtype, w2_dtype: torch.dtype,
             w3_dtype: torch.dtype) -> List[torch.Tensor]:
    grads = _ff()._mlp_backward(gy, saved, _CONFIGS[cfg], (m, d, h), (x_dtype, w1_dtype, w2_dtype, w3_dtype),
                                (need_x, need_w1, need_w2, need_w3))
    return [g if g is not None else gy.new_empty(0) for g in grads]


@_mlp_bwd.register_fake
def _(gy, saved, cfg, m, d, h, need_x, need_w1, need_w2, need_w3, x_dtype, w1_dtype, w2_dtype, w3_dtype):
    none = lambda: gy.new_empty(0)  # noqa: E731
    return [
        gy.new_empty((m, d), dtype=x_dtype) if need_x else none(),
        gy.new_empty((h, d), dtype=w1_dtype) if need_w1 else none(),
        gy.new_empty((d, h), dtype=w2_dtype) if need_w2 else none(),
        gy.new_empty((h, d), dtype=w3_dtype) if need_w3 else none(),
    ]


def _mlp_setup_context(ctx, inputs, output):
    x, w1, w2, w3, cfg, need_x, need_w1, need_w2, need_w3 = inputs[:9]
    ctx.meta = (cfg, x.shape[0], x.shape[1], w1.shape[0], need_x, need_w1, need_w2, need_w3, x.dtype, w1.dtype, w2.dtype,
                w3.dtype)
    ctx.save_for_backward(*output[1:])


def _mlp_backward_fn(ctx, grads):
    need = ctx.meta[4:8]
    gx, gw1, gw2, gw3 = _mlp_bwd(grads[0].contiguous(), list(ctx.saved_tensors), *ctx.meta)
    pick = lambda g, wanted: g if wanted else None  # noqa: E731
    return (pick(gx, need[0]), pick(gw1, need[1]), pick(gw2, need[2]), pick(gw3, need[3])) + (None,) * 8


_mlp_fwd.register_autograd(_mlp_backward_fn, setup_context=_mlp_setup_context)


def swiglu_mlp(x2: torch.Tensor, w1: torch.Tensor, w2: torch.Tensor, w3: torch.Tensor, cfg_id: int,
               module_ids=(-1, -1, -1)) -> torch.Tensor:
    """The fused feed-forward block on ``x2 [M, D]`` as a traceable operator call; ``module_ids``: the registered ids of
    the w1, w2, w3 modules."""
    return _mlp_fwd(x2, w1, w2, w3, cfg_id, x2.requires_grad, w1.requires_grad, w2.requires_grad, w3.requires_grad,
                    module_ids[0], module_ids[1], module_ids[2])[0]


__all__ = ["linear", "swiglu_mlp", "ops"]

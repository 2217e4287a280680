"""
``Float8Linear`` and the model swap.

The module keeps the ``nn.Linear`` surface (same ``weight`` / ``bias`` Parameters, same state-dict keys) and
routes its matmuls through one ``torch.autograd.Function`` that quantises the operands with the HIP cast
kernels and multiplies them on the fp8 matrix cores.  This is the native counterpart of what the reference
obtains from ``torchao.float8.convert_to_float8_training`` (reference call site:
src/olmo_core/float8/__init__.py:133-150).

Per linear and training step (M tokens, weight [N, K]):

    output      y  [M, N] = q(x)  [M, K] . q(W)  [N, K]^T
    grad_input  gx [M, K] = q(go) [M, N] . q(W)^T [K, N]^T
    grad_weight gW [N, K] = q(go)^T [N, M] . q(x)^T [K, M]^T

Every GEMM reads both operands K-contiguous, so the casts emit row-major and/or transposed fp8 copies:
tensorwise casts emit both orientations from one pass with one scale; axiswise ("rowwise" recipes) casts
emit a per-row-scaled row-major copy for operands reduced along their rows and a per-column-scaled
transposed copy for operands reduced along their columns.
"""

from __future__ import annotations

from typing import Callable, Optional, Tuple

import torch
import torch.nn as nn

from . import ops
from .native_config import CastConfig, Float8LinearConfig, ScalingGranularity, ScalingType

__all__ = ["Float8Linear", "convert_to_float8_training", "float8_linear_function", "float8_projections"]


def _is_tensorwise(c: CastConfig) -> bool:
    return c.scaling_type is ScalingType.DYNAMIC and c.scaling_granularity is ScalingGranularity.TENSORWISE


def _is_axiswise(c: CastConfig) -> bool:
    return c.scaling_type is ScalingType.DYNAMIC and c.scaling_granularity is ScalingGranularity.AXISWISE


def _is_disabled(c: CastConfig) -> bool:
    return c.scaling_type is ScalingType.DISABLED


def _shared_tensorwise(a: CastConfig, b: CastConfig) -> bool:
    """Two uses of one tensor that quantise identically (one scale, one dtype): cast once, emit both layouts."""
    return _is_tensorwise(a) and _is_tensorwise(b) and a.target_dtype == b.target_dtype


def _shared_axiswise(a: CastConfig, b: CastConfig) -> bool:
    """Two uses of one tensor, one scaled per row and one per column, in the same fp8 type: both copies come out
    of one two-product cast."""
    return _is_axiswise(a) and _is_axiswise(b) and a.target_dtype == b.target_dtype


def _rows_operand(x: torch.Tensor, c: CastConfig, pow2: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Operand reduced along its rows' elements (K = last dim of x): row-major fp8 + scale [1] or [rows]."""
    if _is_tensorwise(c):
        q, _, s = ops.cast_tensorwise(x, c.target_dtype, pow2=pow2, want_rowmajor=True, want_transposed=False)
        return q, s
    return ops.cast_rowwise(x, c.target_dtype, pow2=pow2)


def _cols_operand(x: torch.Tensor, c: CastConfig, pow2: bool) -> Tuple[torch.Tensor, torch.Tensor]:
    """Operand whose K is x's first dim: transposed fp8 [cols, pad16(rows)] + scale [1] or [cols]."""
    if _is_tensorwise(c):
        _, q_t, s = ops.cast_tensorwise(x, c.target_dtype, pow2=pow2, want_rowmajor=False, want_transposed=True)
        return q_t, s
    return ops.cast_colwise_t(x, c.target_dtype, pow2=pow2)


def _saves_quantised(c: Float8LinearConfig, need_gx: bool, need_gw: bool) -> Tuple[bool, bool]:
    """Whether the forward keeps the transposed fp8 copy (+ scale) of x / of the weight for the backward instead
    of the high-precision tensor: possible when forward and backward quantise that tensor identically."""
    if _is_disabled(c.cast_config_input):
        return False, False
    ci, ciw = c.cast_config_input, c.cast_config_input_for_grad_weight
    cw, cwi = c.cast_config_weight, c.cast_config_weight_for_grad_input
    x_is_q = need_gw and (_shared_tensorwise(ci, ciw) or _shared_axiswise(ci, ciw))
    w_is_q = need_gx and (_shared_tensorwise(cw, cwi) or _shared_axiswise(cw, cwi))
    return x_is_q, w_is_q


def _input_operands(x2, c: Float8LinearConfig, pow2: bool, share_x: bool):
    """``(xq, sx, x_saved)`` for the forward GEMM: the by-rows operand, its scale, and what the backward keeps."""
    ci = c.cast_config_input
    x_saved = None
    if _is_tensorwise(ci):
        xq, xq_t, sx = ops.cast_tensorwise(x2, ci.target_dtype, pow2=pow2, want_rowmajor=True, want_transposed=share_x)
        if share_x:
            x_saved = (xq_t, sx)
    elif share_x:  # per-row copy for this GEMM, per-column transposed copy for grad_weight, one cast
        xq, sx, xq_t, sxc = ops.cast_rows_and_colwise_t(x2, ci.target_dtype, pow2=pow2)
        x_saved = (xq_t, sxc)
    else:
        xq, sx = ops.cast_rowwise(x2, ci.target_dtype, pow2=pow2)
    return xq, sx, x_saved


def _weight_operands(weight, c: Float8LinearConfig, pow2: bool, share_w: bool, weight_scale=None, weight_ops=None):
    """``(wq, sw, w_saved)`` for the forward GEMM: the weight's by-rows operand, its scale(s), and what the backward
    keeps for grad_input (``(q_t, scale)`` or ``None``: keep the weight itself)."""
    w_saved = None
    if weight_ops is not None:
        wq, wq_t, sw = weight_ops
        if share_w:
            w_saved = (wq_t, sw)
    elif _is_tensorwise(c.cast_config_weight):
        wq, wq_t, sw = ops.cast_tensorwise(
            weight, c.cast_config_weight.target_dtype, pow2=pow2, want_rowmajor=True, want_transposed=share_w,
            scale=weight_scale,
        )
        if share_w:
            w_saved = (wq_t, sw)
    elif share_w:
        wq, sw, wq_t, swc = ops.cast_rows_and_colwise_t(weight, c.cast_config_weight.target_dtype, pow2=pow2)
        w_saved = (wq_t, swc)
    else:
        wq, sw = ops.cast_rowwise(weight, c.cast_config_weight.target_dtype, pow2=pow2)
    return wq, sw, w_saved


def _forward_impl(x2, weight, c: Float8LinearConfig, weight_scale, need_gx: bool, need_gw: bool, weight_ops=None):
    """y = x2 @ weight^T in float8.  Returns ``(y, x_saved, w_saved)``: the tensors the backward needs for x and
    for the weight, each either ``(q_t, scale)`` (see :func:`_saves_quantised`) or ``None`` (keep the input).
    ``weight_ops``: ``(q, q_t, scale)`` of the weight kept by the module (:meth:`Float8Linear.weight_operands`);
    the weight is then not quantised here."""
    pow2 = c.round_scales_to_power_of_2
    share_x, share_w = _saves_quantised(c, need_gx, need_gw)
    if _is_disabled(c.cast_config_input):
        return torch.mm(x2, weight.t().to(x2.dtype)), None, None
    xq, sx, x_saved = _input_operands(x2, c, pow2, share_x)
    wq, sw, w_saved = _weight_operands(weight, c, pow2, share_w, weight_scale, weight_ops)
    return ops.gemm_fp8(xq, sx, wq, sw, out_dtype=x2.dtype), x_saved, w_saved


def _backward_impl(go2, c: Float8LinearConfig, N: int, x_dtype, w_dtype, x_part, w_part, x_is_q: bool, w_is_q: bool,
                   need_gx: bool, need_gw: bool, gx_into=None):
    """grad_input and grad_weight from grad_output ``go2 [M, N]``; ``x_part`` / ``w_part`` are what the forward
    kept: ``(q_t, scale)`` if the flag says so, else ``(tensor,)``.  ``gx_into``: a ``[M, K]`` tensor of ``x_dtype``
    that this linear's grad_input is added to (the bits of ``gx_into + grad_input``, formed in the GEMM's epilogue)
    and that is returned as ``gx``."""
    pow2 = c.round_scales_to_power_of_2
    if go2.dtype != x_dtype:
        go2 = go2.to(x_dtype)
    # quantise grad_output once if both backward GEMMs want the same tensorwise cast
    go_rows = go_cols = None
    cg, cgw = c.cast_config_grad_output, c.cast_config_grad_output_for_grad_weight
    if need_gx and need_gw and _shared_tensorwise(cg, cgw):
        q, q_t, s = ops.cast_tensorwise(go2, cg.target_dtype, pow2=pow2, want_rowmajor=True, want_transposed=True)
        go_rows, go_cols = (q, s), (q_t, s)
    elif need_gx and need_gw and _shared_axiswise(cg, cgw):
        q, rs, q_t, cs = ops.cast_rows_and_colwise_t(go2, cg.target_dtype, pow2=pow2)
        go_rows, go_cols = (q, rs), (q_t, cs)

    gx = gw = None
    if need_gx:
        if _is_disabled(cg):
            gx = torch.mm(go2, w_part[0].to(go2.dtype))
            if gx_into is not None:
                gx = gx_into.add_(gx)
        else:
            if go_rows is None:
                go_rows = _rows_operand(go2, cg, pow2)
            w_op = (w_part[0], w_part[1]) if w_is_q else _cols_operand(w_part[0], c.cast_config_weight_for_grad_input, pow2)
            gx = ops.gemm_fp8(go_rows[0], go_rows[1], w_op[0], w_op[1], k=N, out_dtype=x_dtype, out=gx_into,
                              accumulate=gx_into is not None)
    if need_gw:
        if _is_disabled(cgw):
            gw = torch.mm(go2.t(), x_part[0].to(go2.dtype))
        else:
            if go_cols is None:
                go_cols = _cols_operand(go2, cgw, pow2)
            x_op = (x_part[0], x_part[1]) if x_is_q else _cols_operand(x_part[0], c.cast_config_input_for_grad_weight, pow2)
            gw = ops.gemm_fp8(go_cols[0], go_cols[1], x_op[0], x_op[1], out_dtype=x_dtype)
        if gw.dtype != w_dtype:
            gw = gw.to(w_dtype)
    return gx, gw


class _Float8Matmul(torch.autograd.Function):
    """y = x @ W^T with float8 operands; x [M, K] and W [N, K] in high precision."""

    @staticmethod
    def forward(ctx, x2: torch.Tensor, weight: torch.Tensor, config: Float8LinearConfig, weight_scale=None,
                weight_ops=None):
        need_gx, need_gw = ctx.needs_input_grad[0], ctx.needs_input_grad[1]
        y, x_saved, w_saved = _forward_impl(x2, weight, config, weight_scale, need_gx, need_gw, weight_ops)
        ctx.config = config
        ctx.x_dtype, ctx.w_dtype = x2.dtype, weight.dtype
        ctx.shapes = (x2.shape[0], x2.shape[1], weight.shape[0])
        ctx.x_is_q, ctx.w_is_q = x_saved is not None, w_saved is not None
        to_save = []
        if need_gw:
            to_save += list(x_saved) if ctx.x_is_q else [x2]
        if need_gx:
            to_save += list(w_saved) if ctx.w_is_q else [weight]
        ctx.n_x = (2 if ctx.x_is_q else 1) if need_gw else 0
        ctx.save_for_backward(*to_save)
        return y

    @staticmethod
    def backward(ctx, go: torch.Tensor):
        M, K, N = ctx.shapes
        saved = ctx.saved_tensors
        gx, gw = _backward_impl(
            go.reshape(M, N), ctx.config, N, ctx.x_dtype, ctx.w_dtype, saved[: ctx.n_x], saved[ctx.n_x :],
            ctx.x_is_q, ctx.w_is_q, ctx.needs_input_grad[0], ctx.needs_input_grad[1],
        )
        return gx, gw, None, None, None


def _shared_input_forward(x2, weights, c: Float8LinearConfig, scales, w_ops, need_gx: bool, need_gw: bool):
    """``ys[i] = x2 @ weights[i]^T`` with x2 quantised once.  Returns ``(ys, x_saved, w_saved)``, ``x_saved`` and each
    ``w_saved[i]`` as :func:`_forward_impl` returns them."""
    if _is_disabled(c.cast_config_input):
        return [torch.mm(x2, w.t().to(x2.dtype)) for w in weights], None, [None] * len(weights)
    pow2 = c.round_scales_to_power_of_2
    share_x, share_w = _saves_quantised(c, need_gx, need_gw)
    xq, sx, x_saved = _input_operands(x2, c, pow2, share_x)
    ys, w_saved = [], []
    for w, ws, wo in zip(weights, scales, w_ops):
        wq, sw, kept = _weight_operands(w, c, pow2, share_w, ws, wo)
        ys.append(ops.gemm_fp8(xq, sx, wq, sw, out_dtype=x2.dtype))
        w_saved.append(kept)
    return ys, x_saved, w_saved


class _Float8SharedInputMatmul(torch.autograd.Function):
    """``ys[i] = x @ W_i^T`` for several weights applied to ONE input (the q, k and v projections of an attention
    block, reference src/olmo_core/nn/attention/__init__.py:582): x is quantised once by construction, one copy of
    it is kept for all the weight gradients, and the grad_input terms are summed by the GEMM epilogues
    (``C += product``) in the order autograd adds them - the last projection's first - so outputs and gradients carry
    the bits of the modules applied one by one."""

    @staticmethod
    def forward(ctx, x2, config, n, act_dtype, *rest):
        # act_dtype: the type the modules see their input in (the autocast type when autocast is on, else x2's own).
        # Each module would convert x2 itself and autograd would add the converted-back grad_input terms in x2's type:
        # that sum is formed here when the types differ.
        weights, scales, w_ops = rest[:n], rest[n:2 * n], rest[2 * n:3 * n]
        need_gx = ctx.needs_input_grad[0]
        need_gws = [ctx.needs_input_grad[4 + i] for i in range(n)]
        ctx.set_materialize_grads(False)
        ctx.gx_dtype = x2.dtype
        if x2.dtype != act_dtype:
            x2 = x2.to(act_dtype)
        ys, x_saved, w_saved = _shared_input_forward(x2, weights, config, scales, w_ops, need_gx, any(need_gws))
        ctx.config = config
        ctx.x_dtype, ctx.w_dtypes = x2.dtype, [w.dtype for w in weights]
        ctx.M, ctx.ns = x2.shape[0], [w.shape[0] for w in weights]
        ctx.x_is_q, ctx.w_is_q = x_saved is not None, [k is not None for k in w_saved]
        ctx.need_gws = need_gws
        to_save = []
        if any(need_gws):
            to_save += list(x_saved) if ctx.x_is_q else [x2]
        ctx.n_x = len(to_save)
        if need_gx:
            for w, kept in zip(weights, w_saved):
                to_save += list(kept) if kept is not None else [w]
        ctx.save_for_backward(*to_save)
        return tuple(ys)

    @staticmethod
    def backward(ctx, *gos):
        n = len(ctx.ns)
        saved = ctx.saved_tensors
        need_gx = ctx.needs_input_grad[0]
        x_part, pos = saved[:ctx.n_x], ctx.n_x
        w_parts = []
        for i in range(n):
            k = (2 if ctx.w_is_q[i] else 1) if need_gx else 0
            w_parts.append(saved[pos:pos + k])
            pos += k
        gx, gws = None, [None] * n
        chain = ctx.gx_dtype == ctx.x_dtype  # the terms are added in the type the GEMMs write: by their epilogues
        for i in reversed(range(n)):
            if gos[i] is None:
                continue
            term, gws[i] = _backward_impl(
                gos[i].reshape(ctx.M, ctx.ns[i]), ctx.config, ctx.ns[i], ctx.x_dtype, ctx.w_dtypes[i], x_part, w_parts[i],
                ctx.x_is_q, ctx.w_is_q[i], need_gx, ctx.need_gws[i], gx_into=gx if chain else None,
            )
            if need_gx:
                gx = term if chain else (term.to(ctx.gx_dtype) if gx is None else gx.add_(term))
        return (gx, None, None, None, *gws, *([None] * (2 * n)))


@torch.compiler.disable
def _eager_shared_input_matmul(x2, config, act_dtype, weights, scales, w_ops):
    return _Float8SharedInputMatmul.apply(x2, config, len(weights), act_dtype, *weights, *scales, *w_ops)


def float8_projections(x: torch.Tensor, *modules: nn.Module) -> Tuple[torch.Tensor, ...]:
    """``tuple(m(x) for m in modules)`` for linear modules applied to one tensor, e.g. ``q, k, v =
    float8_projections(x, self.w_q, self.w_k, self.w_v)`` in place of the three calls at
    src/olmo_core/nn/attention/__init__.py:582.  When every module is a :class:`Float8Linear` of one config the
    input is quantised once for all of them and its gradient leaves the last grad_input GEMM already summed; outputs
    and gradients have the bits of the separate calls.  Anything else (plain ``nn.Linear``, mixed configs, a traced
    graph) is applied module by module."""
    mods = modules
    fusable = (
        len(mods) > 1 and all(isinstance(m, Float8Linear) for m in mods) and x.is_cuda
        and all(m.config is mods[0].config or m.config == mods[0].config for m in mods)
        and all(m.in_features == x.shape[-1] for m in mods) and not torch.compiler.is_compiling()
    )
    if not fusable:
        return tuple(m(x) for m in mods)
    act_dtype = torch.get_autocast_dtype(x.device.type) if torch.is_autocast_enabled() else x.dtype
    c = mods[0].config
    x2 = x.reshape(-1, x.shape[-1])
    weights = [m.weight for m in mods]
    scales = [m.precomputed_weight_scale() for m in mods]
    w_ops = [m.weight_operands() for m in mods]
    if torch.is_grad_enabled() and (x2.requires_grad or any(w.requires_grad for w in weights)):
        ys = _eager_shared_input_matmul(x2, c, act_dtype, weights, scales, w_ops)
    else:
        ys = _shared_input_forward(x2.to(act_dtype), weights, c, scales, w_ops, False, False)[0]
    outs = []
    for m, y in zip(mods, ys):
        y = y.reshape(*x.shape[:-1], m.weight.shape[0])
        outs.append(y if m.bias is None else y + m.bias.to(y.dtype))
    return tuple(outs)


# Operator arguments must be plain values: under torch.compile a config travels as its index in this list.  Configs
# are registered when a module is built (tracing must not mutate the list).
_COMPILED_CONFIGS: list = []

# Likewise the modules (as weak references): a compiled call names its module by index, and the operator, which runs
# eagerly, asks that module for its precomputed weight scale and kept float8 weight copies - lookups by address and
# version counter that a traced graph cannot contain.
_COMPILED_MODULES: list = []


def _register_module(m) -> int:
    import weakref

    _COMPILED_MODULES.append(weakref.ref(m))
    return len(_COMPILED_MODULES) - 1


def _kept_weight_state(module_id: int, weight: torch.Tensor):
    """``(precomputed scale, kept operands)`` of the registered module if ``weight`` is that module's weight."""
    if module_id < 0 or module_id >= len(_COMPILED_MODULES):
        return None, None
    m = _COMPILED_MODULES[module_id]()
    if m is None or m.weight.data_ptr() != weight.data_ptr() or m.weight.shape != weight.shape:
        return None, None
    return m.precomputed_weight_scale(), m.weight_operands()


def _register_config(c: Float8LinearConfig) -> int:
    idx = getattr(c, "_compiled_id", None)
    if idx is None:
        _COMPILED_CONFIGS.append(c)
        idx = len(_COMPILED_CONFIGS) - 1
        c._compiled_id = idx
    return idx


@torch.compiler.disable
def _eager_matmul(x2, weight, config, weight_scale, weight_ops=None):
    return _Float8Matmul.apply(x2, weight, config, weight_scale, weight_ops)


def float8_linear_function(
    x: torch.Tensor, weight: torch.Tensor, config: Float8LinearConfig, weight_scale: Optional[torch.Tensor] = None,
    weight_ops: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None, module_id: int = -1,
) -> torch.Tensor:
    """``x [*, K] @ weight[N, K].T`` through the float8 path, differentiable in x and weight.

    ``weight_scale``: a precomputed tensorwise scale of ``weight`` (float32 ``[1]``), used instead of reducing the
    weight's amax again; ignored unless the weight cast is tensorwise.
    ``weight_ops``: float8 copies of ``weight`` made earlier (``(q [N, K], q_t [K, pad16(N)], scale [1])``, as
    :meth:`Float8Linear.weight_operands` returns them), used instead of quantising ``weight`` again; eager only.

    Under ``torch.compile`` the call becomes a pair of registered custom operators (forward, backward) with shape
    functions, so a compiled block keeps one graph; eagerly it is an ordinary ``autograd.Function``.
    """
    K = x.shape[-1]
    if weight.dim() != 2 or weight.shape[1] != K:
        raise ValueError(f"float8 linear: input features {K} do not match weight {tuple(weight.shape)}")
    x2 = x.reshape(-1, K)
    cfg_id = getattr(config, "_compiled_id", -1)
    compiling = torch.compiler.is_compiling()
    if compiling and cfg_id >= 0:
        from . import compiled

        y = compiled.linear(x2, weight, cfg_id, weight_scale, module_id)
    elif not compiling and not (torch.is_grad_enabled() and (x2.requires_grad or weight.requires_grad)):
        # nothing to differentiate (evaluation, generation): no autograd node, nothing kept for a backward
        y = _forward_impl(x2, weight, config, weight_scale, False, False, weight_ops)[0]
    else:  # eager, or a config no module registered: a graph break
        y = _eager_matmul(x2, weight, config, weight_scale, weight_ops)
    return y.reshape(*x.shape[:-1], weight.shape[0])


class Float8Linear(nn.Linear):
    """
    Drop-in ``nn.Linear`` whose forward / backward matmuls run in float8 with dynamic scaling.
    Use :meth:`from_float` (or :func:`convert_to_float8_training`) to create it from an existing module.
    """

    def __init__(self, *args, config: Optional[Float8LinearConfig] = None, **kwargs):
        super().__init__(*args, **kwargs)
        self.config = config if config is not None else Float8LinearConfig()
        self._bind_config()

    def _bind_config(self) -> None:
        c = self.config
        _register_config(c)
        self._module_id = _register_module(self)
        self.scaling_type_input = c.cast_config_input.scaling_type
        self.scaling_type_weight = c.cast_config_weight.scaling_type
        self.scaling_type_grad_output = c.cast_config_grad_output.scaling_type

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        if torch.is_autocast_enabled():
            input = input.to(torch.get_autocast_dtype(input.device.type))
        # (the stored scale is checked against the weight's address and version counter: not traceable)
        compiling = torch.compiler.is_compiling()
        scale = None if compiling else self.precomputed_weight_scale()
        w_ops = None if compiling else self.weight_operands()
        out = float8_linear_function(input, self.weight, self.config, scale, w_ops, self._module_id)
        if self.bias is not None:
            out = out + self.bias.to(out.dtype)
        return out

    def precomputed_weight_scale(self) -> Optional[torch.Tensor]:
        """The scale stored by :func:`precompute_float8_dynamic_scale_for_fsdp` if the weight has not been
        modified (or replaced) since; ``None`` otherwise, and the forward then reduces the amax itself."""
        entry = getattr(self, "_precomputed_weight_scale", None)
        if entry is None:
            return None
        scale, ptr, version = entry
        w = self.weight
        if w.is_inference():  # (inference tensors have no version counter)
            return None
        if w.data_ptr() != ptr or w._version != version or not _is_tensorwise(self.config.cast_config_weight):
            return None
        return scale

    def weight_operands(self) -> Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]]:
        """Float8 copies of the weight that outlive one call: ``(q [N, K], q_t [K, pad16(N)], scale [1])``, made
        on first use and kept until the weight is modified or replaced (address and version counter), so that
        the micro-batches of one optimizer step, or the steps of a generation loop, quantise each weight once.

        Only with ``config.enable_fsdp_float8_all_gather``: upstream that switch makes FSDP hold and communicate
        the float8 weight (computed from the precomputed scale, ``src/olmo_core/float8/__init__.py:54-62``,
        ``src/olmo_core/float8/ao.py:173-180``); on one device what remains of it is that the float8 weight is
        materialised once per weight update rather than once per forward.  Costs two bytes per parameter.
        ``None`` when the switch is off, the weight is not a contiguous GPU tensor, or forward and grad_input
        quantise the weight differently.  Bytes and scale equal those a forward would make itself.  (A write
        through ``weight.data`` moves no version counter and goes unnoticed, as for the precomputed scales;
        :func:`precompute_float8_dynamic_scale_for_fsdp` drops the copies.)"""
        c = self.config
        if not c.enable_fsdp_float8_all_gather:
            return None
        w = self.weight
        if not _shared_tensorwise(c.cast_config_weight, c.cast_config_weight_for_grad_input):
            return None
        if not w.is_cuda or not w.is_contiguous() or w.dtype not in (torch.bfloat16, torch.float32) or w.is_inference():
            return None
        key = (w.data_ptr(), w._version, w.dtype, tuple(w.shape))
        entry = getattr(self, "_weight_operands", None)
        if entry is not None and entry[0] == key:
            return entry[1]
        with torch.no_grad():
            made = ops.cast_tensorwise(
                w.detach(), c.cast_config_weight.target_dtype, pow2=c.round_scales_to_power_of_2,
                want_rowmajor=True, want_transposed=True, scale=self.precomputed_weight_scale(),
            )
        self._weight_operands = (key, made)
        return made

    def extra_repr(self) -> str:
        c = self.config
        parts = [
            f"i:{c.cast_config_input.short_str()}",
            f"w:{c.cast_config_weight.short_str()}",
            f"go:{c.cast_config_grad_output.short_str()}",
        ]
        if c.cast_config_input_for_grad_weight != c.cast_config_input:
            parts.append(f"i_gw:{c.cast_config_input_for_grad_weight.short_str()}")
        if c.cast_config_weight_for_grad_input != c.cast_config_weight:
            parts.append(f"w_gi:{c.cast_config_weight_for_grad_input.short_str()}")
        if c.cast_config_grad_output_for_grad_weight != c.cast_config_grad_output:
            parts.append(f"go_gw:{c.cast_config_grad_output_for_grad_weight.short_str()}")
        return f'{super().extra_repr()}, cast_configs={",".join(parts)}'

    @classmethod
    def from_float(cls, mod: nn.Linear, config: Optional[Float8LinearConfig] = None) -> "Float8Linear":
        """New module sharing ``mod``'s Parameters; reads no weight values (works on the meta device)."""
        config = config if config is not None else Float8LinearConfig()
        if config.emulate:
            raise NotImplementedError(
                "emulate=True selects a CPU-emulated matmul upstream; this library only has the native gfx950 path"
            )
        config.check_gemm_operands()
        with torch.device("meta"):
            new = cls(mod.in_features, mod.out_features, bias=False, config=config)
        new.weight = mod.weight
        new.bias = mod.bias
        return new


def _swap(
    module: nn.Module,
    make: Callable[[nn.Linear], nn.Module],
    module_filter_fn: Optional[Callable[[nn.Module, str], bool]],
) -> nn.Module:
    """Post-order walk replacing every ``nn.Linear`` the filter accepts; the filter sees only Linears."""
    if isinstance(module, nn.Linear) and (module_filter_fn is None or module_filter_fn(module, "")):
        if len(list(module.children())) > 0:
            raise AssertionError(f"Does not support a root nn.Linear with children: {module}")
        return make(module)

    visited = set()

    def walk(m: nn.Module, fqn: str, parent: Optional[nn.Module], name: Optional[str]) -> None:
        if id(m) in visited:
            return
        visited.add(id(m))
        for child_name, child in list(m.named_children()):
            walk(child, f"{fqn}.{child_name}" if fqn else child_name, m, child_name)
        if parent is not None and isinstance(m, nn.Linear) and not isinstance(m, Float8Linear):
            if module_filter_fn is None or module_filter_fn(m, fqn):
                setattr(parent, name, make(m))

    walk(module, "", None, None)
    return module


def convert_to_float8_training(
    module: nn.Module,
    *,
    module_filter_fn: Optional[Callable[[nn.Module, str], bool]] = None,
    config: Optional[Float8LinearConfig] = None,
) -> nn.Module:
    """
    Swap ``nn.Linear`` modules for :class:`Float8Linear` in place and return the (possibly new) root.
    ``module_filter_fn(mod, fqn)`` is consulted for Linear modules only; returning False keeps the module.
    """
    config = config if config is not None else Float8LinearConfig()
    return _swap(module, lambda m: Float8Linear.from_float(m, config), module_filter_fn)


def precompute_float8_dynamic_scale_for_fsdp(module: nn.Module) -> None:
    """
    Refresh the tensorwise weight scales of every :class:`Float8Linear` under ``module`` in one batch of kernel
    launches; call it right after the optimizer step (reference: torchao's function of the same name, called
    from ``src/olmo_core/nn/transformer/model.py:1001-1008``).  Forwards then skip the weight's amax pass until
    the weight changes again; the scales are the ones the forward would compute itself, bit for bit.
    """
    groups: dict = {}
    for m in module.modules():
        if not isinstance(m, Float8Linear):
            continue
        m._precomputed_weight_scale = None
        m._weight_operands = None
        c = m.config
        w = m.weight
        if not _is_tensorwise(c.cast_config_weight) or not w.is_cuda or not w.is_contiguous():
            continue
        if w.dtype not in (torch.bfloat16, torch.float32) or w.data_ptr() % 16:
            continue
        key = (w.device, w.dtype, c.cast_config_weight.target_dtype, c.round_scales_to_power_of_2)
        groups.setdefault(key, []).append(m)
    for (_, _, fp8_dtype, pow2), mods in groups.items():
        for start in range(0, len(mods), 65535):
            chunk = mods[start:start + 65535]
            with torch.no_grad():
                scales = ops.multi_tensor_scales([m.weight.detach() for m in chunk], fp8_dtype, pow2=pow2)
            for i, m in enumerate(chunk):
                m._precomputed_weight_scale = (scales[i:i + 1], m.weight.data_ptr(), m.weight._version)

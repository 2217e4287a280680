"""
CPU oracle for the float8 linear path.  TEST INFRASTRUCTURE ONLY.

This module restates, with plain torch-CPU ops, the arithmetic that the reference reaches through
``olmo_core.float8`` (reference: src/olmo_core/float8/__init__.py:133-150 hands the model to
``torchao.float8.convert_to_float8_training``; torchao==0.15.0 is pinned at pyproject.toml:67 and is
not vendored in the reference tree).  The restated algorithm is torchao's published dynamic-scaling
float8 training path with ``emulate=True``:

    amax  -> scale = float32(FP8_MAX / clamp(float64(amax), 1e-12)) [-> round down to a power of 2]
          -> bytes = RNE_fp8(clamp(float32(x) * scale, -FP8_MAX, FP8_MAX))
          -> out   = (float32(a8)/sa) @ (float32(b8)/sb) -> bf16

Only tests, ``__graft_entry__.smoke()`` and ``bench.py``'s ``cpu_baseline`` leg may import this file;
it is the checker and never the product.  The product (``olmo_core_amd``) has no CPU path.

How each function is pinned (a check that a plausible mistake would fail), see tests/test_oracle.py:
  * ``fp8 cast``      - torch-CPU ``.to(float8_*)`` (library routine) against the independent
                        bit-level C restatement in oracle/fp8_cast_ref.c, exhaustively over all
                        65536 bf16 patterns x several scales x {e4m3, e5m2}; plus known RNE ties.
  * ``scale``         - closed form; f64 route against exact rational arithmetic (fractions.Fraction)
                        over every positive finite bf16 amax.
  * ``pow2 rounding`` - against ``math.frexp`` on every bf16-derived scale.
  * ``amax``          - brute force python loop on small inputs; NaN propagation.
  * ``emulated mm``   - tensorwise case against torch-CPU ``torch._scaled_mm`` (library routine)
                        and against float64 matmul of the dequantised operands.
  * ``autograd``      - gradients against bf16 ``F.linear`` autograd (cosine) and the identity
                        grad_W = go^T x / grad_x = go W on exactly-representable inputs.
  * ``swap/filter``   - known answers re-derived from src/olmo_core/float8/__init__.py:86-98,152-162.
  * ``grouped``       - per-expert loop (src/olmo_core/nn/moe/mlp.py:264-270) with the dense oracle
                        per slice, incl. empty groups.
  * ``mlp_fwd_bwd``   - all five results against float32 autograd of w2(silu(w1 x) * w3 x) with w1, w3
                        of different magnitude (cosine and norm ratio per tensor), and stage by stage,
                        bit for bit, against the single-linear oracle plus the closed-form SwiGLU gradient.
  * ``dropless_mlp_fwd_bwd`` - per expert against the float32 loop of mlp.py:264-292 (experts of
                        different magnitude, an empty and a one-row expert), and exactly on
                        small-integer inputs where the whole expert MLP is representable.
Parity unpinned (no reference-held vector exists; only an import of torchao could confirm): the
float64 upcast inside ``amax_to_scale``, the recipe defaults of ``from_recipe_name`` ("rowwise":
e4m3 for grad_output, power-of-2 scales) and e5m2 as the default grad_output dtype.  Each of them is
a configuration knob here.
"""

from __future__ import annotations

from dataclasses import dataclass, field, replace
from typing import Dict, List, Optional, Sequence, Tuple

import torch

EPS = 1e-12

E4M3 = torch.float8_e4m3fn
E5M2 = torch.float8_e5m2

FP8_MAX = {E4M3: 448.0, E5M2: 57344.0}

TENSORWISE = "tensorwise"
AXISWISE = "axiswise"
DYNAMIC = "dynamic"
DISABLED = "disabled"


# --------------------------------------------------------------------------------------------
# config restatement (torchao Float8LinearConfig defaults and recipes)
# --------------------------------------------------------------------------------------------


@dataclass
class CastSpec:
    """One torchao ``CastConfig``: how one operand of one GEMM is quantised."""

    scaling_type: str = DYNAMIC
    granularity: str = TENSORWISE
    dtype: Optional[torch.dtype] = None  # resolved in LinearSpec.__post_init__


@dataclass
class LinearSpec:
    """
    The resolved torchao ``Float8LinearConfig`` (what src/olmo_core/float8/ao.py:152-186 mirrors).
    Defaults: everything dynamic+tensorwise; input/weight e4m3, grad_output e5m2; no pow2 rounding.
    """

    input: CastSpec = field(default_factory=CastSpec)
    weight: CastSpec = field(default_factory=CastSpec)
    grad_output: CastSpec = field(default_factory=CastSpec)
    input_for_grad_weight: Optional[CastSpec] = None
    weight_for_grad_input: Optional[CastSpec] = None
    grad_output_for_grad_weight: Optional[CastSpec] = None
    round_scales_to_power_of_2: bool = False

    def __post_init__(self):
        if self.input_for_grad_weight is None:
            self.input_for_grad_weight = replace(self.input)
        if self.weight_for_grad_input is None:
            self.weight_for_grad_input = replace(self.weight)
        if self.grad_output_for_grad_weight is None:
            self.grad_output_for_grad_weight = replace(self.grad_output)
        for c in (self.input, self.weight, self.input_for_grad_weight, self.weight_for_grad_input):
            if c.dtype is None:
                c.dtype = E4M3
        for c in (self.grad_output, self.grad_output_for_grad_weight):
            if c.dtype is None:
                c.dtype = E5M2

    @property
    def any_axiswise(self) -> bool:
        return any(
            c.granularity == AXISWISE
            for c in (
                self.input,
                self.weight,
                self.grad_output,
                self.input_for_grad_weight,
                self.weight_for_grad_input,
                self.grad_output_for_grad_weight,
            )
        )


def recipe(name: str) -> LinearSpec:
    """torchao ``Float8LinearConfig.from_recipe_name`` for the names at float8/ao.py:100-103."""
    if name == "tensorwise":
        return LinearSpec()
    if name == "rowwise":
        ax = lambda: CastSpec(DYNAMIC, AXISWISE, E4M3)  # noqa: E731
        return LinearSpec(input=ax(), weight=ax(), grad_output=ax(), round_scales_to_power_of_2=True)
    if name == "rowwise_with_gw_hp":
        ax = lambda: CastSpec(DYNAMIC, AXISWISE, E4M3)  # noqa: E731
        return LinearSpec(
            input=ax(),
            weight=ax(),
            grad_output=ax(),
            weight_for_grad_input=CastSpec(DYNAMIC, TENSORWISE, E4M3),
            input_for_grad_weight=CastSpec(DISABLED, TENSORWISE, E4M3),
            grad_output_for_grad_weight=CastSpec(DISABLED, TENSORWISE, E4M3),
            round_scales_to_power_of_2=True,
        )
    raise ValueError(name)


# --------------------------------------------------------------------------------------------
# amax / scale / cast
# --------------------------------------------------------------------------------------------


def tensor_to_amax(x: torch.Tensor, granularity: str = TENSORWISE, axis: Optional[int] = None):
    """max(|x|) in x's own dtype; axiswise keeps the reduced dim (torchao ``tensor_to_amax``)."""
    if granularity == TENSORWISE:
        return torch.max(torch.abs(x))
    assert axis is not None
    return torch.amax(torch.abs(x), dim=axis, keepdim=True)


def amax_to_scale(amax: torch.Tensor, fp8_dtype: torch.dtype, pow2: bool = False) -> torch.Tensor:
    """
    scale = float32(FP8_MAX / clamp(float64(amax), EPS)); ``scalar / tensor`` is evaluated by torch
    as ``tensor.reciprocal() * scalar`` in float64.  Optional round-down to a power of two is
    ``exp2(floor(log2(scale)))`` in float32 (torchao ``amax_to_scale``).
    """
    a64 = amax.to(torch.float64)
    res = FP8_MAX[fp8_dtype] / torch.clamp(a64, min=EPS)
    res = res.to(torch.float32)
    if pow2:
        res = torch.exp2(torch.floor(torch.log2(res)))
    return res


def to_fp8_saturated(y: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    """clamp to the finite fp8 range (NaN stays NaN) then round-to-nearest-even convert."""
    m = FP8_MAX[fp8_dtype]
    return y.clamp(min=-m, max=m).to(fp8_dtype)


def cast_with_scale(x: torch.Tensor, scale: torch.Tensor, fp8_dtype: torch.dtype) -> torch.Tensor:
    """bytes = fp8(clamp(float32(x) * scale)) (torchao ``hp_tensor_and_scale_to_float8``)."""
    return to_fp8_saturated(x.to(torch.float32) * scale, fp8_dtype)


def cast(
    x: torch.Tensor,
    fp8_dtype: torch.dtype,
    granularity: str = TENSORWISE,
    axis: Optional[int] = None,
    pow2: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Dynamic cast: returns (fp8 tensor of x's shape, float32 scale - 0-d or keepdim vector)."""
    amax = tensor_to_amax(x, granularity, axis)
    scale = amax_to_scale(amax, fp8_dtype, pow2)
    return cast_with_scale(x, scale, fp8_dtype), scale


# --------------------------------------------------------------------------------------------
# matmul
# --------------------------------------------------------------------------------------------


def emulated_mm(
    a8: torch.Tensor,
    sa: torch.Tensor,
    b8: torch.Tensor,
    sb: torch.Tensor,
    out_dtype: torch.dtype = torch.bfloat16,
) -> torch.Tensor:
    """torchao's ``emulate=True`` matmul: mm(a.float()/sa, b.float()/sb).to(out_dtype).
    a8 [M,K] with sa 0-d or [M,1]; b8 [K,N] with sb 0-d or [1,N]."""
    return torch.mm(a8.to(torch.float32) / sa, b8.to(torch.float32) / sb).to(out_dtype)


def emulated_mm_f32(a8, sa, b8, sb) -> torch.Tensor:
    """Same contraction kept in float32 (the fp32-accumulated emulation the tolerance is quoted on)."""
    return torch.mm(a8.to(torch.float32) / sa, b8.to(torch.float32) / sb)


# --------------------------------------------------------------------------------------------
# the autograd function, restated as explicit forward / backward (torchao
# ``matmul_with_hp_or_float8_args``) + the module forward (``Float8Linear.forward``)
# --------------------------------------------------------------------------------------------


@dataclass
class LinearTrace:
    """Everything the path produces for one linear, so a test can compare operand by operand."""

    out: Optional[torch.Tensor] = None
    grad_input: Optional[torch.Tensor] = None
    grad_weight: Optional[torch.Tensor] = None
    grad_bias: Optional[torch.Tensor] = None
    operands: Dict[str, Tuple[torch.Tensor, torch.Tensor]] = field(default_factory=dict)


def _maybe_cast(x, spec: CastSpec, axis: int, pow2: bool):
    if spec.scaling_type == DISABLED:
        return None
    if spec.granularity == TENSORWISE:
        return cast(x, spec.dtype, TENSORWISE, None, pow2)
    return cast(x, spec.dtype, AXISWISE, axis, pow2)


def linear_forward(
    x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], spec: LinearSpec
) -> LinearTrace:
    """
    Float8Linear.forward: x [*, K], weight [N, K].  If no cast is axiswise the weight is cast once
    (tensorwise) outside the autograd function and reused by dgrad; otherwise the high-precision
    weight is handed in and cast per GEMM.
    """
    tr = LinearTrace()
    pow2 = spec.round_scales_to_power_of_2
    x2 = x.reshape(-1, x.shape[-1])
    wt = weight.t()  # [K, N]

    xq = _maybe_cast(x2, spec.input, -1, pow2)
    if not spec.any_axiswise:
        wq = _maybe_cast(wt, spec.weight, 0, pow2)
    else:
        wq = _maybe_cast(wt, spec.weight, 0, pow2)
    if xq is None or wq is None:
        assert xq is None and wq is None, "operands of one GEMM must both be fp8 or both hp"
        out = torch.mm(x2, wt.to(x2.dtype))
    else:
        tr.operands["input"] = xq
        tr.operands["weight"] = wq
        out = emulated_mm(xq[0], xq[1], wq[0], wq[1], x.dtype)
    out = out.reshape(*x.shape[:-1], weight.shape[0])
    if bias is not None:
        out = out + bias.to(out.dtype)
    tr.out = out
    return tr


def linear_backward(
    x: torch.Tensor,
    weight: torch.Tensor,
    grad_out: torch.Tensor,
    spec: LinearSpec,
    tr: Optional[LinearTrace] = None,
    has_bias: bool = False,
) -> LinearTrace:
    """dgrad: go[M,N] @ W[N,K]; wgrad: go^T[N,M] @ x[M,K] with the casts of torchao's backward."""
    tr = tr if tr is not None else LinearTrace()
    pow2 = spec.round_scales_to_power_of_2
    x2 = x.reshape(-1, x.shape[-1])
    go2 = grad_out.reshape(-1, grad_out.shape[-1])
    wt = weight.t()  # [K, N]

    # grad_input = go @ W  (right operand is Wt.t() = W [N, K]; its axiswise scale is per row of Wt,
    # i.e. per input channel, shape [K,1] on Wt = [1,K] on W)
    goq = _maybe_cast(go2, spec.grad_output, -1, pow2)
    if not spec.any_axiswise:
        wq = _maybe_cast(wt, spec.weight, 0, pow2)  # the pre-cast tensorwise weight is reused
    else:
        wq = _maybe_cast(wt, spec.weight_for_grad_input, -1, pow2)
    if goq is None or wq is None:
        assert goq is None and wq is None
        gx = torch.mm(go2, weight.to(go2.dtype))
    else:
        tr.operands["grad_output"] = goq
        tr.operands["weight_for_grad_input"] = wq
        gx = emulated_mm(goq[0], goq[1], wq[0].t(), wq[1].t() if wq[1].dim() else wq[1], go2.dtype)
    tr.grad_input = gx.reshape(x.shape)

    # grad_weight = go^T @ x : left operand go^T [N,M] scaled per row (= per column of go),
    # right operand x [M,K] scaled per column.
    goq2 = _maybe_cast(go2, spec.grad_output_for_grad_weight, 0, pow2)
    xq2 = _maybe_cast(x2, spec.input_for_grad_weight, 0, pow2)
    if goq2 is None or xq2 is None:
        assert goq2 is None and xq2 is None
        gw = torch.mm(go2.t(), x2.to(go2.dtype))
    else:
        tr.operands["grad_output_for_grad_weight"] = goq2
        tr.operands["input_for_grad_weight"] = xq2
        sa = goq2[1].t() if goq2[1].dim() else goq2[1]
        gw = emulated_mm(goq2[0].t(), sa, xq2[0], xq2[1], go2.dtype)
    tr.grad_weight = gw.to(weight.dtype)
    if has_bias:
        tr.grad_bias = go2.sum(0)
    return tr


def linear_fwd_bwd(x, weight, bias, grad_out, spec: LinearSpec) -> LinearTrace:
    tr = linear_forward(x, weight, bias, spec)
    return linear_backward(x, weight, grad_out, spec, tr, has_bias=bias is not None)


# --------------------------------------------------------------------------------------------
# SwiGLU MLP composition (src/olmo_core/nn/feed_forward.py:161-171)
# --------------------------------------------------------------------------------------------


@dataclass
class MLPTrace:
    y: torch.Tensor
    h: torch.Tensor
    grad_x: Optional[torch.Tensor] = None
    grad_w1: Optional[torch.Tensor] = None
    grad_w2: Optional[torch.Tensor] = None
    grad_w3: Optional[torch.Tensor] = None
    linears: Dict[str, LinearTrace] = field(default_factory=dict)


def swiglu(x1: torch.Tensor, x3: torch.Tensor) -> torch.Tensor:
    """silu(x1) * x3 as torch evaluates it on bf16 tensors (each op rounds to bf16)."""
    return torch.nn.functional.silu(x1) * x3


def swiglu_backward(x1, x3, gh):
    """Gradients of h = silu(x1) * x3 w.r.t. x1 and x3, evaluated by torch autograd on CPU."""
    x1 = x1.detach().requires_grad_(True)
    x3 = x3.detach().requires_grad_(True)
    h = swiglu(x1, x3)
    h.backward(gh)
    return x1.grad, x3.grad


# ---- magnitude codes: the bound behind the sparse amax of the SwiGLU gradients --------------------------------
# (no counterpart in the reference, which takes the amax with a pass over the gradients, torchao tensor_to_amax;
# the product finds the same amax from these codes and is tested against this restatement and against that pass)

SWIGLU_MARGIN_G3, SWIGLU_MARGIN_G1, BF16_CODE_BIAS = 24, 44, 127 * 128


def bf16_magnitude_code(x: torch.Tensor) -> torch.Tensor:
    """L(x): the 15 exponent-and-mantissa bits of a bf16 value as an integer.  L / 128 - 127 <= log2 |x| <=
    L / 128 - 127 + 0.0861 for normal values (a piecewise-linear logarithm)."""
    assert x.dtype == torch.bfloat16
    return x.contiguous().view(torch.int16).to(torch.int32) & 0x7FFF


def rowseg_max_codes(a: torch.Tensor, b: Optional[torch.Tensor] = None, seg: int = 64) -> torch.Tensor:
    """One code per `seg` consecutive columns of a row: the largest L in the segment (of a, or of a and b), laid out
    [ceil(cols / seg)][rows] like the product's arrays."""
    rows, cols = a.shape
    nseg = -(-cols // seg)
    la = bf16_magnitude_code(a) if b is None else torch.maximum(bf16_magnitude_code(a), bf16_magnitude_code(b))
    padded = torch.zeros((rows, nseg * seg), dtype=torch.int32)
    padded[:, :cols] = la
    return padded.view(rows, nseg, seg).amax(dim=2).t().contiguous().reshape(-1)


def swiglu_gradient_code_bounds(code_sum: torch.Tensor):
    """Largest L a gradient can have where the codes of gh and of (x1, x3) sum to `code_sum`: (for g1, for g3)."""
    return code_sum + SWIGLU_MARGIN_G1 - BF16_CODE_BIAS, code_sum + SWIGLU_MARGIN_G3 - BF16_CODE_BIAS


def mlp_fwd_bwd(x, w1, w2, w3, grad_out, spec: LinearSpec) -> MLPTrace:
    """y = w2(silu(w1 x) * w3 x); all three projections float8; backward through all of them."""
    t1 = linear_forward(x, w1, None, spec)
    t3 = linear_forward(x, w3, None, spec)
    h = swiglu(t1.out, t3.out)
    t2 = linear_forward(h, w2, None, spec)
    tr = MLPTrace(y=t2.out, h=h, linears={"w1": t1, "w2": t2, "w3": t3})
    if grad_out is None:
        return tr
    linear_backward(h, w2, grad_out, spec, t2)
    g1, g3 = swiglu_backward(t1.out, t3.out, t2.grad_input)
    linear_backward(x, w1, g1, spec, t1)
    linear_backward(x, w3, g3, spec, t3)
    tr.grad_x = t1.grad_input + t3.grad_input
    tr.grad_w1, tr.grad_w2, tr.grad_w3 = t1.grad_weight, t2.grad_weight, t3.grad_weight
    return tr


# --------------------------------------------------------------------------------------------
# model swap (torchao ``convert_to_float8_training`` walk + olmo_core's filter)
# --------------------------------------------------------------------------------------------


def expected_swaps(model: torch.nn.Module, modules_to_ignore: Optional[Sequence[str]] = None) -> List[str]:
    """
    Names of the nn.Linear modules that the reference converts: every Linear whose fqn is not ignored
    and whose weight dims are all multiples of 16 (src/olmo_core/float8/__init__.py:86-98).
    """
    ignore = set(modules_to_ignore or ())
    names = []
    for fqn, m in model.named_modules():
        if isinstance(m, torch.nn.Linear) and fqn not in ignore:
            if all(d % 16 == 0 for d in m.weight.shape):
                names.append(fqn)
    return names


# --------------------------------------------------------------------------------------------
# grouped (dropless MoE experts): per-expert loop of src/olmo_core/nn/moe/mlp.py:264-270 with the
# rowwise float8 linear applied to each expert's slice independently.
# --------------------------------------------------------------------------------------------


def grouped_linear_fwd_bwd(
    x: torch.Tensor,
    w: torch.Tensor,
    batch_sizes: Sequence[int],
    grad_out: Optional[torch.Tensor],
    spec: LinearSpec,
    trans_b: bool,
):
    """
    x [T,K]; w [E,N,K] if trans_b (out = x_e @ w[e].t()) else [E,K,N] (out = x_e @ w[e]).
    Returns (out [T,N], grad_x [T,K] or None, grad_w like w or None, per-expert traces).
    """
    outs, gxs, gws, traces = [], [], [], []
    start = 0
    for e, size in enumerate(int(s) for s in batch_sizes):
        w_e = w[e] if trans_b else w[e].t()  # -> [N, K] nn.Linear layout
        xe = x[start : start + size]
        if size == 0:
            outs.append(x.new_zeros((0, w_e.shape[0])))
            gxs.append(x.new_zeros((0, x.shape[1])))
            gws.append(torch.zeros_like(w[e]))
            traces.append(None)
            continue
        tr = linear_forward(xe, w_e, None, spec)
        outs.append(tr.out)
        if grad_out is not None:
            linear_backward(xe, w_e, grad_out[start : start + size], spec, tr)
            gxs.append(tr.grad_input)
            gws.append(tr.grad_weight if trans_b else tr.grad_weight.t())
        traces.append(tr)
        start += size
    out = torch.cat(outs)
    if grad_out is None:
        return out, None, None, traces
    return out, torch.cat(gxs), torch.stack(gws), traces


def dropless_mlp_fwd_bwd(x, w1, w2, w3, batch_sizes, grad_out, spec: LinearSpec):
    """
    DroplessMoEMLP.forward (src/olmo_core/nn/moe/mlp.py:272-292): w1,w3 [E,H,D] used transposed,
    w2 [E,H,D] used as-is; h = silu(x1) * x2.
    Returns dict with y and (if grad_out) grad_x, grad_w1, grad_w2, grad_w3.
    """
    x1, _, _, _ = grouped_linear_fwd_bwd(x, w1, batch_sizes, None, spec, trans_b=True)
    x2, _, _, _ = grouped_linear_fwd_bwd(x, w3, batch_sizes, None, spec, trans_b=True)
    h = swiglu(x1, x2)
    y, gh, gw2, _ = grouped_linear_fwd_bwd(h, w2, batch_sizes, grad_out, spec, trans_b=False)
    res = {"y": y, "h": h, "x1": x1, "x2": x2}
    if grad_out is None:
        return res
    g1, g2 = swiglu_backward(x1, x2, gh)
    _, gx_a, gw1, _ = grouped_linear_fwd_bwd(x, w1, batch_sizes, g1, spec, trans_b=True)
    _, gx_b, gw3, _ = grouped_linear_fwd_bwd(x, w3, batch_sizes, g2, spec, trans_b=True)
    res.update(grad_x=gx_a + gx_b, grad_w1=gw1, grad_w2=gw2, grad_w3=gw3, grad_h=gh, g1=g1, g2=g2)
    return res


# --------------------------------------------------------------------------------------------
# routing that produces the ragged group sizes (src/olmo_core/nn/moe/router.py:339-359,
# src/olmo_core/ops/moe.py:289-297, src/olmo_core/nn/moe/parallel_mlp.py:102-125)
# --------------------------------------------------------------------------------------------


def batched_histc(x: torch.Tensor, num_classes: int) -> torch.Tensor:
    hist = torch.zeros((*x.shape[:-1], num_classes), dtype=x.dtype)
    hist.scatter_add_(-1, x, torch.ones_like(x))
    return hist


def route_top_k(logits: torch.Tensor, top_k: int):
    """softmax -> topk -> histogram -> sort: returns (indices, bin_ids, bins, batch_size_per_expert)."""
    scores = logits.float().softmax(dim=-1)
    _, expert_indices = torch.topk(scores, top_k, dim=-1)
    flat = expert_indices.reshape(-1)
    batch_size_per_expert = batched_histc(flat.unsqueeze(0), logits.shape[-1])[0]
    bin_ids, indices = torch.sort(flat.int())
    bins = torch.cumsum(batch_size_per_expert, 0).to(torch.int32)
    return indices.int(), bin_ids, bins, batch_size_per_expert

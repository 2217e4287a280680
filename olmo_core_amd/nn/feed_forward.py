"""
SwiGLU feed-forward block: the host of the float8 linears in the dense models
(reference: src/olmo_core/nn/feed_forward.py:142-171, ``w2(silu(w1(x)) * w3(x))``; flops convention
:206-209).  The three projections are ordinary ``nn.Linear`` modules so that
``Float8Config.apply_float8_linear`` swaps them.

When all three are tensorwise ``Float8Linear`` modules without bias the block runs as one autograd function
that performs exactly the casts and GEMMs the three modules would perform one by one (same bytes, same scales,
same outputs), but quantises ``x`` once for ``w1`` and ``w3``, takes the amax of ``h`` and of the two gate
gradients inside the SwiGLU kernels that produce them (no separate pass over the largest tensors), and saves
fp8 copies instead of the bf16 activations ``x`` and ``h``.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from ..float8 import ops
from ..float8.linear import Float8Linear, _is_tensorwise, _shared_tensorwise

__all__ = ["FeedForward", "swiglu"]

# Test hook: when set to a dict, the fused function stores clones of its bf16 intermediates (x1, x3, h, gh) there,
# so that a checker can feed each stage's actual input to a reference of that stage, together with the float8
# operands it made of h, g1 and g3 and their scales (sh, hq, sg1, g1q, sg3, g3q): what the GEMMs actually consumed.
STAGE_SINK = None

# Run the two input projections and the SwiGLU between them as one launch where the shape allows (same bits as the
# three separate launches); a switch so that the two routes can be compared.
FUSE_SWIGLU_EPILOGUE = True

# Take the amax of the two gate gradients from the row-segment codes that the fused forward launch and the GEMM that
# produces grad_h record (same bits as the pass over gh, x1 and x3 it replaces); a switch so that the two routes can be
# compared.
SWIGLU_AMAX_FROM_CODES = True


class _SwiGLU(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x1: torch.Tensor, x3: torch.Tensor):
        h, _ = ops.swiglu_fwd(x1, x3, want_amax=False)
        ctx.save_for_backward(x1, x3)
        return h

    @staticmethod
    def backward(ctx, gh: torch.Tensor):
        x1, x3 = ctx.saved_tensors
        g1, g3, _, _ = ops.swiglu_bwd(x1, x3, gh, want_amax=False)
        return g1, g3


@torch.compiler.disable
def swiglu(x1: torch.Tensor, x3: torch.Tensor) -> torch.Tensor:
    """``silu(x1) * x3`` for bfloat16 GPU tensors (one fused kernel forward, one backward)."""
    return _SwiGLU.apply(x1, x3)


def _use_codes(M: int, D: int, H: int, any_grad: bool) -> bool:
    """Whether the fused forward launch records the row-segment codes of x1 and x3 for the backward pass."""
    return any_grad and SWIGLU_AMAX_FROM_CODES and H % 64 == 0


def _fused_launch_ok(M: int, D: int, H: int) -> bool:
    return FUSE_SWIGLU_EPILOGUE and ops.swiglu_gemm_matches_separate(M, H, D)


def _mlp_forward(x, w1, w2, w3, c, need, ws=(None, None, None), wo=(None, None, None)):
    """y = (silu(x W1^T) * (x W3^T)) W2^T with tensorwise float8 GEMMs; x [M, D], W1/W3 [H, D], W2 [D, H].  x is
    converted to bfloat16 first if it is of another type (float32 activations under autocast: each of the three
    modules would convert its own input).
    need: which of (x, w1, w2, w3) get a gradient.  ws: weight scales precomputed after the optimizer step (None: reduce
    the amax here); wo: float8 copies the modules keep between calls (None: quantise the weight here); both in the
    order (w1, w2, w3).  Returns ``(y, saved)``, ``saved`` being the 13 tensors :func:`_mlp_backward` takes (an empty
    tensor where nothing is kept)."""
    pow2 = c.round_scales_to_power_of_2
    in_dt, w_dt = c.cast_config_input.target_dtype, c.cast_config_weight.target_dtype
    any_grad = any(need)
    ws1, ws2, ws3 = ws
    wo1, wo2, wo3 = wo
    x_codes = None
    if x.dtype != torch.bfloat16:
        x = x.to(torch.bfloat16)
    # The amax of x and of every weight that still needs one is taken in a single launch.
    todo = [x] + [w for w, s, o in ((w1, ws1, wo1), (w3, ws3, wo3), (w2, ws2, wo2)) if s is None and o is None]
    part = {}
    if len(todo) > 1 and all(t.dtype == x.dtype and t.is_contiguous() for t in todo):
        part = {id(t): p for t, p in zip(todo, ops.amax_partials_batch(todo))}
    xq, xq_t, sx = ops.cast_tensorwise(x, in_dt, pow2=pow2, want_transposed=need[1] or need[3], slots=part.get(id(x)))
    w1q, w1q_t, s1 = wo1 or ops.cast_tensorwise(w1, w_dt, pow2=pow2, want_transposed=need[0], scale=ws1,
                                                slots=part.get(id(w1)))
    w3q, w3q_t, s3 = wo3 or ops.cast_tensorwise(w3, w_dt, pow2=pow2, want_transposed=need[0], scale=ws3,
                                                slots=part.get(id(w3)))
    w2q, w2q_t, s2 = wo2 or ops.cast_tensorwise(w2, w_dt, pow2=pow2, want_transposed=any_grad, scale=ws2,
                                                slots=part.get(id(w2)))
    M, D, H = x.shape[0], x.shape[1], w1.shape[0]
    if _fused_launch_ok(M, D, H):
        # both input projections and the activation in one launch: x1 and x3 are never read back
        if _use_codes(M, D, H, any_grad):
            x1, x3, h, h_slots, x_codes = ops.gemm_fp8_swiglu(xq, sx, w1q, s1, w3q, s3, want_codes=True)
        else:
            x1, x3, h, h_slots = ops.gemm_fp8_swiglu(xq, sx, w1q, s1, w3q, s3)
    else:
        x1 = ops.gemm_fp8(xq, sx, w1q, s1, out_dtype=x.dtype)
        x3 = ops.gemm_fp8(xq, sx, w3q, s3, out_dtype=x.dtype)
        h, h_slots = ops.swiglu_fwd(x1, x3, want_amax=True)
    if STAGE_SINK is not None:
        STAGE_SINK.update(x1=x1.clone(), x3=x3.clone(), h=h.clone())
    hq, hq_t, sh = ops.cast_tensorwise(h, in_dt, pow2=pow2, want_transposed=need[2], slots=h_slots)
    if STAGE_SINK is not None:
        STAGE_SINK.update(sh=sh.clone(), hq=hq.clone())
    y = ops.gemm_fp8(hq, sh, w2q, s2, out_dtype=x.dtype)
    opt = lambda t: t if t is not None else x.new_empty(0)  # noqa: E731
    saved = (opt(xq_t), sx, x1, x3, opt(hq_t), sh, opt(w1q_t), s1, opt(w2q_t), s2, opt(w3q_t), s3, opt(x_codes))
    return y, saved


def _mlp_backward(gy, saved, c, dims, dtypes, need):
    """The four gradients ``(gx, gw1, gw2, gw3)`` (``None`` where not needed) of :func:`_mlp_forward`.  dtypes: of the
    x the forward was given and of the three weights.  For a bfloat16 x the two grad_x terms are added by the second
    GEMM's epilogue; for an x of another type they are added in that type, as autograd adds the converted-back
    gradients of the two modules that each converted x."""
    xq_t, sx, x1, x3, hq_t, sh, w1q_t, s1, w2q_t, s2, w3q_t, s3, x_codes = saved
    pow2 = c.round_scales_to_power_of_2
    go_dt = c.cast_config_grad_output.target_dtype
    gx_dt, w1_dt, w2_dt, w3_dt = dtypes
    x_dt = torch.bfloat16
    M, D, H = dims
    need_x, need_w1, need_w2, need_w3 = need
    gy = gy.reshape(M, D)
    if gy.dtype != x_dt:
        gy = gy.to(x_dt)
    need_gh = need_x or need_w1 or need_w3
    gyq, gyq_t, sgy = ops.cast_tensorwise(gy, go_dt, pow2=pow2, want_rowmajor=need_gh, want_transposed=need_w2)
    gw2 = ops.gemm_fp8(gyq_t, sgy, hq_t, sh, out_dtype=x_dt) if need_w2 else None
    gx = gw1 = gw3 = None
    if need_gh:
        # g1 and g3 are needed in fp8 only, and their tensorwise scales need the amax of both first.  Where the
        # forward recorded the row-segment codes of x1 and x3, the GEMM that produces gh records those of gh, and the
        # amax follows by computing a small share of the segments; otherwise a pass over the three tensors takes it.
        codes = None
        if x_codes.numel() and x_dt == torch.bfloat16 and ops.gemm_codes_supported(M, H, D):
            gh, gh_codes = ops.gemm_fp8_codes(gyq, sgy, w2q_t, s2, k=D)
            codes = (gh_codes, x_codes)
        else:
            gh = ops.gemm_fp8(gyq, sgy, w2q_t, s2, k=D, out_dtype=x_dt)
        if STAGE_SINK is not None:
            STAGE_SINK.update(gh=gh.clone())
        need_t = need_w1 or need_w3
        # then the recompute-and-cast pass (no bf16 round trip of g1, g3)
        g1q, g1q_t, sg1, g3q, g3q_t, sg3 = ops.swiglu_bwd_cast(
            x1, x3, gh, go_dt, pow2=pow2, want_rowmajor=need_x, want_transposed=need_t, codes=codes)
        del gh
        if STAGE_SINK is not None:
            STAGE_SINK.update(sg1=sg1.clone(), sg3=sg3.clone(), amax_from_codes=codes is not None,
                              g1q=None if g1q is None else g1q.clone(), g3q=None if g3q is None else g3q.clone())
        if need_x and gx_dt == x_dt:
            # the sum of the two halves as autograd forms it (two bf16 tensors added), by the second GEMM's epilogue
            gx = ops.gemm_fp8(g1q, sg1, w1q_t, s1, k=H, out_dtype=x_dt)
            ops.gemm_fp8(g3q, sg3, w3q_t, s3, k=H, out_dtype=x_dt, out=gx, accumulate=True)
        elif need_x:
            # (autograd runs w3's backward first: its term is the one the other is added to)
            gx = ops.gemm_fp8(g3q, sg3, w3q_t, s3, k=H, out_dtype=x_dt).to(gx_dt)
            gx.add_(ops.gemm_fp8(g1q, sg1, w1q_t, s1, k=H, out_dtype=x_dt))
        if need_w1:
            gw1 = ops.gemm_fp8(g1q_t, sg1, xq_t, sx, out_dtype=x_dt)
        if need_w3:
            gw3 = ops.gemm_fp8(g3q_t, sg3, xq_t, sx, out_dtype=x_dt)

    def as_param(g, dt):
        return g if g is None or g.dtype == dt else g.to(dt)

    return gx, as_param(gw1, w1_dt), as_param(gw2, w2_dt), as_param(gw3, w3_dt)


class _Float8SwiGLUMLP(torch.autograd.Function):
    """The fused block as an eager autograd function (a traced graph takes the registered operators of
    ``olmo_core_amd.float8.compiled`` instead, which run the same two routines)."""

    @staticmethod
    def forward(ctx, x, w1, w2, w3, config, ws1=None, ws2=None, ws3=None, wo1=None, wo2=None, wo3=None):
        need = tuple(ctx.needs_input_grad[:4])
        y, saved = _mlp_forward(x, w1, w2, w3, config, need, (ws1, ws2, ws3), (wo1, wo2, wo3))
        ctx.config = config
        ctx.dtypes = (x.dtype, w1.dtype, w2.dtype, w3.dtype)
        ctx.dims = (x.shape[0], x.shape[1], w1.shape[0])
        ctx.save_for_backward(*saved)
        return y

    @staticmethod
    def backward(ctx, gy):
        grads = _mlp_backward(gy, ctx.saved_tensors, ctx.config, ctx.dims, ctx.dtypes, tuple(ctx.needs_input_grad[:4]))
        return grads + (None,) * 7


def _fusable_modules(ff: "FeedForward", same_object: bool = False) -> bool:
    """The three projections are float8 modules of one tensorwise config without bias.  same_object: only accept one
    shared config object (what a model conversion hands to every module), without comparing configs field by field:
    the form a traced graph evaluates."""
    if not ff.fuse_float8:
        return False
    for m in (ff.w1, ff.w2, ff.w3):
        if not isinstance(m, Float8Linear) or m.bias is not None:
            return False
    c = ff.w1.config
    for m in (ff.w2, ff.w3):
        if m.config is not c and (same_object or m.config != c):
            return False
    return (
        _shared_tensorwise(c.cast_config_input, c.cast_config_input_for_grad_weight)
        and _shared_tensorwise(c.cast_config_weight, c.cast_config_weight_for_grad_input)
        and _shared_tensorwise(c.cast_config_grad_output, c.cast_config_grad_output_for_grad_weight)
    )


@torch.compiler.disable
def _fused_mlp(x2, w1, w2, w3, config, ws1=None, ws2=None, ws3=None, wo1=None, wo2=None, wo3=None):
    return _Float8SwiGLUMLP.apply(x2, w1, w2, w3, config, ws1, ws2, ws3, wo1, wo2, wo3)


class FeedForward(nn.Module):
    """Gated feed-forward with SiLU activation: ``w2(silu(w1 x) * w3 x)``."""

    def __init__(
        self,
        *,
        d_model: int,
        hidden_size: int,
        bias: bool = True,
        dtype: torch.dtype = torch.float32,
        init_device: str = "cpu",
        fuse_float8: bool = True,
    ):
        super().__init__()
        self.d_model = d_model
        self.hidden_size = hidden_size
        self.fuse_float8 = fuse_float8
        self.w1 = nn.Linear(d_model, hidden_size, bias=bias, dtype=dtype, device=init_device)
        self.w2 = nn.Linear(hidden_size, d_model, bias=bias, dtype=dtype, device=init_device)
        self.w3 = nn.Linear(d_model, hidden_size, bias=bias, dtype=dtype, device=init_device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        # The fused block does what the three modules do one by one, including their first step under autocast (the
        # input goes to the autocast type: src/olmo_core/train/train_module/transformer/train_module.py:593-597 runs the
        # model that way); it takes bfloat16 activations on the GPU.
        compiling = torch.compiler.is_compiling()
        act_dtype = torch.get_autocast_dtype("cuda") if x.is_cuda and torch.is_autocast_enabled() else x.dtype
        xa = x  # (the conversion to the autocast type happens inside the fused function)
        if compiling:
            # a traced graph (the reference compiles every block, src/olmo_core/nn/transformer/block.py:78-79) keeps the
            # fused launches: the block is one registered operator with a shape function
            cfg_id = getattr(self.w1.config, "_compiled_id", -1) if _fusable_modules(self, same_object=True) else -1
            if cfg_id >= 0 and xa.is_cuda and act_dtype == torch.bfloat16:
                from ..float8 import compiled

                x2 = xa.reshape(-1, xa.shape[-1])
                y = compiled.swiglu_mlp(x2, self.w1.weight, self.w2.weight, self.w3.weight, cfg_id,
                                        (self.w1._module_id, self.w2._module_id, self.w3._module_id))
                return y.reshape(*x.shape[:-1], self.w2.weight.shape[0])
        elif xa.is_cuda and act_dtype == torch.bfloat16 and _fusable_modules(self):
            x2 = xa.reshape(-1, xa.shape[-1])
            y = _fused_mlp(x2, self.w1.weight, self.w2.weight, self.w3.weight, self.w1.config,
                           self.w1.precomputed_weight_scale(), self.w2.precomputed_weight_scale(),
                           self.w3.precomputed_weight_scale(), self.w1.weight_operands(), self.w2.weight_operands(),
                           self.w3.weight_operands())
            return y.reshape(*x.shape[:-1], self.w2.weight.shape[0])
        x1, x3 = self.w1(x), self.w3(x)
        if x1.is_cuda and x1.dtype == torch.bfloat16 and not compiling:
            h = swiglu(x1, x3)
        else:
            h = torch.nn.functional.silu(x1) * x3
        return self.w2(h)

    def num_flops_per_token(self, seq_len: int) -> int:
        del seq_len
        return 6 * sum(p.numel() for p in self.parameters())

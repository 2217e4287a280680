"""
Dropless-MoE expert MLP with float8 grouped GEMMs.

Same parameters and call signature as the reference's ``DroplessMoEMLP`` (reference:
src/olmo_core/nn/moe/mlp.py:198-292): ``w1, w2, w3`` of shape ``[num_experts * hidden_size, d_model]``,
``forward(x [T, d_model], batch_size_per_expert [E])`` with the rows of ``x`` already permuted so that each
expert's tokens are consecutive, ``w1``/``w3`` used transposed and ``w2`` as stored, ``h = silu(x1) * x2``.
The reference runs the expert GEMMs in bf16 (its float8 conversion never touches these raw Parameters); here
every expert's slice goes through the axiswise float8 recipe (per-row scales for activations, per-channel
scales per expert for weights, per-group column scales for the weight gradients, e4m3 everywhere, power-of-two
scales) on ragged grouped kernels.  Group sizes stay on the device: there is no host synchronisation.
"""

from __future__ import annotations

import math

import torch
import torch.nn as nn

from ..float8 import ops

__all__ = ["DroplessMoEMLP", "float8_dropless_mlp"]

_E4M3 = torch.float8_e4m3fn

# Test hook: when set to a dict, the expert MLP stores clones of its bf16 intermediates (x1, x2, h, gh, g1, g2)
# there, so that a checker can feed each stage's actual input to a reference of that stage.
STAGE_SINK = None

# The grad_input of the expert layer (the sum of the gate and up projections' terms) as one grouped GEMM over both
# contractions where the shape allows; False: two launches, the second adding into the first one's output (each term
# rounded to bf16 before the sum).
DUAL_GRAD_INPUT = True


class _Float8DroplessMLP(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, w1, w2, w3, sizes, num_experts, pow2, indices=None, top_k=1, kept=None, scatter_weights=None):
        # indices: None - the rows of x are already sorted by expert; else x is [tokens, D] in token order and row i
        # of the expert-sorted side is token indices[i] // top_k: the gather is fused into the casts of x.
        # scatter_weights (with indices): the expert outputs are scattered back to token order, weighted per slot,
        # inside this function, so that the backward can quantise the weighted gather of grad_output directly
        E = num_experts
        D = x.shape[1]
        T = x.shape[0] if indices is None else x.shape[0] * top_k
        H = w1.shape[0] // E
        dev = x.device
        equal = torch.full((E,), H, dtype=torch.int64, device=dev)  # the experts' weights as equal-size groups
        # in the transposed copies every expert's segment starts on a multiple of 128 columns
        Hp = (H + 127) // 128 * 128

        need = ctx.needs_input_grad
        need_w13 = need[1] or need[3]
        any_grad = any(need[:4])
        # operands that are needed in both layouts (by rows for the forward / grad-input GEMMs, by the group's
        # columns for the weight-gradient GEMMs) come out of one pair of passes
        xt = sxc = ht = shc = w1t = s1c = w3t = s3c = w2q = s2r = None
        if indices is not None:
            xq, sx, xt, sxc = ops.gather_cast_rows_and_colwise_t(x, indices, top_k, sizes, _E4M3, pow2=pow2)
        elif need_w13:
            xq, sx, xt, sxc = ops.grouped_cast_rows_and_colwise_t(x, sizes, _E4M3, pow2=pow2)
        else:
            xq, sx = ops.cast_rowwise(x, _E4M3, pow2=pow2)
        # w1/w3: one scale per output channel (row of w[e]) forward, per input channel of w[e] for grad_input
        # (kept: the float8 copies of the three weights made by an earlier call and still valid)
        if kept is not None:
            (w1q, s1, w1t, s1c), (w3q, s3, w3t, s3c), _ = kept
        elif need[0]:
            w1q, s1, w1t, s1c = ops.grouped_cast_rows_and_colwise_t(w1, equal, _E4M3, pow2=pow2)
            w3q, s3, w3t, s3c = ops.grouped_cast_rows_and_colwise_t(w3, equal, _E4M3, pow2=pow2)
        else:
            w1q, s1 = ops.cast_rowwise(w1, _E4M3, pow2=pow2)
            w3q, s3 = ops.cast_rowwise(w3, _E4M3, pow2=pow2)
        x1 = ops.grouped_gemm_fp8(xq, sx, w1q, s1, sizes, n=H, k=D, b_group_stride=H * w1q.stride(0), sb_group_stride=H)
        x2 = ops.grouped_gemm_fp8(xq, sx, w3q, s3, sizes, n=H, k=D, b_group_stride=H * w3q.stride(0), sb_group_stride=H)
        if need[2]:
            # the pointwise kernel also takes the amax of h per row and per (expert, column): the cast is one pass
            h, h_amax = ops.grouped_swiglu_fwd(x1, x2, sizes)
            if STAGE_SINK is not None:
                STAGE_SINK.update(x1=x1.clone(), x2=x2.clone(), h=h.clone())
            hq, sh, ht, shc = ops.grouped_cast_rows_and_colwise_t(h, sizes, _E4M3, pow2=pow2, amax=h_amax)
        else:
            h, _ = ops.swiglu_fwd(x1, x2, want_amax=False)
            hq, sh = ops.cast_rowwise(h, _E4M3, pow2=pow2)
        del h
        # w2[e] is [H, D] and is used as-is (h_e @ w2[e]): its output channel is the column -> transposed copy
        # [D, E*H] with one scale per (expert, column); the by-rows copy is the grad_h GEMM's right operand
        if kept is not None:
            w2q, s2r, w2t, s2 = kept[2]
        elif any_grad:
            w2q, s2r, w2t, s2 = ops.grouped_cast_rows_and_colwise_t(w2, equal, _E4M3, pow2=pow2)
        else:
            w2t, s2 = ops.grouped_cast_colwise_t(w2, equal, _E4M3, pow2=pow2)
        y = ops.grouped_gemm_fp8(hq, sh, w2t, s2, sizes, n=D, k=H, b_group_stride=Hp, sb_group_stride=D)
        none = x.new_empty(0)
        opt = lambda t: none if t is None else t  # noqa: E731
        y_sorted = None
        ctx.scattered = scatter_weights is not None
        if ctx.scattered:
            from ..ops import moe as moe_ops

            if indices is None:
                raise ValueError("scatter_weights needs the permutation (indices)")
            if len(need) > 10 and need[10]:
                y_sorted = y  # the router-weight gradient is a dot product with the unweighted expert output
            y = moe_ops._scatter(y, indices, scatter_weights, top_k)
        ctx.save_for_backward(opt(xt), opt(sxc), x1, x2, opt(ht), opt(shc), opt(w1t), opt(s1c), opt(w3t), opt(s3c),
                              opt(w2q), opt(s2r), sizes, opt(indices), opt(scatter_weights), opt(y_sorted))
        ctx.top_k = top_k if indices is not None else 0
        ctx.meta = (E, T, D, H, Hp, pow2, (x.dtype, w1.dtype, w2.dtype, w3.dtype))
        return y

    @staticmethod
    def backward(ctx, gy):
        (xt, sxc, x1, x2, ht, shc, w1t, s1c, w3t, s3c, w2q, s2r, sizes, indices, scatter_weights,
         y_sorted) = ctx.saved_tensors
        E, T, D, H, Hp, pow2, (x_dt, w1_dt, w2_dt, w3_dt) = ctx.meta
        gy = gy.reshape(-1, D).contiguous()
        if gy.dtype != x_dt:
            gy = gy.to(x_dt)
        need_x, need_w1, need_w2, need_w3 = ctx.needs_input_grad[:4]

        gw2 = g_router = None
        if ctx.scattered:
            # gy is in token order: the gradient of the expert outputs is its weighted gather, which goes straight to
            # float8 (both layouts) without being written in bf16
            from ..ops import moe as moe_ops

            if y_sorted.numel():
                g_router = moe_ops._scatter_wgrad(y_sorted, gy, indices, ctx.top_k)
                if g_router.dtype != scatter_weights.dtype:
                    g_router = g_router.to(scatter_weights.dtype)
            gyq, sgy, gyt, sgyc = ops.gather_cast_rows_and_colwise_t(gy, indices, ctx.top_k, sizes, _E4M3, pow2=pow2,
                                                                     weights=scatter_weights)
            if need_w2:
                gw2 = ops.grouped_wgrad_fp8(ht, shc, gyt, sgyc, sizes, tokens=T, out_dtype=x_dt).reshape(E * H, D)
            del gyt
        elif need_w2:
            gyq, sgy, gyt, sgyc = ops.grouped_cast_rows_and_colwise_t(gy, sizes, _E4M3, pow2=pow2)
            # gw2[e] [H, D] = h_e^T @ gy_e : contraction over the group's tokens
            gw2 = ops.grouped_wgrad_fp8(ht, shc, gyt, sgyc, sizes, tokens=T, out_dtype=x_dt).reshape(E * H, D)
            del gyt
        else:
            gyq, sgy = ops.cast_rowwise(gy, _E4M3, pow2=pow2)
        gx = gw1 = gw3 = None
        if need_x or need_w1 or need_w3:
            # gh_e = gy_e @ w2[e]^T : contraction over D, the right operand is w2[e] itself, one scale per row
            gh = ops.grouped_gemm_fp8(gyq, sgy, w2q, s2r, sizes, n=H, k=D, b_group_stride=H * w2q.stride(0),
                                      sb_group_stride=H)
            fused_amax = need_x and (need_w1 or need_w3)
            if fused_amax:
                g1, g2, amax1, amax2 = ops.grouped_swiglu_bwd(x1, x2, gh, sizes)
            else:
                g1, g2, _, _ = ops.swiglu_bwd(x1, x2, gh, want_amax=False)
                amax1 = amax2 = None
            if STAGE_SINK is not None:
                STAGE_SINK.update(gh=gh.clone(), g1=g1.clone(), g2=g2.clone())
            del gh

            def both(g, want_rows, want_cols, amax):
                if want_rows and want_cols:
                    return ops.grouped_cast_rows_and_colwise_t(g, sizes, _E4M3, pow2=pow2, amax=amax)
                if want_rows:
                    return (*ops.cast_rowwise(g, _E4M3, pow2=pow2), None, None)
                if want_cols:
                    return (None, None, *ops.grouped_cast_colwise_t(g, sizes, _E4M3, pow2=pow2))
                return None, None, None, None

            g1q, sg1, g1t, sg1c = both(g1, need_x, need_w1, amax1)
            g2q, sg2, g2t, sg2c = both(g2, need_x, need_w3, amax2)
            del g1, g2
            if need_x and DUAL_GRAD_INPUT and pow2 and ops.grouped_gemm_dual_supported(T, D, H, H):
                # gx_e = g1_e @ w1[e] + g2_e @ w3[e] as ONE contraction over 2 H: the scales of both products (powers of
                # two) are applied inside the matrix instructions, so the terms meet in one float32 accumulator
                gx = ops.grouped_gemm_fp8_dual(g1q, sg1, w1t, s1c, g2q, sg2, w3t, s3c, sizes, n=D, k1=H, k2=H,
                                               b_group_stride=Hp, sb_group_stride=D)
            elif need_x:
                # gx_e = g_e @ w[e] : contraction over H, the right operand is w[e]^T [D, H], one scale per input channel
                gx = ops.grouped_gemm_fp8(g1q, sg1, w1t, s1c, sizes, n=D, k=H, b_group_stride=Hp, sb_group_stride=D)
                ops.grouped_gemm_fp8(g2q, sg2, w3t, s3c, sizes, n=D, k=H, b_group_stride=Hp, sb_group_stride=D,
                                     accumulate_into=gx)
            if need_w1:
                gw1 = ops.grouped_wgrad_fp8(g1t, sg1c, xt, sxc, sizes, tokens=T, out_dtype=x_dt).reshape(E * H, D)
            if need_w3:
                gw3 = ops.grouped_wgrad_fp8(g2t, sg2c, xt, sxc, sizes, tokens=T, out_dtype=x_dt).reshape(E * H, D)

        def as_param(g, dt):
            return g if g is None or g.dtype == dt else g.to(dt)

        if gx is not None and ctx.top_k:
            # the gather's backward: every token sums the gradients of its top_k slots (the scatter kernel, unweighted)
            from ..ops import moe as moe_ops

            gx = moe_ops._scatter(gx, indices, None, ctx.top_k)
        return (gx, as_param(gw1, w1_dt), as_param(gw2, w2_dt), as_param(gw3, w3_dt), None, None, None, None, None, None,
                g_router)


@torch.compiler.disable
def float8_dropless_mlp(x, w1, w2, w3, batch_size_per_expert, num_experts: int, pow2: bool = True, indices=None,
                        top_k: int = 1, kept=None, scatter_weights=None):
    """``gmm(silu(gmm(x, w1^T)) * gmm(x, w3^T), w2)`` with float8 grouped GEMMs; ``x`` is ``[T, d_model]`` bf16 with
    rows sorted by expert, or, with ``indices`` (int32 ``[tokens * top_k]``, the slot held by each sorted row),
    ``[tokens, d_model]`` in token order: the result is then the expert output of the gathered rows,
    ``[tokens * top_k, d_model]``, and the gather never writes its bf16 result.  With ``scatter_weights`` (one router
    weight per slot) the weighted scatter back to token order happens here as well (result ``[tokens, d_model]``), and
    the backward quantises the weighted gather of the incoming gradient without writing it in bf16 either."""
    return _Float8DroplessMLP.apply(x, w1, w2, w3, batch_size_per_expert, num_experts, pow2, indices, top_k, kept,
                                    scatter_weights)


class DroplessMoEMLP(nn.Module):
    """A dropless expert MLP module with SwiGLU activation and float8 grouped GEMMs."""

    def __init__(
        self,
        *,
        d_model: int,
        hidden_size: int,
        num_experts: int,
        dtype: torch.dtype = torch.float32,
        init_device: str = "cpu",
        keep_float8_weights: bool = False,
    ):
        super().__init__()
        if d_model % 16 or hidden_size % 16:
            raise ValueError("float8 grouped GEMMs need d_model and hidden_size to be multiples of 16")
        self.d_model = d_model
        self.hidden_size = hidden_size
        self.num_experts = num_experts
        # Keep the float8 copies of the expert weights (two layouts, 2 bytes per parameter) from one call to the
        # next for as long as the weights are not modified: the micro-batches of one optimizer step then quantise
        # the experts once (what enable_fsdp_float8_all_gather does for a Float8Linear).  Off: every call quantises.
        self.keep_float8_weights = keep_float8_weights
        self._kept = None
        shape = (num_experts * hidden_size, d_model)
        self.w1 = nn.Parameter(torch.empty(*shape, device=init_device, dtype=dtype))
        self.w2 = nn.Parameter(torch.empty(*shape, device=init_device, dtype=dtype))
        self.w3 = nn.Parameter(torch.empty(*shape, device=init_device, dtype=dtype))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        for w in (self.w1, self.w2, self.w3):
            if not w.is_meta:
                nn.init.kaiming_uniform_(w, a=math.sqrt(5))

    def weight_operands(self):
        """The float8 operands of the three expert weights, ``((w1q, s1, w1t, s1c), (w3q, ...), (w2q, s2r, w2t, s2))``
        as the expert function makes them itself, kept until a weight is modified or replaced (address and version
        counter; a write through ``.data`` goes unnoticed).  ``None`` unless ``keep_float8_weights``."""
        if not self.keep_float8_weights:
            return None
        ws = (self.w1, self.w3, self.w2)
        if not all(w.is_cuda and w.is_contiguous() and w.dtype in (torch.bfloat16, torch.float32) for w in ws):
            return None
        key = tuple((w.data_ptr(), w._version, w.dtype) for w in ws)
        if self._kept is not None and self._kept[0] == key:
            return self._kept[1]
        equal = torch.full((self.num_experts,), self.hidden_size, dtype=torch.int64, device=self.w1.device)
        with torch.no_grad():
            made = tuple(ops.grouped_cast_rows_and_colwise_t(w.detach(), equal, _E4M3, pow2=True) for w in ws)
        self._kept = (key, made)
        return made

    def forward(self, x: torch.Tensor, batch_size_per_expert: torch.Tensor) -> torch.Tensor:
        """
        :param x: the expert inputs of shape ``(*, d_model)``, rows ordered by expert.
        :param batch_size_per_expert: how many rows go to each expert, a 1-D ``LongTensor``.
        """
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.d_model)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        y = float8_dropless_mlp(x2, self.w1, self.w2, self.w3, batch_size_per_expert, self.num_experts,
                                kept=self.weight_operands())
        return y.reshape(*lead, self.d_model).to(x.dtype)

    def forward_gathered(self, x: torch.Tensor, indices: torch.Tensor, top_k: int,
                         batch_size_per_expert: torch.Tensor) -> torch.Tensor:
        """``forward(gather(x, indices, ..., top_k), batch_size_per_expert)`` (``olmo_core_amd.ops.moe.gather``) with
        the gather fused into the quantisation of the expert inputs: ``x`` is ``(tokens, d_model)`` in token order,
        the result ``(tokens * top_k, d_model)`` in expert order."""
        x2 = x.reshape(-1, self.d_model)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        y = float8_dropless_mlp(x2, self.w1, self.w2, self.w3, batch_size_per_expert, self.num_experts,
                                indices=indices, top_k=top_k, kept=self.weight_operands())
        return y.to(x.dtype)

    def forward_routed(self, x: torch.Tensor, indices: torch.Tensor, expert_weights: torch.Tensor, top_k: int,
                       batch_size_per_expert: torch.Tensor) -> torch.Tensor:
        """``scatter(forward(gather(x, ...)), ..., expert_weights, ...)`` (``olmo_core_amd.ops.moe``) as one autograd
        function: ``x`` ``(tokens, d_model)`` and the result are in token order; neither the gathered inputs nor, in
        backward, the weighted gather of the incoming gradient is written in bf16."""
        x2 = x.reshape(-1, self.d_model)
        if x2.dtype != torch.bfloat16:
            x2 = x2.to(torch.bfloat16)
        y = float8_dropless_mlp(x2, self.w1, self.w2, self.w3, batch_size_per_expert, self.num_experts,
                                indices=indices, top_k=top_k, kept=self.weight_operands(),
                                scatter_weights=expert_weights)
        return y.to(x.dtype)


class ParallelDroplessMLP(nn.Module):
    """
    Routing wrapper around :class:`DroplessMoEMLP`: sorts the token slots by expert, gathers the rows, runs the
    experts and scatters the weighted results back (reference ``ParallelDroplessMLP`` /
    ``ParallelMLPBase.forward``, ``src/olmo_core/nn/moe/parallel_mlp.py:102-183``, ``:634-666``, ``:851-871``).
    Single-device path only: expert parallelism needs more than one GPU.
    """

    def __init__(self, *, mlp: DroplessMoEMLP, top_k: int, fuse_gather: bool = True):
        super().__init__()
        self.mlp = mlp
        self.top_k = top_k
        # gather -> quantise in one pass (the gathered bf16 rows are never written); False: the separate gather op
        self.fuse_gather = fuse_gather

    @property
    def d_model(self) -> int:
        return self.mlp.d_model

    @property
    def num_experts(self) -> int:
        return self.mlp.num_experts

    def apply_ep(self, *args, **kwargs):
        raise NotImplementedError("expert parallelism is outside the single-GPU scope of this build")

    def indices_and_bins(self, expert_indices: torch.Tensor, batch_size_per_expert: torch.Tensor):
        """``(indices, bin_ids, bins)``: argsort of the flattened expert assignment, the sorted expert ids and
        the inclusive prefix sums of the per-expert counts (all int32)."""
        bin_ids, indices = torch.sort(expert_indices.int())
        bins = torch.cumsum(batch_size_per_expert, 0).to(torch.int32)
        return indices.int(), bin_ids, bins

    def forward(self, x, expert_weights, expert_indices, batch_size_per_expert):
        """
        :param x: ``(N, d_model)`` (any leading shape).
        :param expert_weights: ``(N, top_k)`` router weights.
        :param expert_indices: ``(N, top_k)`` expert ids.
        :param batch_size_per_expert: ``(num_experts,)`` token slots per expert.
        :returns: the output with the shape of ``x``.
        """
        in_shape = x.size()
        x = x.view(-1, x.shape[-1])
        expert_weights = expert_weights.flatten()
        expert_indices = expert_indices.flatten()
        with torch.no_grad():
            indices, bin_ids, bins = self.indices_and_bins(expert_indices, batch_size_per_expert)
        out = self.forward_once(x, expert_weights=expert_weights, expert_indices=expert_indices, indices=indices,
                                bin_ids=bin_ids, bins=bins, batch_size_per_expert=batch_size_per_expert)
        return out.view(in_shape)

    def forward_once(self, x, *, expert_weights, expert_indices, indices, bin_ids, bins, batch_size_per_expert):
        del expert_indices
        return self.permute_and_compute(x, batch_size_per_expert=batch_size_per_expert, indices=indices,
                                        bin_ids=bin_ids, expert_weights=expert_weights, bins=bins, top_k=self.top_k)

    def permute_and_compute(self, x, *, batch_size_per_expert, indices, bin_ids, expert_weights, bins, top_k: int):
        from ..ops import moe as moe_ops

        x = x.view(-1, x.shape[-1])
        if self.fuse_gather and x.is_cuda and expert_weights is not None:
            return self.mlp.forward_routed(x, indices, expert_weights, top_k, batch_size_per_expert)
        if self.fuse_gather and x.is_cuda:
            x = self.mlp.forward_gathered(x, indices, top_k, batch_size_per_expert)
        else:
            x = moe_ops.gather(x, indices, bin_ids, bins, top_k)
            x = self.mlp(x, batch_size_per_expert)
        return moe_ops.scatter(x, indices, bin_ids, expert_weights, bins, top_k)

"""
SwiGLU feed-forward block: the host of the float8 linears in the dense models
(reference: src/olmo_core/nn/feed_forward.py:142-171, ``w2(silu(w1(x)) * w3(x))``; flops convention
:206-209).  The three projections are ordinary ``nn.Linear`` modules so that
``Float8Config.apply_float8_linear`` swaps them; the gate runs in one HIP kernel per direction.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from ..float8 import ops

__all__ = ["FeedForward", "swiglu"]


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


def swiglu(x1: torch.Tensor, x3: torch.Tensor) -> torch.Tensor:
    """``silu(x1) * x3`` for bfloat16 GPU tensors (one fused kernel forward, one backward)."""
    return _SwiGLU.apply(x1, x3)


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
    ):
        super().__init__()
        self.d_model = d_model
        self.hidden_size = hidden_size
        self.w1 = nn.Linear(d_model, hidden_size, bias=bias, dtype=dtype, device=init_device)
        self.w2 = nn.Linear(hidden_size, d_model, bias=bias, dtype=dtype, device=init_device)
        self.w3 = nn.Linear(d_model, hidden_size, bias=bias, dtype=dtype, device=init_device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        x1, x3 = self.w1(x), self.w3(x)
        if x1.is_cuda and x1.dtype == torch.bfloat16:
            h = swiglu(x1, x3)
        else:
            h = torch.nn.functional.silu(x1) * x3
        return self.w2(h)

    def num_flops_per_token(self, seq_len: int) -> int:
        del seq_len
        return 6 * sum(p.numel() for p in self.parameters())

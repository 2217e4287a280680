"""Activation checkpointing over converted modules (the reference wraps transformer blocks in
torch.utils.checkpoint: full / selected-blocks modes re-run the block's forward in backward, the selected-ops mode
saves only aten.mm / abs / max outputs, src/olmo_core/nn/utils.py:12-48, so the float8 operators are recomputed).
The re-run must reproduce the first run bit for bit: outputs and every gradient equal those of the plain call."""

from collections import defaultdict

import pytest
import torch
from torch.utils.checkpoint import CheckpointPolicy, checkpoint, create_selective_checkpoint_contexts

from helpers import seeded

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import AOFloat8LinearRecipe, Float8Config  # noqa: E402
from olmo_core_amd.nn import FeedForward  # noqa: E402


def _block(dev, recipe, fuse, D=512, H=1280):
    g = torch.Generator().manual_seed(5)
    ff = FeedForward(d_model=D, hidden_size=H, bias=False, dtype=torch.bfloat16, fuse_float8=fuse)
    with torch.no_grad():
        for p in ff.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    ff = ff.to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe(recipe)).apply_float8_linear(ff)
    return ff


def _selected_ops_context_fn():
    """The reference's policy: save mm (every second one) / abs / max, recompute the rest."""
    meta = defaultdict(int)
    save = {torch.ops.aten.mm.default, torch.ops.aten.abs.default, torch.ops.aten.max.default}

    def policy(ctx, func, *args, **kwargs):
        mode = "recompute" if ctx.is_recompute else "forward"
        if func == torch.ops.aten.mm.default:
            meta[f"{mode}_mm_count"] += 1
        to_save = func in save and not (func == torch.ops.aten.mm.default and meta[f"{mode}_mm_count"] % 2 == 0)
        return CheckpointPolicy.MUST_SAVE if to_save else CheckpointPolicy.PREFER_RECOMPUTE

    return create_selective_checkpoint_contexts(policy)


def _run(ff, x, go, wrap):
    for p in ff.parameters():
        p.grad = None
    xd = x.clone().requires_grad_(True)
    y = wrap(ff, xd)
    y.backward(go)
    return [y.detach().clone(), xd.grad.clone()] + [p.grad.clone() for p in ff.parameters()]


@pytest.mark.parametrize("recipe", ["tensorwise", "rowwise"])
@pytest.mark.parametrize("fuse", [True, False], ids=["fused", "per-linear"])
def test_checkpointed_block_reruns_bit_identically(dev, recipe, fuse):
    ff = _block(dev, recipe, fuse)
    x = seeded((3, 200, 512), 1).to(dev)  # (batch, seq, d_model)
    go = seeded((3, 200, 512), 2, std=1e-3).to(dev)
    plain = _run(ff, x, go, lambda m, t: m(t))
    full = _run(ff, x, go, lambda m, t: checkpoint(m, t, use_reentrant=False))
    selected = _run(ff, x, go, lambda m, t: checkpoint(m, t, use_reentrant=False, context_fn=_selected_ops_context_fn))
    names = ["y", "grad_x"] + [n for n, _ in ff.named_parameters()]
    for name, a, b, c in zip(names, plain, full, selected):
        assert torch.equal(a, b), f"{name}: full re-run differs from the plain call"
        assert torch.equal(a, c), f"{name}: selected-ops re-run differs from the plain call"

"""SwiGLU feed-forward block with float8 projections: fused function vs module-by-module path (identical
bits), both vs the oracle's composition (tolerance), and the fused amax against a separate pass."""

import pytest
import torch

from helpers import E4M3, E5M2, assert_gemm_close, assert_scale_equal, gemm_errors, seeded
from oracle import float8_oracle as O

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import AOFloat8LinearRecipe, Float8Config  # noqa: E402
from olmo_core_amd.float8 import ops  # noqa: E402
from olmo_core_amd.nn import FeedForward  # noqa: E402


def _make(dev, D, H, fuse, recipe="tensorwise", seed=0):
    g = torch.Generator().manual_seed(seed)
    ff = FeedForward(d_model=D, hidden_size=H, bias=False, dtype=torch.bfloat16, fuse_float8=fuse)
    with torch.no_grad():
        for p in ff.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    ff = ff.to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe(recipe)).apply_float8_linear(ff)
    return ff


def _run(ff, x, go):
    xd = x.clone().requires_grad_(True)
    y = ff(xd)
    y.backward(go)
    return y, xd.grad, ff.w1.weight.grad, ff.w2.weight.grad, ff.w3.weight.grad


@pytest.mark.parametrize("mdh", [(512, 256, 768), (300, 272, 528), (2048, 1024, 2816)], ids=lambda s: "x".join(map(str, s)))
def test_fused_equals_unfused_bitwise(dev, mdh):
    M, D, H = mdh
    x = seeded((M, D), 1).to(dev)
    go = seeded((M, D), 2, std=1e-3).to(dev)
    a = _run(_make(dev, D, H, fuse=True), x, go)
    b = _run(_make(dev, D, H, fuse=False), x, go)
    for name, u, v in zip(("y", "gx", "gw1", "gw2", "gw3"), a, b):
        assert torch.equal(u, v), f"{name}: fused and module-by-module results differ"


@pytest.mark.parametrize("recipe", ["tensorwise", "rowwise"])
def test_mlp_against_oracle(dev, recipe):
    M, D, H = 640, 512, 1280
    x, go = seeded((M, D), 1), seeded((M, D), 2, std=1e-3)
    ff = _make(dev, D, H, fuse=True, recipe=recipe, seed=3)
    w1, w2, w3 = (ff.w1.weight.detach().cpu(), ff.w2.weight.detach().cpu(), ff.w3.weight.detach().cpu())
    ref = O.mlp_fwd_bwd(x, w1, w2, w3, go, O.recipe(recipe))
    y, gx, gw1, gw2, gw3 = _run(ff, x.to(dev), go.to(dev))
    assert_gemm_close(y, ref.y, "y")
    # The 1e-2 / 0.9999 bar is for one GEMM on identical operands.  The gradients are compositions:
    # the device's bf16 intermediates (h, the gate gradients) differ from the host's in the last bf16 ulp on a
    # few elements (different exp), and a re-quantisation to e5m2 (2 mantissa bits) can turn such an ulp into
    # one fp8 step.  The cosine bar is kept, the max-error bar is doubled for the compositions.
    for name, got, want in (("grad_x", gx, ref.grad_x), ("grad_w1", gw1, ref.grad_w1), ("grad_w2", gw2, ref.grad_w2),
                            ("grad_w3", gw3, ref.grad_w3)):
        rel, cos = gemm_errors(got, want)
        assert rel <= 2e-2 and cos >= 0.9999, (name, rel, cos)


def test_swiglu_kernels_and_fused_amax(dev):
    x1, x3, gh = seeded((333, 528), 1).to(dev), seeded((333, 528), 2).to(dev), seeded((333, 528), 3, std=1e-3).to(dev)
    h, slots = ops.swiglu_fwd(x1, x3)
    ref = O.swiglu(x1.cpu(), x3.cpu())
    # the device exp differs from the host's in the last ulp: at most a bf16 ulp on a few elements
    assert (h.cpu().float() - ref.float()).abs().max() <= 2 ** -7 * ref.float().abs().max()
    assert float((h.cpu() != ref).float().mean()) < 1e-2
    got = slots[0][: slots[1]].view(torch.float32).max()
    assert float(got) == float(h.abs().max().float())
    g1, g3, s1, s3 = ops.swiglu_bwd(x1, x3, gh)
    r1, r3 = O.swiglu_backward(x1.cpu(), x3.cpu(), gh.cpu())
    for got_t, ref_t in ((g1, r1), (g3, r3)):
        assert (got_t.cpu().float() - ref_t.float()).abs().max() <= 2 ** -6 * ref_t.float().abs().max()
    assert float(s1[0][: s1[1]].view(torch.float32).max()) == float(g1.abs().max().float())
    assert float(s3[0][: s3[1]].view(torch.float32).max()) == float(g3.abs().max().float())
    # a cast fed by the fused amax equals a cast that takes its own amax
    q_a, _, s_a = ops.cast_tensorwise(h, E4M3, slots=slots)
    q_b, _, s_b = ops.cast_tensorwise(h, E4M3)
    assert torch.equal(q_a.view(torch.uint8), q_b.view(torch.uint8))
    assert_scale_equal(s_a, s_b)


@pytest.mark.parametrize("shape", [(333, 528), (128, 128), (1, 16), (1000, 2064)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("layouts", [(True, True), (True, False), (False, True)], ids=["both", "rows", "transposed"])
@pytest.mark.parametrize("fp8", [E5M2, E4M3], ids=["e5m2", "e4m3"])
def test_swiglu_backward_cast_equals_two_steps(dev, shape, layouts, fp8):
    """The recompute-and-cast route writes the bytes and scales of swiglu_bwd followed by cast_tensorwise on each
    gradient, in both layouts, including the zero padding of the transposed copies."""
    x1, x3, gh = seeded(shape, 11).to(dev), seeded(shape, 12).to(dev), seeded(shape, 13, std=1e-3).to(dev)
    rowmajor, transposed = layouts
    g1, g3, s1, s3 = ops.swiglu_bwd(x1, x3, gh)
    want = []
    for g, sl in ((g1, s1), (g3, s3)):
        want.append(ops.cast_tensorwise(g, fp8, want_rowmajor=rowmajor, want_transposed=transposed, slots=sl))
    q1, q1t, sc1, q3, q3t, sc3 = ops.swiglu_bwd_cast(x1, x3, gh, fp8, want_rowmajor=rowmajor, want_transposed=transposed)
    for (wq, wqt, ws), (q, qt, sc) in zip(want, ((q1, q1t, sc1), (q3, q3t, sc3))):
        assert_scale_equal(sc, ws)
        if rowmajor:
            assert torch.equal(q.view(torch.uint8), wq.view(torch.uint8))
        else:
            assert q is None
        if transposed:
            assert torch.equal(qt.view(torch.uint8), wqt.view(torch.uint8))
        else:
            assert qt is None


@pytest.mark.parametrize("mdh", [(640, 512, 1280), (1024, 768, 2048)], ids=lambda s: "x".join(map(str, s)))
def test_mlp_stage_by_stage_against_oracle(dev, mdh):
    """Every stage of the fused block against the oracle of THAT stage fed with the device's own bf16 input of the
    stage (stage_checks.check_mlp_stages): GEMM stages at the single-GEMM bar (1e-2 / 0.9999), casts bit-exact,
    SwiGLU stages within bf16 steps on < 1-2 % of the elements.  The end-to-end comparison in
    test_mlp_against_oracle is then a secondary check."""
    from stage_checks import check_mlp_stages

    M, D, H = mdh
    x, go = seeded((M, D), 1), seeded((M, D), 2, std=1e-3)
    check_mlp_stages(dev, _make(dev, D, H, fuse=True, seed=3), x, go)


@pytest.mark.parametrize("mhk", [(256, 128, 128), (512, 256, 256), (300, 272, 384), (1024, 1416, 512), (2560, 2816, 1024),
                                 (4100, 1672, 256)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("a_fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
def test_swiglu_fused_into_the_projection_gemm(dev, mhk, a_fp8):
    """x1, x3, h and the amax of h from the one-launch route are the bits of gemm_fp8 twice + swiglu_fwd (token and
    hidden sizes that are not multiples of the tile included: the shifted-back edge tiles rewrite identical values)."""
    M, H, K = mhk
    x, w1, w3 = seeded((M, K), 61), seeded((H, K), 62, std=0.05), seeded((H, K), 63, std=0.02)
    xq, _, sx = ops.cast_tensorwise(x.to(dev), a_fp8)
    w1q, _, s1 = ops.cast_tensorwise(w1.to(dev), E4M3)
    w3q, _, s3 = ops.cast_tensorwise(w3.to(dev), E4M3)
    assert ops.swiglu_gemm_supported(M, H, K)
    x1, x3, h, (slots, n) = ops.gemm_fp8_swiglu(xq, sx, w1q, s1, w3q, s3)
    # the projections: bit-identical to the persistent tile kernel (the library's choice for large problems; forced
    # here where the library would pick another tile kernel, which sums in another order)
    m16 = ops.gemm_variants().index("256x256_dma_w4x128_m16x128")
    same_kernel = ops.swiglu_gemm_matches_separate(M, H, K)
    assert same_kernel == (-(-M // 256) * -(-H // 256) > 96 and H >= 256)
    kw = {} if same_kernel else ({"variant": m16} if H >= 256 else None)
    if kw is not None:
        assert torch.equal(x1, ops.gemm_fp8(xq, sx, w1q, s1, **kw)), "x1"
        assert torch.equal(x3, ops.gemm_fp8(xq, sx, w3q, s3, **kw)), "x3"
    # h and its amax: the bits of the pointwise kernel on these x1, x3
    rh, (rslots, rn) = ops.swiglu_fwd(x1, x3)
    assert torch.equal(h.view(torch.int16), rh.view(torch.int16)), "h"
    assert 0 < n <= 1024
    got = slots[:n].view(torch.float32).max()
    assert float(got) == float(rh.abs().max().float()) == float(rslots[:rn].view(torch.float32).max())
    assert_gemm_close(x3, O.emulated_mm_f32(xq.cpu(), sx.cpu()[0], w3q.cpu().t(), s3.cpu()[0]), "x3 vs oracle")
    # and against the oracle of each stage
    assert_gemm_close(x1, O.emulated_mm_f32(xq.cpu(), sx.cpu()[0], w1q.cpu().t(), s1.cpu()[0]), "x1 vs oracle")
    from helpers import assert_bf16_pointwise_close
    assert_bf16_pointwise_close(h, O.swiglu(x1.cpu(), x3.cpu()), "h vs oracle")


def test_fused_swiglu_epilogue_switch_gives_identical_block_results(dev):
    from olmo_core_amd.nn import feed_forward as ff_mod

    M, D, H = 4096, 512, 1792  # 16 x 7 tiles: the library runs the separate projections on the persistent kernel too
    assert ops.swiglu_gemm_matches_separate(M, H, D)
    x, go = seeded((M, D), 1).to(dev), seeded((M, D), 2, std=1e-3).to(dev)
    res = []
    for flag in (True, False):
        ff_mod.FUSE_SWIGLU_EPILOGUE = flag
        try:
            res.append(_run(_make(dev, D, H, fuse=True), x, go))
        finally:
            ff_mod.FUSE_SWIGLU_EPILOGUE = True
    for name, u, v in zip(("y", "gx", "gw1", "gw2", "gw3"), *res):
        assert torch.equal(u, v), name


@pytest.mark.parametrize("mdh", [(4096, 512, 1792), (512, 256, 768)], ids=["fused_launch", "separate_launches"])
def test_compiled_block_keeps_the_fused_function(dev, mdh):
    """torch.compile(fullgraph=True) over a converted FeedForward (the reference compiles every transformer block,
    src/olmo_core/nn/transformer/block.py:78-79): one graph, the block is one registered operator, and output and all
    four gradients carry the bits of the eager fused block - the same launches run."""
    from olmo_core_amd.nn import feed_forward as ff_mod

    M, D, H = mdh
    x = seeded((4, M // 4, D), 1).to(dev)
    go = seeded((4, M // 4, D), 2, std=1e-3).to(dev)
    ff = _make(dev, D, H, fuse=True)
    ff.w3.weight.requires_grad_(False)  # a frozen projection: no gradient for it, no transposed copy of g3

    def run(fn):
        ff.zero_grad()
        xd = x.clone().requires_grad_(True)
        ff_mod.STAGE_SINK = sink = {}
        try:
            y = fn(xd)
            y.backward(go)
        finally:
            ff_mod.STAGE_SINK = None
        return sink, (y, xd.grad, ff.w1.weight.grad.clone(), ff.w2.weight.grad.clone())

    sink0, eager = run(ff)
    compiled = torch.compile(ff, fullgraph=True)
    sink1, traced = run(compiled)
    assert "sh" in sink0 and "sh" in sink1 and "sg1" in sink1, "the fused function did not run inside the graph"
    assert ff.w3.weight.grad is None
    for name, a, b in zip(("y", "gx", "gw1", "gw2"), traced, eager):
        assert torch.equal(a, b), f"{name}: the compiled block differs from the eager fused block"
    with torch.no_grad():
        assert torch.equal(compiled(x), ff(x))
    # a block that cannot run fused (a bias) still traces into one graph, through the per-linear operators
    plain = FeedForward(d_model=D, hidden_size=H, bias=True, dtype=torch.bfloat16).to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(plain)
    y = torch.compile(plain, fullgraph=True)(x)
    assert y.shape == x.shape


@pytest.mark.parametrize("param_dtype", [torch.float32, torch.bfloat16], ids=["fp32_params", "bf16_params"])
def test_fused_block_under_autocast(dev, param_dtype):
    """The model runs under torch.autocast when autocast_precision is set
    (src/olmo_core/train/train_module/transformer/train_module.py:593-597): the block casts its input to the autocast
    type, as each Float8Linear does, stays fused, and gives the bits of the three modules one by one."""
    from olmo_core_amd.nn import feed_forward as ff_mod

    M, D, H = 2048, 512, 1792
    g = torch.Generator().manual_seed(5)
    blocks = []
    for fuse in (True, False):
        ff = FeedForward(d_model=D, hidden_size=H, bias=False, dtype=param_dtype, fuse_float8=fuse)
        gg = torch.Generator().manual_seed(6)
        with torch.no_grad():
            for p in ff.parameters():
                p.copy_((torch.randn(p.shape, generator=gg) * 0.02).to(param_dtype))
        ff = ff.to(dev)
        Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(ff)
        blocks.append(ff)
    x = torch.randn(M, D, generator=g).to(dev)  # float32 activations, as a norm under autocast produces
    go = (torch.randn(M, D, generator=g) * 1e-3).bfloat16().to(dev)
    results = []
    for ff in blocks:
        xd = x.clone().requires_grad_(True)
        ff_mod.STAGE_SINK = sink = {}
        try:
            with torch.autocast("cuda", dtype=torch.bfloat16):
                y = ff(xd)
            y.backward(go)
        finally:
            ff_mod.STAGE_SINK = None
        results.append((sink, (y, xd.grad, ff.w1.weight.grad, ff.w2.weight.grad, ff.w3.weight.grad)))
    assert "sh" in results[0][0] and not results[1][0], "fused block under autocast / module-by-module reference"
    assert results[0][1][0].dtype == torch.bfloat16 and results[0][1][1].dtype == torch.float32
    assert results[0][1][2].dtype == param_dtype
    for name, a, b in zip(("y", "gx", "gw1", "gw2", "gw3"), results[0][1], results[1][1]):
        assert a.dtype == b.dtype and torch.equal(a, b), f"{name}: fused and module-by-module results differ under autocast"


def test_compiled_modules_use_their_kept_weights(dev, monkeypatch):
    """AOFloat8LinearConfig.recommended() (what every production script sets, src/olmo_core/float8/ao.py:173-180) under
    torch.compile: the registered operators ask their modules for the float8 weight copies kept since the last weight
    update, so the micro-batches of a step quantise each weight once - in a compiled block as in an eager one - and the
    results are the bits of the eager modules."""
    import torch.nn as nn

    from olmo_core_amd.float8 import AOFloat8LinearConfig

    D, H, M = 512, 1792, 4096
    torch.manual_seed(3)
    model = nn.ModuleDict({"ff": FeedForward(d_model=D, hidden_size=H, bias=False, dtype=torch.bfloat16),
                           "proj": nn.Linear(D, 256, bias=True, dtype=torch.bfloat16)}).to(dev)
    Float8Config(ao=AOFloat8LinearConfig.recommended()).apply_float8_linear(model)
    weight_shapes = {(H, D), (D, H), (256, D)}
    casts = []
    orig = ops.cast_tensorwise

    def counted(t, *a, **k):
        if tuple(t.shape) in weight_shapes:
            casts.append(tuple(t.shape))
        return orig(t, *a, **k)

    monkeypatch.setattr(ops, "cast_tensorwise", counted)

    def fwd(m, x):
        return m["proj"](m["ff"](x))

    compiled = torch.compile(lambda x: fwd(model, x), fullgraph=True)
    xs = [seeded((M, D), 20 + i).to(dev) for i in range(3)]
    go = seeded((M, 256), 30, std=1e-3).to(dev)
    outs = []
    for x in xs:
        xd = x.clone().requires_grad_(True)
        y = compiled(xd)
        y.backward(go)
        outs.append((y, xd.grad))
    assert len(casts) == 4, casts  # w1, w2, w3 and the projection, once each for the three micro-batches
    model.zero_grad()
    for x, (y1, g1) in zip(xs, outs):
        xd = x.clone().requires_grad_(True)
        y0 = fwd(model, xd)
        y0.backward(go)
        assert torch.equal(y0, y1) and torch.equal(xd.grad, g1)
    assert len(casts) == 4
    with torch.no_grad():  # a weight update is seen: the copies are made again
        for p in model.parameters():
            p.mul_(1.5)
    y = compiled(xs[0])
    assert len(casts) == 8 and torch.equal(y, fwd(model, xs[0]))

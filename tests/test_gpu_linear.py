"""Float8Linear forward/backward on the GPU against the oracle's restated autograd function:
operands (bytes + scales) bit-exact, outputs and gradients within the GEMM tolerance."""

import pytest
import torch
import torch.nn as nn

from helpers import E4M3, E5M2, assert_bytes_equal, assert_gemm_close, assert_scale_equal, seeded
from oracle import float8_oracle as O

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import AOFloat8LinearConfig, AOFloat8LinearRecipe, Float8Config  # noqa: E402
from olmo_core_amd.float8 import ops  # noqa: E402
from olmo_core_amd.float8.linear import Float8Linear, convert_to_float8_training  # noqa: E402
from olmo_core_amd.float8.native_config import Float8LinearConfig  # noqa: E402

RECIPES = ["tensorwise", "rowwise", "rowwise_with_gw_hp"]


def _run_linear(dev, recipe, M, K, N, bias, seed, go_std=1e-3):
    x = seeded((M, K), seed)
    w = seeded((N, K), seed + 1, std=0.02)
    b = seeded((N,), seed + 2, std=0.1) if bias else None
    go = seeded((M, N), seed + 3, std=go_std)
    ref = O.linear_fwd_bwd(x, w, b, go, O.recipe(recipe))

    lin = nn.Linear(K, N, bias=bias, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
        if bias:
            lin.bias.copy_(b)
    lin = lin.to(dev)
    f8 = Float8Linear.from_float(lin, Float8LinearConfig.from_recipe_name(recipe))
    xd = x.to(dev).requires_grad_(True)
    y = f8(xd)
    y.backward(go.to(dev))
    return ref, y, xd.grad, f8.weight.grad, (f8.bias.grad if bias else None)


@pytest.mark.parametrize("recipe", RECIPES)
@pytest.mark.parametrize("mkn", [(256, 256, 512), (300, 144, 272), (2048, 4096, 1024), (17, 16, 32)], ids=lambda s: "x".join(map(str, s)))
def test_linear_fwd_bwd(dev, recipe, mkn):
    M, K, N = mkn
    ref, y, gx, gw, gb = _run_linear(dev, recipe, M, K, N, bias=True, seed=M + N)
    assert y.dtype == torch.bfloat16 and y.shape == (M, N)
    assert_gemm_close(y, ref.out, f"{recipe} out")
    assert_gemm_close(gx, ref.grad_input, f"{recipe} grad_input")
    assert_gemm_close(gw, ref.grad_weight, f"{recipe} grad_weight")
    assert_gemm_close(gb, ref.grad_bias, f"{recipe} grad_bias")


def test_config1_forward(dev):
    """x bf16 [2048,4096] ~N(0,1), W bf16 [11008,4096] ~N(0,0.02), no bias, e4m3, tensorwise, seed 0."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2048, 4096, generator=g).bfloat16()
    w = (torch.randn(11008, 4096, generator=g) * 0.02).bfloat16()
    spec = O.recipe("tensorwise")
    ref = O.linear_forward(x, w, None, spec)
    xq, _, sx = ops.cast_tensorwise(x.to(dev), E4M3)
    wq, _, sw = ops.cast_tensorwise(w.to(dev), E4M3)
    assert_bytes_equal(xq, ref.operands["input"][0], "x bytes")
    assert_scale_equal(sx, ref.operands["input"][1], "x scale")
    assert_bytes_equal(wq, ref.operands["weight"][0].t(), "W bytes")
    assert_scale_equal(sw, ref.operands["weight"][1], "W scale")
    lin = nn.Linear(4096, 11008, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    f8 = Float8Linear.from_float(lin.to(dev), Float8LinearConfig())
    with torch.no_grad():
        y = f8(x.to(dev))
    assert_gemm_close(y, ref.out, "config 1 output")


@pytest.mark.parametrize("recipe", ["tensorwise", "rowwise"])
def test_operands_bit_exact(dev, recipe):
    """Every cast on the path (six for the rowwise recipe) reproduces the oracle's bytes and scales."""
    M, K, N = 384, 272, 528
    x, w, go = seeded((M, K), 1), seeded((N, K), 2, std=0.02), seeded((M, N), 3, std=1e-3)
    spec = O.recipe(recipe)
    ref = O.linear_fwd_bwd(x, w, None, go, spec).operands
    pow2 = spec.round_scales_to_power_of_2
    xd, wd, god = x.to(dev), w.to(dev), go.to(dev)
    if recipe == "tensorwise":
        xq, xq_t, sx = ops.cast_tensorwise(xd, E4M3, want_transposed=True)
        wq, wq_t, sw = ops.cast_tensorwise(wd, E4M3, want_transposed=True)
        gq, gq_t, sg = ops.cast_tensorwise(god, E5M2, want_transposed=True)
        assert_bytes_equal(xq, ref["input"][0]); assert_scale_equal(sx, ref["input"][1])
        assert_bytes_equal(wq, ref["weight"][0].t()); assert_scale_equal(sw, ref["weight"][1])
        assert_bytes_equal(gq, ref["grad_output"][0]); assert_scale_equal(sg, ref["grad_output"][1])
        assert_bytes_equal(wq_t[:, :N], ref["weight_for_grad_input"][0])
        assert_bytes_equal(gq_t[:, :M], ref["grad_output_for_grad_weight"][0].t())
        assert_bytes_equal(xq_t[:, :M], ref["input_for_grad_weight"][0].t())
    else:
        q, s = ops.cast_rowwise(xd, E4M3, pow2=pow2)
        assert_bytes_equal(q, ref["input"][0]); assert_scale_equal(s, ref["input"][1])
        q, s = ops.cast_rowwise(wd, E4M3, pow2=pow2)  # per output channel
        assert_bytes_equal(q, ref["weight"][0].t()); assert_scale_equal(s, ref["weight"][1])
        q, s = ops.cast_rowwise(god, E4M3, pow2=pow2)
        assert_bytes_equal(q, ref["grad_output"][0]); assert_scale_equal(s, ref["grad_output"][1])
        q_t, s = ops.cast_colwise_t(wd, E4M3, pow2=pow2)  # per input channel, [K, N]
        assert_bytes_equal(q_t[:, :N], ref["weight_for_grad_input"][0]); assert_scale_equal(s, ref["weight_for_grad_input"][1])
        q_t, s = ops.cast_colwise_t(god, E4M3, pow2=pow2)  # [N, M]
        assert_bytes_equal(q_t[:, :M], ref["grad_output_for_grad_weight"][0].t()); assert_scale_equal(s, ref["grad_output_for_grad_weight"][1])
        q_t, s = ops.cast_colwise_t(xd, E4M3, pow2=pow2)  # [K, M]
        assert_bytes_equal(q_t[:, :M], ref["input_for_grad_weight"][0].t()); assert_scale_equal(s, ref["input_for_grad_weight"][1])


def test_gradients_against_bf16_autograd(dev):
    """Independent of the oracle: float8 gradients track plain bf16 autograd of F.linear."""
    M, K, N = 512, 1024, 768
    x, w, go = seeded((M, K), 1), seeded((N, K), 2, std=0.02), seeded((M, N), 3, std=1e-3)
    xr = x.float().requires_grad_(True); wr = w.float().requires_grad_(True)
    (xr @ wr.t()).backward(go.float())
    for recipe in RECIPES:
        _, y, gx, gw, _ = _run_linear(dev, recipe, M, K, N, bias=False, seed=0)
    lin = nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    for recipe in RECIPES:
        f8 = Float8Linear.from_float(lin.to(dev), Float8LinearConfig.from_recipe_name(recipe))
        f8.weight.grad = None
        xd = x.to(dev).requires_grad_(True)
        f8(xd).backward(go.to(dev))
        for got, want in ((xd.grad, xr.grad), (f8.weight.grad, wr.grad)):
            g, r = got.float().cpu().reshape(-1), want.reshape(-1)
            cos = float(torch.dot(g, r) / (g.norm() * r.norm()))
            assert cos > 0.995, (recipe, cos)


def test_module_contract(dev):
    """Leading dims, frozen weight, autocast, float32 parameters, state dict keys."""
    lin = nn.Linear(64, 128, bias=True).to(dev)  # float32 parameters
    f8 = convert_to_float8_training(nn.Sequential(lin), config=Float8LinearConfig())[0]
    assert isinstance(f8, Float8Linear) and isinstance(f8, nn.Linear)
    assert f8.weight is lin.weight and f8.bias is lin.bias
    assert set(f8.state_dict().keys()) == {"weight", "bias"}
    x = torch.randn(2, 3, 5, 64, device=dev)
    with torch.autocast("cuda", dtype=torch.bfloat16):
        y = f8(x)
    assert y.shape == (2, 3, 5, 128) and y.dtype == torch.bfloat16
    y.float().sum().backward()
    assert f8.weight.grad is not None and f8.weight.grad.dtype == torch.float32
    # float32 activations without autocast: float32 output
    y32 = f8(x)
    assert y32.dtype == torch.float32
    ref = torch.nn.functional.linear(x, lin.weight, lin.bias)
    cos = torch.nn.functional.cosine_similarity(y32.detach().reshape(-1), ref.detach().reshape(-1), dim=0)
    assert float(cos) > 0.995
    # frozen weight: no weight gradient is computed, input gradient still flows
    f8.weight.requires_grad_(False)
    f8.weight.grad = None
    xg = torch.randn(8, 64, device=dev, dtype=torch.bfloat16, requires_grad=True)
    f8(xg).float().sum().backward()
    assert xg.grad is not None and f8.weight.grad is None


def test_apply_float8_linear_on_gpu_model(dev):
    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.w1 = nn.Linear(64, 256, bias=False)
            self.w3 = nn.Linear(64, 256, bias=False)
            self.w2 = nn.Linear(256, 64, bias=False)
            self.odd = nn.Linear(64, 10, bias=False)  # 10 % 16 != 0: stays nn.Linear

        def forward(self, x):
            return self.odd(self.w2(torch.nn.functional.silu(self.w1(x)) * self.w3(x)))

    m = Block().to(dev).bfloat16()
    Float8Config(ao_recipe=AOFloat8LinearRecipe.rowwise).apply_float8_linear(m)
    assert isinstance(m.w1, Float8Linear) and isinstance(m.w2, Float8Linear) and not isinstance(m.odd, Float8Linear)
    x = torch.randn(4, 32, 64, device=dev, dtype=torch.bfloat16)
    m(x).float().sum().backward()
    assert all(p.grad is not None for p in m.parameters())


@pytest.mark.parametrize("recipe", [None, "rowwise"], ids=["tensorwise", "rowwise"])
def test_torch_compile_composes(dev, recipe):
    """A block with converted linears compiles into ONE graph (fullgraph: the float8 linear is a registered
    operator with a shape function, not a graph break) and reproduces eager."""
    import torch.nn as nn

    from olmo_core_amd.float8 import Float8Config

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.norm = nn.LayerNorm(256)
            self.w1 = nn.Linear(256, 512, bias=False)
            self.w2 = nn.Linear(512, 256, bias=True)
            self.frozen = nn.Linear(256, 256, bias=False)
            self.frozen.weight.requires_grad_(False)

        def forward(self, x):
            return x + self.frozen(self.w2(torch.nn.functional.silu(self.w1(self.norm(x)))))

    torch.manual_seed(0)
    m = Block().to(dev).bfloat16()
    cfg = Float8Config(enabled=True) if recipe is None else Float8Config(ao_recipe=AOFloat8LinearRecipe(recipe), enabled=True)
    cfg.apply_float8_linear(m)
    x = torch.randn(64, 256, device=dev, dtype=torch.bfloat16, requires_grad=True)
    y0 = m(x)
    y0.float().sum().backward()
    g0, gw0 = x.grad.clone(), m.w1.weight.grad.clone()
    x.grad = None
    m.zero_grad()
    mc = torch.compile(m, fullgraph=True)
    y1 = mc(x)
    y1.float().sum().backward()
    # inductor fuses the bf16 pointwise parts with fewer roundings than eager: close, not identical
    assert torch.allclose(y1.float(), y0.float(), rtol=2e-2, atol=2e-2)
    assert torch.allclose(x.grad.float(), g0.float(), rtol=5e-2, atol=5e-2)
    assert torch.allclose(m.w1.weight.grad.float(), gw0.float(), rtol=5e-2, atol=5e-2)
    assert m.frozen.weight.grad is None
    # inference under no_grad, and a second shape (recompile or dynamic shapes, either way it must run)
    with torch.no_grad():
        y2 = mc(torch.randn(48, 256, device=dev, dtype=torch.bfloat16))
    assert y2.shape == (48, 256)


def test_torch_compile_feed_forward(dev):
    from olmo_core_amd.float8 import Float8Config
    from olmo_core_amd.nn import FeedForward

    torch.manual_seed(0)
    ff = FeedForward(d_model=256, hidden_size=512, bias=False, dtype=torch.bfloat16).to(dev)
    Float8Config(enabled=True).apply_float8_linear(ff)
    x = torch.randn(128, 256, device=dev, dtype=torch.bfloat16, requires_grad=True)
    y0 = ff(x)
    y0.float().sum().backward()
    g0 = x.grad.clone()
    x.grad = None
    y1 = torch.compile(ff, fullgraph=True)(x)
    y1.float().sum().backward()
    assert torch.allclose(y1.float(), y0.float(), rtol=3e-2, atol=3e-2)
    assert torch.allclose(x.grad.float(), g0.float(), rtol=5e-2, atol=5e-2)


def test_precomputed_weight_scales(dev):
    """precompute_float8_dynamic_scale_for_fsdp (reference: model.post_optim_step,
    src/olmo_core/nn/transformer/model.py:1001-1008): one batch of launches gives every weight the scale its
    forward would compute, forwards with it are bit-identical, and a scale goes stale with the weight."""
    import torch.nn as nn

    from olmo_core_amd.float8 import Float8Config, precompute_float8_dynamic_scale_for_fsdp
    from olmo_core_amd.float8.linear import Float8Linear
    from olmo_core_amd.nn import FeedForward

    torch.manual_seed(1)
    model = nn.ModuleDict(
        {
            "ff": FeedForward(d_model=256, hidden_size=512, bias=False, dtype=torch.bfloat16),
            "proj": nn.Linear(256, 128, bias=True, dtype=torch.float32),
            "odd": nn.Linear(256, 24, bias=False, dtype=torch.bfloat16),  # 24 % 16 != 0: left unconverted
        }
    ).to(dev)
    with torch.no_grad():
        model["proj"].weight.mul_(37.0)
    Float8Config(enabled=True).apply_float8_linear(model)
    lins = [m for m in model.modules() if isinstance(m, Float8Linear)]
    assert len(lins) == 4
    x = torch.randn(192, 256, device=dev, dtype=torch.bfloat16)
    before = (model["ff"](x), model["proj"](x.float()))
    precompute_float8_dynamic_scale_for_fsdp(model)
    for m in lins:
        s = m.precomputed_weight_scale()
        assert s is not None and s.shape == (1,)
        ref = ops.tensor_to_scale(m.weight.detach(), torch.float8_e4m3fn)
        assert_scale_equal(s, ref.reshape(1), "precomputed weight scale")
    after = (model["ff"](x), model["proj"](x.float()))
    assert torch.equal(before[0], after[0]) and torch.equal(before[1], after[1])
    # gradients flow as before
    xg = x.clone().requires_grad_(True)
    model["ff"](xg).float().sum().backward()
    assert xg.grad is not None and model["ff"].w1.weight.grad is not None
    # an optimizer step (any in-place update) invalidates the stored scale of that weight
    with torch.no_grad():
        model["proj"].weight.mul_(0.5)
    assert model["proj"].precomputed_weight_scale() is None
    assert model["ff"].w1.precomputed_weight_scale() is not None
    out = model["proj"](x.float())
    precompute_float8_dynamic_scale_for_fsdp(model)
    assert torch.equal(out, model["proj"](x.float()))


def test_kept_weight_operands(dev, monkeypatch):
    """With enable_fsdp_float8_all_gather (what AOFloat8LinearConfig.recommended() sets,
    src/olmo_core/float8/ao.py:173-180) a module quantises its weight once per weight update, not once per
    forward: the micro-batches of a step reuse the float8 copies, results stay bit-identical to a module that
    quantises every time, and an in-place update of the weight makes the next forward quantise it again."""
    import copy

    import torch.nn as nn

    from olmo_core_amd.float8 import AOFloat8LinearConfig, Float8Config, precompute_float8_dynamic_scale_for_fsdp
    from olmo_core_amd.float8.linear import Float8Linear
    from olmo_core_amd.nn import FeedForward

    torch.manual_seed(3)
    base = nn.ModuleDict(
        {
            "ff": FeedForward(d_model=256, hidden_size=512, bias=False, dtype=torch.bfloat16),
            "proj": nn.Linear(256, 384, bias=True, dtype=torch.bfloat16),
        }
    ).to(dev)
    plain, kept = copy.deepcopy(base), copy.deepcopy(base)
    Float8Config(ao=AOFloat8LinearConfig(round_scales_to_power_of_2=True)).apply_float8_linear(plain)
    Float8Config(ao=AOFloat8LinearConfig.recommended()).apply_float8_linear(kept)
    assert all(m.weight_operands() is None for m in plain.modules() if isinstance(m, Float8Linear))

    weight_ptrs = {m.weight.data_ptr() for m in kept.modules() if isinstance(m, Float8Linear)}
    casts = []
    real_cast = ops.cast_tensorwise

    def counting_cast(x, *a, **k):
        if x.data_ptr() in weight_ptrs:
            casts.append(x.data_ptr())
        return real_cast(x, *a, **k)

    monkeypatch.setattr(ops, "cast_tensorwise", counting_cast)

    def step(model, x):
        xg = x.clone().requires_grad_(True)
        y = model["proj"](model["ff"](xg))
        y.backward(torch.ones_like(y) * 1e-3)
        return y.detach(), xg.grad

    xs = [torch.randn(192, 256, device=dev, dtype=torch.bfloat16) for _ in range(3)]
    for i, x in enumerate(xs):  # three micro-batches, gradients accumulate
        y0, g0 = step(plain, x)
        y1, g1 = step(kept, x)
        assert torch.equal(y0, y1) and torch.equal(g0, g1), i
        assert len(casts) == 4, (i, len(casts))  # w1, w2, w3, proj: once each, in the first micro-batch only
    for (n0, p0), (n1, p1) in zip(plain.named_parameters(), kept.named_parameters()):
        assert n0 == n1 and torch.equal(p0.grad, p1.grad), n0

    # optimizer step: every weight changes in place; the next forward quantises again (and only once)
    with torch.no_grad():
        for model in (plain, kept):
            for p in model.parameters():
                p.add_(p.grad, alpha=-0.5)
                p.grad = None
    precompute_float8_dynamic_scale_for_fsdp(kept)
    for x in xs[:2]:
        y0, g0 = step(plain, x)
        y1, g1 = step(kept, x)
        assert torch.equal(y0, y1) and torch.equal(g0, g1)
    assert len(casts) == 8

    # generation-style use: no gradients, frozen weights, nothing is quantised again
    with torch.no_grad():
        for x in xs:
            assert torch.equal(kept["proj"](kept["ff"](x)), plain["proj"](plain["ff"](x)))
    assert len(casts) == 8



def _projection_modules(dev, recipe, K, ns, bias_on=()):
    mods = []
    for i, N in enumerate(ns):
        lin = nn.Linear(K, N, bias=i in bias_on, dtype=torch.bfloat16)
        with torch.no_grad():
            lin.weight.copy_(seeded((N, K), 40 + i, std=0.02))
            if lin.bias is not None:
                lin.bias.copy_(seeded((N,), 60 + i, std=0.1))
        mods.append(Float8Linear.from_float(lin.to(dev), Float8LinearConfig.from_recipe_name(recipe)))
    return mods


@pytest.mark.parametrize("recipe", RECIPES)
@pytest.mark.parametrize("shape", [(384, 256, (320, 128, 128)), (1024, 512, (512, 512, 512)), (4096, 1024, (1024, 256, 256))],
                         ids=["small", "tiles", "gqa"])
def test_projections_of_one_input(dev, recipe, shape, monkeypatch):
    """float8_projections(x, w_q, w_k, w_v): the input is quantised once, and outputs, grad_x (summed by the GEMM
    epilogues) and the weight gradients carry the bits of the three modules applied one by one and differentiated in
    one backward call (src/olmo_core/nn/attention/__init__.py:582)."""
    from olmo_core_amd.float8.linear import float8_projections

    M, K, ns = shape
    mods = _projection_modules(dev, recipe, K, ns, bias_on=(1,))
    gos = [seeded((2, M // 2, N), 50 + i, std=1e-3).to(dev) for i, N in enumerate(ns)]
    calls = {"n": 0}
    for name in ("cast_tensorwise", "cast_rows_and_colwise_t", "cast_rowwise"):
        orig = getattr(ops, name)

        def counted(t, *a, _orig=orig, **k):
            if t.shape == (M, K):
                calls["n"] += 1
            return _orig(t, *a, **k)

        monkeypatch.setattr(ops, name, counted)

    def run(fused, used=(0, 1, 2)):
        calls["n"] = 0
        x = seeded((2, M // 2, K), 7).to(dev).requires_grad_(True)
        for m in mods:
            m.weight.grad = None
            if m.bias is not None:
                m.bias.grad = None
        ys = float8_projections(x, *mods) if fused else tuple(m(x) for m in mods)
        n_fwd = calls["n"]
        torch.autograd.backward([ys[i] for i in used], [gos[i] for i in used])
        grads = [None if m.weight.grad is None else m.weight.grad.clone() for m in mods]
        return n_fwd, ys, x.grad, grads, mods[1].bias.grad

    for used in ((0, 1, 2), (0, 2), (1,)):
        n1, ys1, gx1, gw1, gb1 = run(True, used)
        n0, ys0, gx0, gw0, gb0 = run(False, used)
        assert (n1, n0) == (1, 3)
        assert torch.equal(gx1, gx0), used
        for a, b in zip(list(ys1) + gw1 + [gb1], list(ys0) + gw0 + [gb0]):
            assert (a is None and b is None) or torch.equal(a, b), used

    # no gradients: same outputs, one cast; frozen weights: only grad_x
    with torch.no_grad():
        xs = seeded((M, K), 11).to(dev)
        calls["n"] = 0
        outs = float8_projections(xs, *mods)
        assert calls["n"] == 1
        for o, m in zip(outs, mods):
            assert torch.equal(o, m(xs))
    for m in mods:
        m.weight.requires_grad_(False)
    n1, ys1, gx1, gw1, _ = run(True)
    n0, ys0, gx0, gw0, _ = run(False)
    assert torch.equal(gx1, gx0) and all(g is None for g in gw1 + gw0)

    # anything that is not a set of Float8Linear modules of one config is applied module by module
    plain = nn.Linear(K, 64, bias=False, dtype=torch.bfloat16).to(dev)
    outs = float8_projections(xs, mods[0], plain)
    assert torch.equal(outs[0], mods[0](xs)) and torch.equal(outs[1], plain(xs))


@pytest.mark.parametrize("recipe", ["tensorwise", "rowwise"])
def test_projections_under_autocast(dev, recipe):
    """Float32 activations under autocast: every module converts its own input, so autograd adds the three grad_input
    terms after converting each back to float32; float8_projections forms that same sum."""
    from olmo_core_amd.float8.linear import float8_projections

    M, K = 512, 256
    mods = _projection_modules(dev, recipe, K, (256, 128, 128))
    for m in mods:
        m.float()
    gos = [seeded((M, N), 50 + i, std=1e-3).to(dev) for i, N in enumerate((256, 128, 128))]
    out = []
    for fused in (True, False):
        x = seeded((M, K), 7, dtype=torch.float32).to(dev).requires_grad_(True)
        for m in mods:
            m.weight.grad = None
        with torch.autocast("cuda", dtype=torch.bfloat16):
            ys = float8_projections(x, *mods) if fused else tuple(m(x) for m in mods)
        torch.autograd.backward(ys, gos)
        out.append(list(ys) + [x.grad] + [m.weight.grad.clone() for m in mods])
    assert out[0][3].dtype == torch.float32 and out[0][0].dtype == torch.bfloat16 and out[0][4].dtype == torch.float32
    for a, b in zip(*out):
        assert a.dtype == b.dtype and torch.equal(a, b)


@pytest.mark.parametrize("recipe", RECIPES)
def test_forward_under_inference_mode(dev, recipe):
    """Generation runs under torch.inference_mode (src/olmo_core/generate/generation_module/transformer/
    generation_module.py:135,141): inputs are inference tensors without a version counter; modules, projections and
    the feed-forward block give the bits of the no_grad call."""
    from olmo_core_amd.float8.linear import float8_projections
    from olmo_core_amd.nn import FeedForward

    M, K = 320, 256
    mods = _projection_modules(dev, recipe, K, (256, 128, 128))
    ff = FeedForward(d_model=K, hidden_size=512, bias=False, dtype=torch.bfloat16).to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe(recipe)).apply_float8_linear(ff)
    x_plain = seeded((M, K), 3).to(dev)
    with torch.no_grad():
        want = [m(x_plain) for m in mods] + [ff(x_plain)]
    with torch.inference_mode():
        x = seeded((M, K), 3).to(dev)
        assert x.is_inference()
        got = [m(x) for m in mods] + [ff(x)]
        fused = float8_projections(x, *mods)
    for a, b in zip(got, want):
        assert torch.equal(a, b)
    for a, b in zip(fused, want[:3]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("tokens", [16, 300], ids=["few_rows", "split_k"])
def test_forward_replays_from_a_captured_graph(dev, tokens):
    """A generation loop captures one step in a HIP graph and replays it: every launch of the forward (casts,
    SwiGLU, the few-rows / split-K / tiled GEMMs) goes to the capturing stream, nothing synchronises or reads
    back, so each replay on new input equals the eager result bit for bit.  Eager work runs between replays."""
    from olmo_core_amd.nn import FeedForward

    torch.manual_seed(11)
    model = nn.Sequential(
        FeedForward(d_model=1024, hidden_size=2048, bias=False, dtype=torch.bfloat16),
        nn.Linear(1024, 512, bias=True, dtype=torch.bfloat16),
    ).to(dev)
    Float8Config(ao=AOFloat8LinearConfig.recommended()).apply_float8_linear(model)
    x_static = torch.randn(tokens, 1024, device=dev, dtype=torch.bfloat16)
    with torch.no_grad():
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(3):  # first calls configure kernels and fill the kept weight copies
                model(x_static)
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            y_static = model(x_static)
        for i in range(4):
            x_new = torch.randn(tokens, 1024, device=dev, dtype=torch.bfloat16) * (i + 1)
            x_static.copy_(x_new)
            graph.replay()
            torch.cuda.synchronize()
            eager = model(x_new)
            assert torch.equal(y_static, eager), i

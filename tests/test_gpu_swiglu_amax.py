"""amax of the SwiGLU gradients from row-segment codes: the bound the codes imply is valid for every element (every
bf16 pattern of x1), the codes equal a host restatement bit for bit whichever kernel writes them, and the amax found
through them equals the dense pass's on ordinary, heavy-tailed, sparse, tiny and non-finite inputs; the cast that
consumes it writes the same bytes and scales."""

import pytest
import torch

from helpers import E5M2, O, seeded

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import ops  # noqa: E402

M3, M1, BIAS = 24, 44, 127 * 128  # margins of the bounds on log2 |g3|, log2 |g1| (units of 1/128), exponent bias


def _L(t):
    return t.contiguous().view(torch.int16).to(torch.int32) & 0x7FFF


def _dense_amax(x1, x3, gh):
    _, _, (s1, n1), (s3, n3) = ops.swiglu_bwd(x1, x3, gh)
    return int(s1[:n1].max().item()), int(s3[:n3].max().item())


def _host_codes(a, b=None):
    rows, cols = a.shape
    C = -(-cols // 64)
    la = _L(a) if b is None else torch.maximum(_L(a), _L(b))
    p = torch.zeros((rows, C * 64), dtype=torch.int32, device=a.device)
    p[:, :cols] = la
    return p.view(rows, C, 64).amax(dim=2).t().contiguous().reshape(-1).to(torch.int16)


def _amax_via_codes(x1, x3, gh):
    state = ops.swiglu_bwd_amax_from_codes(x1, x3, gh, ops.rowseg_max_codes(gh), ops.rowseg_max_codes(x1, x3))
    return int(state[0].item()), int(state[1].item())


def _inputs(dev, rows, cols, kind, seed=0):
    x1 = seeded((rows, cols), seed + 1).to(dev)
    x3 = seeded((rows, cols), seed + 2).to(dev)
    gh = seeded((rows, cols), seed + 3, std=1e-3).to(dev)
    g = torch.Generator().manual_seed(seed + 9)
    if kind == "outliers":
        mask = (torch.rand((rows, cols), generator=g) < 1e-3).to(dev)
        x1 = torch.where(mask, x1 * 100, x1)
        gh = torch.where((torch.rand((rows, cols), generator=g) < 1e-3).to(dev), gh * 50, gh)
    elif kind == "negative_x1":
        x1 = -x1.abs()
    elif kind == "zero_gh":
        gh = torch.zeros_like(gh)
    elif kind == "mostly_zero_gh":
        keep = torch.zeros((rows, cols), dtype=torch.bool, device=dev)
        keep[rows // 3 : rows // 3 + 5, cols // 2 : cols // 2 + 9] = True
        gh = torch.where(keep, gh, torch.zeros_like(gh))
    elif kind == "tiny":
        x1, x3, gh = x1 * 1e-20, x3 * 1e-18, gh * 1e-15
    elif kind == "huge":
        x1, x3, gh = x1 * 1e18, x3 * 1e19, gh * 1e22  # products overflow bf16
    elif kind == "nan_x1":
        x1[rows // 2, cols // 3] = float("nan")
    elif kind == "inf_x3":
        x3[rows - 1, cols - 1] = float("inf")
    elif kind == "inf_gh_zero_x":
        gh[3, 5] = float("-inf")
        x1[3, 5] = 0.0
        x3[3, 5] = 0.0
    elif kind == "neginf_x1":
        x1[0, 0] = float("-inf")
    return x1.contiguous(), x3.contiguous(), gh.contiguous()


KINDS = ["normal", "outliers", "negative_x1", "zero_gh", "mostly_zero_gh", "tiny", "huge", "nan_x1", "inf_x3",
         "inf_gh_zero_x", "neginf_x1"]


@pytest.mark.parametrize("shape", [(256, 128), (1000, 200), (4096, 1024)], ids=lambda s: "x".join(map(str, s)))
def test_codes_kernel_equals_host_restatement(dev, shape):
    x1, x3, gh = _inputs(dev, *shape, "outliers")
    assert torch.equal(ops.rowseg_max_codes(gh), _host_codes(gh))
    assert torch.equal(ops.rowseg_max_codes(x1, x3), _host_codes(x1, x3))
    assert torch.equal(ops.rowseg_max_codes(x1, x3).cpu().to(torch.int32), O.rowseg_max_codes(x1.cpu(), x3.cpu()))


def test_bound_holds_for_every_x1_pattern(dev):
    """All 65536 bf16 patterns of x1 against a spread of gh and x3 values: wherever the gradient is finite, its
    magnitude is below what the element's own bound allows (the property the skipping of blocks rests on)."""
    pats = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).to(dev)
    others = torch.tensor([1.0, -3.0, 0.37, 1e-3, 255.0, 1.99, 1e-30, 3e20, -7.5e-4, 0.0078125], dtype=torch.bfloat16, device=dev)
    # mantissas where the sum of two codes under-estimates the product's logarithm the most (around sqrt(2) - 1) and
    # where the product's mantissa wraps (around 2 - sqrt(2)), on several exponents, for gh and for x3
    worst = torch.tensor([m * e for m in (1.4140625, 1.4765625, 1.171875, 1.5859375, 1.40625, 1.421875)
                          for e in (1.0, -2.0 ** -10, 2.0 ** 7, 2.0 ** -20)], dtype=torch.bfloat16, device=dev)
    for gv in torch.cat([others, worst]).tolist():
        for bv in torch.cat([others[:6], worst[::4], worst[1::4]]).tolist():
            x1 = pats.view(256, 256).contiguous()
            x3 = torch.full_like(x1, bv)
            gh = torch.full_like(x1, gv)
            g1, g3, _, _ = ops.swiglu_bwd(x1, x3, gh, want_amax=False)
            lg, la, lb = _L(gh), _L(x1), _L(x3)
            finite_in = (la < 0x7F80) & (lb < 0x7F80) & (lg < 0x7F80)
            for name, grad, s, margin in (("g3", g3, lg + la, M3), ("g1", g1, lg + lb, M1)):
                lgr = _L(grad)
                ok = finite_in & (lgr < 0x7F80) & (lgr >= 0x0400)
                # log2 |grad| >= L(grad) / 128 - 127 must not exceed the bound (s + margin) / 128 - 254 (the sum of the
                # elements' own codes: segment codes are maxima of these and only loosen the bound)
                bad = ok & (lgr + BIAS > s + margin)
                assert not bad.any(), f"{name}: bound violated for x1 pattern {int(pats.view(-1)[bad.view(-1)][0].view(torch.int16))}, gh {gv}, x3 {bv}"


@pytest.mark.parametrize("kind", KINDS)
@pytest.mark.parametrize("shape", [(512, 256), (1000, 200), (2048, 1408)], ids=lambda s: "x".join(map(str, s)))
def test_amax_from_codes_equals_dense_pass(dev, shape, kind):
    x1, x3, gh = _inputs(dev, *shape, kind)
    want1, want3 = _dense_amax(x1, x3, gh)
    got1, got3 = _amax_via_codes(x1, x3, gh)
    assert (got1, got3) == (want1, want3), f"{kind}: amax bits {got1:#x}, {got3:#x} != dense {want1:#x}, {want3:#x}"


def test_maximum_in_a_single_element(dev):
    """One element far above the rest, at corners and edges of segments (the ragged last segment of a row among them)."""
    rows, cols = 200, 136
    for (r, c) in ((0, 0), (31, 63), (32, 64), (199, 135), (199, 0), (0, 135), (96, 127), (170, 128)):
        x1, x3, gh = _inputs(dev, rows, cols, "normal", seed=r * 1000 + c)
        x1[r, c], x3[r, c], gh[r, c] = 9.0, -17.0, 0.5
        assert _amax_via_codes(x1, x3, gh) == _dense_amax(x1, x3, gh), (r, c)


@pytest.mark.parametrize("kind", ["normal", "outliers", "nan_x1"])
def test_cast_through_codes_writes_the_same_bytes(dev, kind):
    x1, x3, gh = _inputs(dev, 768, 640, kind)
    a = ops.swiglu_bwd_cast(x1, x3, gh, E5M2, want_rowmajor=True, want_transposed=True)
    b = ops.swiglu_bwd_cast(x1, x3, gh, E5M2, want_rowmajor=True, want_transposed=True,
                            codes=(ops.rowseg_max_codes(gh), ops.rowseg_max_codes(x1, x3)))
    for u, v in zip(a, b):
        assert torch.equal(u.view(torch.uint8) if u.dtype != torch.float32 else u.view(torch.int32),
                           v.view(torch.uint8) if v.dtype != torch.float32 else v.view(torch.int32))


def test_few_segments_are_computed_on_gaussian_data(dev):
    """The point of the codes: on N(0, 1) activations the exact pass is needed for a small share of the segments."""
    x1, x3, gh = _inputs(dev, 4096, 2816, "normal")
    gc, xc = ops.rowseg_max_codes(gh), ops.rowseg_max_codes(x1, x3)
    state = ops.swiglu_bwd_amax_from_codes(x1, x3, gh, gc, xc)
    s = gc.to(torch.int32) + xc.to(torch.int32)
    l1, l3 = (int(state[0].item()) >> 16) & 0xFFFF, (int(state[1].item()) >> 16) & 0xFFFF
    needed = ((s + M3 > l3 + BIAS) | (s + M1 > l1 + BIAS)).float().mean().item()
    assert needed < 0.02, f"{needed:.4f} of the segments exceed the final thresholds"


@pytest.mark.parametrize("mnk", [(2560, 2816, 512), (2600, 2880, 384), (4096, 1792, 1024)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("a_dt", [E5M2, torch.float8_e4m3fn], ids=["e5m2", "e4m3"])
def test_gemm_records_the_codes_of_what_it_writes(dev, mnk, a_dt):
    """Same output as the plain call, and the codes of the stand-alone kernel on that output (tiles shifted back at
    the ragged ends rewrite their segments with the same codes)."""
    M, N, K = mnk
    assert ops.gemm_codes_supported(M, N, K)
    a = seeded((M, K), 1, std=1e-3).to(dev)
    b = seeded((N, K), 2, std=0.02).to(dev)
    aq, _, sa = ops.cast_tensorwise(a, a_dt)
    bq, _, sb = ops.cast_tensorwise(b, torch.float8_e4m3fn)
    want = ops.gemm_fp8(aq, sa, bq, sb)
    out, codes = ops.gemm_fp8_codes(aq, sa, bq, sb)
    assert torch.equal(out, want)
    ref = ops.rowseg_max_codes(out)
    assert torch.equal(codes, ref), f"{int((codes != ref).sum())} of {codes.numel()} codes differ"


@pytest.mark.parametrize("mhk", [(2560, 2816, 512), (2600, 1472, 384)], ids=lambda s: "x".join(map(str, s)))
def test_fused_forward_records_the_codes_of_x1_and_x3(dev, mhk):
    M, H, K = mhk
    a = seeded((M, K), 1).to(dev)
    w1, w3 = seeded((H, K), 2, std=0.02).to(dev), seeded((H, K), 3, std=0.05).to(dev)
    aq, _, sa = ops.cast_tensorwise(a, torch.float8_e4m3fn)
    w1q, _, s1 = ops.cast_tensorwise(w1, torch.float8_e4m3fn)
    w3q, _, s3 = ops.cast_tensorwise(w3, torch.float8_e4m3fn)
    x1, x3, h, (slots, n) = ops.gemm_fp8_swiglu(aq, sa, w1q, s1, w3q, s3)
    y1, y3, g, (slots2, n2), codes = ops.gemm_fp8_swiglu(aq, sa, w1q, s1, w3q, s3, want_codes=True)
    assert torch.equal(x1, y1) and torch.equal(x3, y3) and torch.equal(h, g)
    assert int(slots[:n].max().item()) == int(slots2[:n2].max().item())
    ref = ops.rowseg_max_codes(x1, x3)
    assert torch.equal(codes, ref), f"{int((codes != ref).sum())} of {codes.numel()} codes differ"


def test_shapes_the_gemm_does_not_take(dev):
    assert not ops.gemm_codes_supported(2560, 2816 + 8, 512)   # N % 64
    assert not ops.gemm_codes_supported(512, 512, 512)         # few tiles: another kernel runs the plain call
    a = torch.zeros((512, 512), dtype=torch.float8_e4m3fn, device=dev)
    one = torch.ones(1, device=dev)
    with pytest.raises(RuntimeError):
        ops.gemm_fp8_codes(a, one, a, one)


def test_mlp_backward_same_bits_with_and_without_codes(dev):
    from olmo_core_amd.float8 import AOFloat8LinearRecipe, Float8Config
    from olmo_core_amd.nn import FeedForward, feed_forward

    M, D, H = 2560, 512, 2816
    assert ops.gemm_codes_supported(M, H, D)
    g = torch.Generator().manual_seed(0)
    ff = FeedForward(d_model=D, hidden_size=H, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        for p in ff.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    ff = ff.to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe("tensorwise")).apply_float8_linear(ff)
    x, go = seeded((M, D), 1).to(dev), seeded((M, D), 2, std=1e-3).to(dev)
    outs = []
    for flag in (True, False):
        feed_forward.SWIGLU_AMAX_FROM_CODES = flag
        try:
            for p in ff.parameters():
                p.grad = None
            xd = x.clone().requires_grad_(True)
            y = ff(xd)
            y.backward(go)
            outs.append((y, xd.grad, ff.w1.weight.grad.clone(), ff.w2.weight.grad.clone(), ff.w3.weight.grad.clone()))
        finally:
            feed_forward.SWIGLU_AMAX_FROM_CODES = True
    for name, u, v in zip(("y", "gx", "gw1", "gw2", "gw3"), *outs):
        assert torch.equal(u, v), f"{name}: results differ between the two amax routes"

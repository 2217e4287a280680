"""Parity at the stated shapes of the benchmark configurations 2, 3, 4 and 5 (single GEMMs of the 7B shapes of
configuration 2 are in test_gpu_gemm.py): casts bit-exact on the whole tensor or on whole experts, GEMM outputs on
samples of rows and columns so that the host side stays at seconds.

  config 2: the fused 7B feed-forward block fwd+bwd at the shape bench.py times (16384 tokens, 4096 -> 11008 -> 4096)
  config 3: q/k/v/o projection 4096 -> 4096 at 16384 tokens, rowwise recipe (per-row, per-channel, power-of-two scales)
  config 4: 32B-shape MLP, d_model 5120, hidden 27648, 8192 tokens, tensorwise, 0.1 % of x scaled x100
  config 5: 64 experts, d_model 2048, hidden 1024, 131072 routed rows with Zipf-skewed group sizes (7 empty, one of 1 row)
"""

import pytest
import torch

from helpers import (E4M3, E5M2, assert_bytes_equal, assert_gemm_close, assert_scale_equal, seeded, u8)
from oracle import float8_oracle as O

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import AOFloat8LinearRecipe, Float8Config, ops  # noqa: E402
from olmo_core_amd.float8.linear import Float8Linear  # noqa: E402
from olmo_core_amd.float8.native_config import Float8LinearConfig  # noqa: E402
from olmo_core_amd.nn import DroplessMoEMLP, FeedForward  # noqa: E402


# ---- config 2 ------------------------------------------------------------------------------------------------------


def test_config2_fused_mlp_bench_shape(dev):
    """The block bench.py times, at its shape and seed: the dual-B SwiGLU launch over 86 x 64 tiles, the code-recording
    grad_h GEMM, the amax of g1, g3 from 2.8 M row segments and the accumulating grad_x GEMM, stage by stage; every
    byte and the scale of q(h), q(g1), q(g3) as the block used them against the oracle's cast of the device's tensors."""
    from stage_checks import check_mlp_stages

    M, D, H = 16384, 4096, 11008
    g = torch.Generator().manual_seed(1002)
    ff = FeedForward(d_model=D, hidden_size=H, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        for p in ff.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).to(torch.bfloat16))
    ff = ff.to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(ff)
    x = torch.randn(M, D, generator=g).to(torch.bfloat16)
    go = (torch.randn(M, D, generator=g) * 1e-3).to(torch.bfloat16)
    sink = check_mlp_stages(dev, ff, x, go, sample=12)
    assert sink["amax_from_codes"], "the benchmark's shape takes the row-segment-code route"


# ---- config 3 ------------------------------------------------------------------------------------------------------


def test_config3_rowwise_projection_full_shape(dev):
    M, K, N = 16384, 4096, 4096
    spec = O.recipe("rowwise")
    x, w, go = seeded((M, K), 1003), seeded((N, K), 1013, std=0.02), seeded((M, N), 1023, std=1e-3)
    xd, god = x.to(dev), go.to(dev)

    # the two-product cast of x and grad_output (per-row copy + per-column transposed copy): every byte, every scale
    for name, t, td in (("x", x, xd), ("grad_output", go, god)):
        q, srow, q_t, scol = ops.cast_rows_and_colwise_t(td, E4M3, pow2=True)
        ref_r, ref_sr = O.cast(t, E4M3, O.AXISWISE, -1, True)
        ref_c, ref_sc = O.cast(t, E4M3, O.AXISWISE, 0, True)
        assert_scale_equal(srow, ref_sr, f"{name}: row scales")
        assert_scale_equal(scol, ref_sc, f"{name}: column scales")
        assert_bytes_equal(q, ref_r, what=f"{name}: per-row bytes")
        assert_bytes_equal(q_t[:, :M], ref_c.t(), what=f"{name}: per-column bytes (transposed copy)")
        assert int(u8(q_t[:, M:]).max()) == 0 if q_t.shape[1] > M else True
        del q, q_t, ref_r, ref_c

    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        lin.weight.copy_(w)
    f8 = Float8Linear.from_float(lin.to(dev), Float8LinearConfig.from_recipe_name("rowwise"))
    xg = xd.clone().requires_grad_(True)
    y = f8(xg)
    y.backward(god)

    # output and grad_input rows depend on their own row of x / grad_output only (per-row scales): the oracle runs on
    # the sampled rows
    rows = torch.arange(7, M, 1021)
    tr = O.linear_forward(x[rows], w, None, spec)
    assert_gemm_close(y[rows.to(dev)], tr.out, "out rows")
    gi = O.linear_backward(x[rows], w, go[rows], spec).grad_input
    assert_gemm_close(xg.grad[rows.to(dev)], gi, "grad_input rows")
    # grad_weight sums over all tokens with per-column scales of both operands: whole-tensor casts, sampled rows of W
    go8, sgo = O.cast(go, E4M3, O.AXISWISE, 0, True)
    x8, sx = O.cast(x, E4M3, O.AXISWISE, 0, True)
    nrows = torch.arange(3, N, 331)
    ref_gw = O.emulated_mm_f32(go8.t()[nrows], sgo.t()[nrows], x8, sx)
    assert_gemm_close(f8.weight.grad[nrows.to(dev)], ref_gw, "grad_weight rows")


# ---- config 4 ------------------------------------------------------------------------------------------------------


def _outlier_x(m, d, seed):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(m, d, generator=g)
    pos = torch.randperm(m * d, generator=g)[: m * d // 1000]
    x.view(-1)[pos] *= 100
    return x.bfloat16()


def test_config4_outlier_activations_cast_full_shape(dev):
    """x [8192, 5120] with 0.1 % of the entries x100: amax, scale, every byte of both copies; most of the mass then
    sits in the lowest e4m3 codes and the subnormal range."""
    M, D = 8192, 5120
    x = _outlier_x(M, D, 1004)
    assert float(x.abs().max()) > 300
    q, q_t, s = ops.cast_tensorwise(x.to(dev), E4M3, want_transposed=True)
    ref_q, ref_s = O.cast(x, E4M3)
    assert_scale_equal(s, ref_s, "tensorwise scale")
    assert_bytes_equal(q, ref_q, what="row-major")
    assert_bytes_equal(q_t[:, :M], ref_q.t(), what="transposed")
    codes = u8(q) & 0x7F
    # with the outliers setting the scale (about 1 instead of about 100) a visible part of the N(0,1) bulk lands in
    # the subnormal codes
    assert float((codes < 0x08).float().mean()) > 0.005


@pytest.mark.parametrize("shape,a_dtype", [((8192, 27648, 5120), E4M3), ((8192, 5120, 27648), E5M2),
                                           ((27648, 5120, 8192), E5M2)], ids=["fwd", "dgrad", "wgrad"])
def test_config4_gemm_shapes_row_sample(dev, shape, a_dtype):
    M, N, K = shape
    a = _outlier_x(M, K, 4001) if a_dtype is E4M3 else seeded((M, K), 4002, std=1e-3)
    b = seeded((N, K), 4003, std=0.02)
    aq, _, sa = ops.cast_tensorwise(a.to(dev), a_dtype)
    bq, _, sb = ops.cast_tensorwise(b.to(dev), E4M3)
    out = ops.gemm_fp8(aq, sa, bq, sb)
    rows = torch.arange(5, M, max(M // 11, 1))
    ref = O.emulated_mm_f32(aq[rows.to(dev)].cpu(), sa.cpu()[0], bq.cpu().t(), sb.cpu()[0])
    assert_gemm_close(out[rows.to(dev)], ref, "row sample")
    cols = torch.arange(1, N, max(N // 7, 1))
    ref_c = O.emulated_mm_f32(aq.cpu(), sa.cpu()[0], bq[cols.to(dev)].cpu().t(), sb.cpu()[0])
    assert_gemm_close(out[:, cols.to(dev)], ref_c, "column sample")


def test_config4_mlp_full_weights_reduced_tokens(dev):
    """The whole block with the full 5120 x 27648 weights and outlier activations on 256 tokens, stage by stage."""
    from stage_checks import check_mlp_stages

    M, D, H = 256, 5120, 27648
    g = torch.Generator().manual_seed(1004)
    ff = FeedForward(d_model=D, hidden_size=H, bias=False, dtype=torch.bfloat16)
    with torch.no_grad():
        for p in ff.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    ff = ff.to(dev)
    Float8Config(ao_recipe=AOFloat8LinearRecipe.tensorwise).apply_float8_linear(ff)
    check_mlp_stages(dev, ff, _outlier_x(M, D, 1014), seeded((M, D), 1024, std=1e-3))


# ---- config 5 ------------------------------------------------------------------------------------------------------


def _zipf_sizes():
    """The group sizes of the benchmark's configuration 5 (bench.py): Zipf(s=1.1) bias on the router logits."""
    g = torch.Generator().manual_seed(1005)
    E, T, top_k = 64, 16384, 8
    rank = torch.arange(1, E + 1, dtype=torch.float64)
    pmf = rank ** -1.1
    pmf = pmf / pmf.sum()
    logits = torch.randn(T, E, generator=g) + (1.75 * torch.log(pmf)).float()
    idx = logits.float().softmax(-1).topk(top_k, dim=-1).indices.reshape(-1)
    return torch.bincount(idx, minlength=E).tolist()


def test_config5_grouped_casts_full_shape(dev):
    """The two-product grouped cast of x [131072, 2048] with the 64 Zipf group sizes: whole experts bit-exact (the
    largest, a mid-sized one, the one-row expert, the neighbours of empty experts), scales included; the transposed
    copy's 128-aligned segments and zero padding."""
    sizes = _zipf_sizes()
    E, T, D = 64, 131072, 2048
    assert len(sizes) == E and sum(sizes) == T and sizes.count(0) == 7 and 1 in sizes
    x = seeded((T, D), 1005)
    sz = torch.tensor(sizes).to(dev)
    q, srow, q_t, scol = ops.grouped_cast_rows_and_colwise_t(x.to(dev), sz, E4M3, pow2=True)
    starts, seg = [0], [0]
    for n in sizes:
        starts.append(starts[-1] + n)
        seg.append(seg[-1] + (n + 127) // 128 * 128)
    assert q_t.shape[1] >= seg[-1]
    picked = [0, 20, sizes.index(1), 50, 62]
    for e in picked:
        n = sizes[e]
        xe = x[starts[e]:starts[e] + n]
        ref_r, ref_sr = O.cast(xe, E4M3, O.AXISWISE, -1, True)
        ref_c, ref_sc = O.cast(xe, E4M3, O.AXISWISE, 0, True)
        assert_scale_equal(srow[starts[e]:starts[e] + n], ref_sr, f"expert {e}: row scales")
        assert_scale_equal(scol[e], ref_sc, f"expert {e}: column scales")
        assert_bytes_equal(q[starts[e]:starts[e] + n], ref_r, what=f"expert {e}: per-row bytes")
        assert_bytes_equal(q_t[:, seg[e]:seg[e] + n], ref_c.t(), what=f"expert {e}: per-column bytes")
        if seg[e + 1] > seg[e] + n:
            assert int(u8(q_t[:, seg[e] + n:seg[e + 1]]).max()) == 0, f"expert {e}: padding must be zero bytes"
    for e, n in enumerate(sizes):
        if n == 0:
            assert seg[e + 1] == seg[e]  # an empty expert owns no segment


def test_config5_expert_layer_full_shape(dev):
    """DroplessMoEMLP fwd+bwd at the benchmark's shape (64 experts, 131072 rows, the Zipf sizes), every stage of
    selected experts against the per-expert oracle on the device's own intermediates; zero weight gradients for the
    empty experts."""
    from stage_checks import check_dropless_stages

    sizes = _zipf_sizes()
    E, T, D, H = 64, 131072, 2048, 1024
    mlp = DroplessMoEMLP(d_model=D, hidden_size=H, num_experts=E, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(1015)
    with torch.no_grad():
        for p in mlp.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    x, go = seeded((T, D), 1025), seeded((T, D), 1035, std=1e-3)
    empty = [e for e, n in enumerate(sizes) if n == 0]
    picked = [0, 17, 33, sizes.index(1), 63 if sizes[63] else 62] + empty
    check_dropless_stages(dev, mlp, x, go, sizes, experts=picked)

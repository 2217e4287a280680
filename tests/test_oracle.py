"""
Pins the CPU oracle (oracle/float8_oracle.py, oracle/fp8_cast_ref.c) without importing the reference:
library routines against an independent bit-level implementation, closed forms against exact rational
arithmetic, brute force on small inputs, and invariants a plausible mistake would break.
"""

import math
from fractions import Fraction

import numpy as np
import pytest
import torch

from helpers import E4M3, E5M2, all_bf16_patterns, seeded
from oracle import c_oracle as C
from oracle import float8_oracle as O

CODE = {E4M3: C.E4M3, E5M2: C.E5M2}


# ---- cast: torch-CPU converter vs bit-level C restatement, exhaustively ----------------------------


@pytest.mark.parametrize("fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
def test_cast_exhaustive_torch_vs_c(fp8):
    x = all_bf16_patterns()
    bits = x.view(torch.int16).numpy().view(np.uint16)
    for s in (1.0, 0.37, 2.0**-3, 448 / 3.14159, 1e-3, 57344 / 0.0113, 4.48e14, 0.0):
        st = torch.tensor(s, dtype=torch.float32)
        ref = O.cast_with_scale(x, st, fp8).view(torch.uint8).numpy()
        got = C.cast_bf16_bits(bits, float(st), CODE[fp8])
        assert np.array_equal(ref, got), f"scale {s}: {(ref != got).sum()} mismatches"


def test_cast_known_answers():
    """Hand-derived encodings: ties to even, subnormals, saturation, -0, NaN, inf."""
    def enc(vals, fp8):
        return O.to_fp8_saturated(torch.tensor(vals, dtype=torch.float32), fp8).view(torch.uint8).tolist()

    # e4m3fn: 16 = 0x58 (exp 11, mant 0); spacing 2 in [16,32): 17 ties to 16, 19 ties to 20
    assert enc([16, 17, 18, 19, 20, 21, 23], E4M3) == [0x58, 0x58, 0x59, 0x5A, 0x5A, 0x5A, 0x5C]
    # smallest subnormal 2^-9; half of it ties to zero (even); just above goes up
    assert enc([2.0**-9, 2.0**-10, 1.5 * 2.0**-10, 3 * 2.0**-10], E4M3) == [0x01, 0x00, 0x01, 0x02]
    # saturation at 448 = 0x7E, sign kept; -0 kept; inf clamps to max; NaN stays NaN with its sign
    assert enc([448, 449, 1e9, -1e9, float("inf"), -float("inf")], E4M3) == [0x7E, 0x7E, 0x7E, 0xFE, 0x7E, 0xFE]
    assert enc([-0.0, 0.0], E4M3) == [0x80, 0x00]
    assert enc([float("nan")], E4M3) == [0x7F]
    # e5m2: 57344 = 0x7B max; spacing 8192 in [32768, 65536): 61440 would tie to inf but is clamped first
    assert enc([57344, 61440, 1e9, -1e9], E5M2) == [0x7B, 0x7B, 0x7B, 0xFB]
    assert enc([1.0, 1.125, 1.25, 1.375, 1.5], E5M2) == [0x3C, 0x3C, 0x3D, 0x3E, 0x3E]
    assert enc([2.0**-16, 2.0**-17, 1.5 * 2.0**-17], E5M2) == [0x01, 0x00, 0x01]
    # the unsaturated converter overflows to NaN (e4m3fn has no inf) - what the clamp protects against
    assert torch.tensor([1e9]).to(E4M3).view(torch.uint8).item() == 0x7F


def test_decoders_against_format_tables():
    """Every fp8 code decodes to the value the format specification gives it (tests/golden/fp8_decode_tables.json,
    built from the closed form with exact rationals): torch-CPU and the C restatement, independently."""
    import json
    import math
    from pathlib import Path

    tables = json.loads((Path(__file__).parent / "golden" / "fp8_decode_tables.json").read_text())
    for fp8, name in ((E4M3, "float8_e4m3fn"), (E5M2, "float8_e5m2")):
        codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
        got_torch = codes.view(fp8).float()
        for c, want in enumerate(tables[name]):
            got_c = C.lib().orc_fp8_to_f32(c, CODE[fp8])
            for got in (float(got_torch[c]), float(got_c)):
                if want == "nan":
                    assert math.isnan(got), (name, c)
                elif want in ("inf", "-inf"):
                    assert got == float(want), (name, c)
                elif want == "-0.0":
                    assert got == 0.0 and math.copysign(1.0, got) < 0, (name, c)
                else:
                    assert got == float.fromhex(want), (name, c, got, want)


def test_cast_decode_roundtrip():
    """Every finite fp8 code decodes (C table) to a float that encodes back to the same code."""
    for fp8 in (E4M3, E5M2):
        for b in range(256):
            v = C.fp8_to_f32(b, CODE[fp8])
            tv = torch.tensor([b], dtype=torch.uint8).view(fp8).float().item()
            assert (math.isnan(v) and math.isnan(tv)) or v == tv, (fp8, b)
            if math.isfinite(v):
                assert C.lib().orc_f32_to_fp8(v, CODE[fp8]) == b


# ---- scale: closed form against exact rational arithmetic -------------------------------------


def _exact_scale(amax: float, fmax: float) -> float:
    """float32(fmax / max(amax, 1e-12)) with the division done exactly (rationals), rounded once."""
    a = max(Fraction(amax), Fraction(1e-12))
    q = Fraction(fmax) / a
    # round the exact rational to float64 then float32 would double-round; go to float32 directly
    f = np.float32(float(q))
    lo, hi = np.nextafter(f, np.float32(-np.inf)), np.nextafter(f, np.float32(np.inf))
    best = min((lo, f, hi), key=lambda c: (abs(Fraction(float(c)) - q), int(np.float32(c).view(np.uint32)) & 1))
    return float(best)


def test_scale_every_bf16_amax_against_rationals():
    vals = all_bf16_patterns()
    vals = vals[(vals > 0) & torch.isfinite(vals)]
    assert vals.numel() == 32639
    for fp8, fmax in ((E4M3, 448.0), (E5M2, 57344.0)):
        got = O.amax_to_scale(vals, fp8).numpy()
        step = 7  # every 7th value keeps the rational arithmetic fast yet covers all exponents/mantissas
        for i in range(0, vals.numel(), step):
            assert float(got[i]) == _exact_scale(float(vals[i]), fmax), (fp8, float(vals[i]))
        c = np.array([C.scale_from_amax(float(v), CODE[fp8], False) for v in vals[::step]], dtype=np.float32)
        assert np.array_equal(c, got[::step])


def test_scale_special_values():
    for fp8, fmax in ((E4M3, 448.0), (E5M2, 57344.0)):
        s = O.amax_to_scale(torch.tensor(0.0, dtype=torch.bfloat16), fp8)
        assert float(s) == float(np.float32(fmax / 1e-12)) == C.scale_from_amax(0.0, CODE[fp8], False)
        assert float(O.amax_to_scale(torch.tensor(float("inf")), fp8)) == 0.0
        assert C.scale_from_amax(float("inf"), CODE[fp8], False) == 0.0
        assert math.isnan(float(O.amax_to_scale(torch.tensor(float("nan")), fp8)))
        assert math.isnan(C.scale_from_amax(float("nan"), CODE[fp8], False))


def test_pow2_rounding_is_round_down():
    vals = all_bf16_patterns()
    vals = vals[(vals > 0) & torch.isfinite(vals)]
    for fp8 in (E4M3, E5M2):
        s = O.amax_to_scale(vals, fp8, pow2=False)
        p = O.amax_to_scale(vals, fp8, pow2=True)
        m, e = np.frexp(s.numpy().astype(np.float64))
        want = np.ldexp(0.5, e)  # s = m * 2^e with m in [0.5, 1): largest power of two <= s
        assert np.array_equal(p.numpy().astype(np.float64), want)
        c = np.array([C.scale_from_amax(float(v), CODE[fp8], True) for v in vals[::5]], dtype=np.float32)
        assert np.array_equal(c, p.numpy()[::5])


# ---- amax -------------------------------------------------------------------------------------------


def test_amax_brute_force():
    x = seeded((13, 48), 3)
    assert float(O.tensor_to_amax(x)) == max(abs(float(v)) for v in x.reshape(-1))
    rows = O.tensor_to_amax(x, O.AXISWISE, -1)
    cols = O.tensor_to_amax(x, O.AXISWISE, 0)
    assert rows.shape == (13, 1) and cols.shape == (1, 48) and rows.dtype == torch.bfloat16
    for r in range(13):
        assert float(rows[r, 0]) == max(abs(float(v)) for v in x[r])
    for c in range(48):
        assert float(cols[0, c]) == max(abs(float(v)) for v in x[:, c])
    bits = x.view(torch.int16).numpy().view(np.uint16)
    assert C.amax_bf16_bits(bits) == float(O.tensor_to_amax(x))
    x[2, 2] = float("nan")
    assert math.isnan(float(O.tensor_to_amax(x)))
    assert math.isnan(C.amax_bf16_bits(x.view(torch.int16).numpy().view(np.uint16)))


# ---- emulated mm -----------------------------------------------------------------------------------


def test_emulated_mm_against_library_and_float64():
    x, w = seeded((48, 128), 1), seeded((80, 128), 2, std=0.02)
    a8, sa = O.cast(x, E4M3)
    b8, sb = O.cast(w, E4M3)
    out = O.emulated_mm_f32(a8, sa, b8.t(), sb)
    lib = torch._scaled_mm(a8, b8.t(), scale_a=sa.reciprocal(), scale_b=sb.reciprocal(), out_dtype=torch.float32)
    assert (out - lib).abs().max() <= 1e-3 * out.abs().max()
    f64 = (a8.double() / sa.double()) @ (b8.double() / sb.double()).t()
    assert (out.double() - f64).abs().max() <= 1e-5 * f64.abs().max()
    # the C restatement (double accumulation) on the same bytes
    cmm = C.emulated_mm(a8.view(torch.uint8).numpy(), C.E4M3, sa.numpy(), b8.view(torch.uint8).numpy(), C.E4M3, sb.numpy())
    assert np.abs(cmm - f64.numpy()).max() <= 1e-6 * np.abs(cmm).max()
    # axiswise scales broadcast on the right axes: rows of a, columns of b
    a8r, sar = O.cast(x, E4M3, O.AXISWISE, -1, True)
    b8c, sbc = O.cast(w.t(), E4M3, O.AXISWISE, 0, True)
    assert sar.shape == (48, 1) and sbc.shape == (1, 80)
    outr = O.emulated_mm_f32(a8r, sar, b8c, sbc)
    cr = C.emulated_mm(a8r.view(torch.uint8).numpy(), C.E4M3, sar.numpy(), b8c.t().contiguous().view(torch.uint8).numpy(), C.E4M3, sbc.numpy())
    assert np.abs(outr.double().numpy() - cr).max() <= 1e-5 * np.abs(cr).max()


# ---- autograd wiring -----------------------------------------------------------------------------


@pytest.mark.parametrize("recipe", ["tensorwise", "rowwise", "rowwise_with_gw_hp"])
def test_linear_gradients_track_autograd(recipe):
    M, K, N = 96, 128, 160
    x, w, go = seeded((M, K), 1), seeded((N, K), 2, std=0.02), seeded((M, N), 3, std=1e-3)
    b = seeded((N,), 4)
    tr = O.linear_fwd_bwd(x, w, b, go, O.recipe(recipe))
    xr, wr, br = x.float().requires_grad_(), w.float().requires_grad_(), b.float().requires_grad_()
    y = torch.nn.functional.linear(xr, wr, br)
    y.backward(go.float())

    def cos(a, b_):
        a, b_ = a.float().reshape(-1), b_.float().reshape(-1)
        return float(torch.dot(a, b_) / (a.norm() * b_.norm()))

    assert cos(tr.out, y.detach()) > 0.999
    assert cos(tr.grad_input, xr.grad) > 0.998
    assert cos(tr.grad_weight, wr.grad) > 0.998
    assert cos(tr.grad_bias, br.grad) > 0.9999
    assert tr.grad_input.shape == x.shape and tr.grad_weight.shape == w.shape


def test_linear_exact_on_representable_inputs():
    """Small integers under power-of-two scales are held exactly by fp8 (|v| <= 4 or 8 needs <= 2 mantissa
    bits), so the float8 path must equal the exact product: a transposed operand, a swapped scale or a scale
    applied on the wrong axis shows up as an inequality."""
    g = torch.Generator().manual_seed(0)
    x = torch.randint(-4, 5, (32, 64), generator=g).float(); x[0, 0] = 8.0
    w = torch.randint(-4, 5, (48, 64), generator=g).float(); w[0, 0] = 8.0
    go = torch.randint(-4, 5, (32, 48), generator=g).float(); go[0, 0] = 8.0
    tr = O.linear_fwd_bwd(x, w, None, go, O.LinearSpec(round_scales_to_power_of_2=True))
    assert float(tr.operands["input"][1]) == 32.0 and float(tr.operands["grad_output"][1]) == 4096.0
    assert torch.equal(tr.out, x @ w.t())
    assert torch.equal(tr.grad_input, go @ w)
    assert torch.equal(tr.grad_weight, go.t() @ x)


def test_rowwise_exact_on_representable_inputs():
    """Same idea for the axiswise recipe with rows and columns of different magnitude: exact only if every
    scale vector is applied along the right axis of the right operand."""
    g = torch.Generator().manual_seed(1)
    M, K, N = 24, 32, 40
    x = torch.randint(-4, 5, (M, K), generator=g).float() * (2.0 ** (torch.arange(M) % 4)).unsqueeze(1)
    x = x * (2.0 ** (torch.arange(K) % 3)).unsqueeze(0)
    w = torch.randint(-4, 5, (N, K), generator=g).float() * (2.0 ** (torch.arange(N) % 5)).unsqueeze(1)
    go = torch.randint(-4, 5, (M, N), generator=g).float() * (2.0 ** (torch.arange(N) % 2)).unsqueeze(0)
    tr = O.linear_fwd_bwd(x, w, None, go, O.recipe("rowwise"))
    assert torch.equal(tr.out, x @ w.t())
    assert torch.equal(tr.grad_input, go @ w)
    assert torch.equal(tr.grad_weight, go.t() @ x)


def test_operand_layouts_of_the_six_casts():
    M, K, N = 32, 48, 64
    x, w, go = seeded((M, K), 1), seeded((N, K), 2), seeded((M, N), 3)
    ops_ = O.linear_fwd_bwd(x, w, None, go, O.recipe("rowwise")).operands
    assert ops_["input"][1].shape == (M, 1)
    assert ops_["weight"][0].shape == (K, N) and ops_["weight"][1].shape == (1, N)
    assert ops_["grad_output"][1].shape == (M, 1)
    assert ops_["weight_for_grad_input"][1].shape == (K, 1)
    assert ops_["grad_output_for_grad_weight"][1].shape == (1, N)
    assert ops_["input_for_grad_weight"][1].shape == (1, K)
    # all e4m3 and power-of-two scales in this recipe
    for q, s in ops_.values():
        assert q.dtype == E4M3
        m, _ = np.frexp(s.numpy())
        assert np.all(m == 0.5)
    t = O.linear_fwd_bwd(x, w, None, go, O.recipe("tensorwise")).operands
    assert t["grad_output"][0].dtype == E5M2 and t["input"][0].dtype == E4M3
    assert torch.equal(t["weight"][0].view(torch.uint8), t["weight_for_grad_input"][0].view(torch.uint8))


# ---- grouped / routing -----------------------------------------------------------------------------


def test_grouped_matches_per_expert_dense_and_handles_empty_groups():
    E, D, H = 4, 32, 48
    sizes = [5, 0, 9, 2]
    T = sum(sizes)
    x, go = seeded((T, D), 1), seeded((T, H), 2, std=1e-3)
    w = seeded((E, H, D), 3, std=0.02)
    spec = O.recipe("rowwise")
    out, gx, gw, _ = O.grouped_linear_fwd_bwd(x, w, sizes, go, spec, trans_b=True)
    assert out.shape == (T, H) and gx.shape == (T, D) and gw.shape == (E, H, D)
    assert torch.count_nonzero(gw[1]) == 0
    start = 0
    for e, n in enumerate(sizes):
        if n:
            tr = O.linear_fwd_bwd(x[start:start + n], w[e], None, go[start:start + n], spec)
            assert torch.equal(out[start:start + n], tr.out)
            assert torch.equal(gw[e], tr.grad_weight)
        start += n
    # w2 layout [E, K, N] used as-is
    w2 = seeded((E, D, H), 4, std=0.02)
    out2, _, gw2, _ = O.grouped_linear_fwd_bwd(x, w2, sizes, go, spec, trans_b=False)
    ref = torch.cat([x[0:5] @ w2[0], x[5:14] @ w2[2], x[14:16] @ w2[3]])
    cos = torch.nn.functional.cosine_similarity(out2.float().reshape(-1), ref.float().reshape(-1), dim=0)
    assert out2.shape == (T, H) and gw2.shape == w2.shape and float(cos) > 0.999


def test_dropless_mlp_shape_contract():
    """x [5,128], tokens_per_expert [3,2] -> [5,128] (reference: src/test/nn/moe/mlp_test.py:30-39)."""
    E, D, H = 2, 128, 256
    x = seeded((5, D), 1)
    w1, w2, w3 = (seeded((E, H, D), s, std=0.05) for s in (2, 3, 4))
    res = O.dropless_mlp_fwd_bwd(x, w1, w2, w3, [3, 2], None, O.recipe("rowwise"))
    assert res["y"].shape == (5, 128)


def test_batched_histc_known_answer():
    """reference: src/test/ops/moe_test.py:158-164."""
    x = torch.tensor([[0, 1, 1], [2, 0, 0]])
    assert O.batched_histc(x, 5).tolist() == [[1, 2, 0, 0, 0], [2, 0, 1, 0, 0]]


def test_routing_bins():
    g = torch.Generator().manual_seed(0)
    logits = torch.randn(64, 8, generator=g)
    indices, bin_ids, bins, sizes = O.route_top_k(logits, 2)
    assert int(sizes.sum()) == 128 and bins[-1] == 128
    assert torch.equal(bins.long(), torch.cumsum(sizes, 0))
    assert bool((bin_ids[1:] >= bin_ids[:-1]).all())


# ---- compositions: SwiGLU MLP and dropless-MoE MLP against float32 autograd ---------------------------


def _cos(a, b):
    a, b = a.double().reshape(-1), b.double().reshape(-1)
    return float(torch.dot(a, b) / (a.norm() * b.norm()))


def _norm_ratio(a, b):
    return float(a.double().norm() / b.double().norm())


# float8 noise bounds for the cosine: one e4m3 x e4m3 product is ~0.9993, the product of two such results
# (h) ~0.9985; a gradient that passes through two e5m2 re-quantisations is ~0.9955.  A mis-wired composition
# (g1/g3 swapped, an operand transposed, one grad_x term dropped, w2 used like w1) scores <= 0.95 on at least
# one tensor with these inputs (asserted below), far outside these bounds.
_COS_FWD, _COS_BWD = 0.998, 0.994


@pytest.mark.parametrize("recipe", ["tensorwise", "rowwise"])
def test_mlp_composition_tracks_autograd(recipe):
    """All five results of mlp_fwd_bwd against float32 autograd of w2(silu(w1 x) * w3 x)
    (src/olmo_core/nn/feed_forward.py:161-171).  w3 is three times larger than w1, so grad_w1 and grad_w3 (and the
    two terms of grad_x) differ in magnitude as well as direction: a swap or a dropped term fails both the cosine
    and the norm-ratio bound."""
    M, D, H = 192, 128, 256
    x = seeded((M, D), 1)
    w1, w3 = seeded((H, D), 2, std=0.08), seeded((H, D), 3, std=0.24)
    w2 = seeded((D, H), 4, std=0.05)
    go = seeded((M, D), 5, std=1e-3)
    tr = O.mlp_fwd_bwd(x, w1, w2, w3, go, O.recipe(recipe))

    xr = x.float().requires_grad_()
    p1, p2, p3 = (w.float().requires_grad_() for w in (w1, w2, w3))
    F = torch.nn.functional
    h = F.silu(F.linear(xr, p1)) * F.linear(xr, p3)
    y = F.linear(h, p2)
    y.backward(go.float())

    assert tr.y.shape == (M, D) and tr.grad_x.shape == x.shape
    assert tr.grad_w1.shape == w1.shape and tr.grad_w2.shape == w2.shape and tr.grad_w3.shape == w3.shape
    assert _cos(tr.h, h.detach()) > _COS_FWD
    assert _cos(tr.y, y.detach()) > 0.997
    for name, got, want in (("grad_x", tr.grad_x, xr.grad), ("grad_w1", tr.grad_w1, p1.grad),
                            ("grad_w2", tr.grad_w2, p2.grad), ("grad_w3", tr.grad_w3, p3.grad)):
        assert _cos(got, want) > _COS_BWD, (name, _cos(got, want))
        assert 0.97 < _norm_ratio(got, want) < 1.03, (name, _norm_ratio(got, want))
    # the inputs do separate the mistakes this test is for
    assert abs(_cos(p1.grad, p3.grad)) < 0.5 and not 0.8 < _norm_ratio(p1.grad, p3.grad) < 1.25
    gx1 = torch.autograd.grad(F.linear(F.silu(F.linear(xr, p1)) * F.linear(xr, p3).detach(), p2), xr, go.float())[0]
    assert _cos(gx1, xr.grad) < 0.95  # one term of grad_x alone is not grad_x


def test_mlp_composition_feeds_each_stage_the_previous_stage():
    """Wiring of the stages, bit for bit: w2 consumes the cast of h, w1/w3's backward consume the casts of the SwiGLU
    gradients of w2's grad_input, and every stage equals the single-linear oracle on those tensors."""
    M, D, H = 64, 64, 96
    x, go = seeded((M, D), 1), seeded((M, D), 5, std=1e-3)
    w1, w3, w2 = seeded((H, D), 2, std=0.1), seeded((H, D), 3, std=0.2), seeded((D, H), 4, std=0.1)
    spec = O.recipe("tensorwise")
    tr = O.mlp_fwd_bwd(x, w1, w2, w3, go, spec)
    x1 = O.linear_forward(x, w1, None, spec).out
    x3 = O.linear_forward(x, w3, None, spec).out
    h = torch.nn.functional.silu(x1) * x3
    assert torch.equal(tr.h, h)
    t2 = O.linear_fwd_bwd(h, w2, None, go, spec)
    assert torch.equal(tr.y, t2.out) and torch.equal(tr.grad_w2, t2.grad_weight)
    # SwiGLU gradient in closed form (float64), compared after the bf16 roundings torch applies
    gh = t2.grad_input.double()
    s = torch.sigmoid(x1.double())
    g1_ref = gh * x3.double() * (s * (1 + x1.double() * (1 - s)))
    g3_ref = gh * (x1.double() * s)
    g1, g3 = O.swiglu_backward(x1, x3, t2.grad_input)
    assert _cos(g1, g1_ref) > 0.99995 and _cos(g3, g3_ref) > 0.99995
    assert torch.equal(tr.grad_w1, O.linear_backward(x, w1, g1, spec).grad_weight)
    assert torch.equal(tr.grad_w3, O.linear_backward(x, w3, g3, spec).grad_weight)
    want_gx = O.linear_backward(x, w1, g1, spec).grad_input + O.linear_backward(x, w3, g3, spec).grad_input
    assert torch.equal(tr.grad_x, want_gx)


def _dropless_autograd(x, w1, w2, w3, sizes, go):
    """The reference's per-expert loop in float32 (src/olmo_core/nn/moe/mlp.py:264-292): w1, w3 [E,H,D] used
    transposed, w2 [E,H,D] used as stored."""
    xr = x.float().requires_grad_()
    p1, p2, p3 = (w.float().requires_grad_() for w in (w1, w2, w3))
    outs, start = [], 0
    for e, n in enumerate(sizes):
        xe = xr[start:start + n]
        he = torch.nn.functional.silu(xe @ p1[e].t()) * (xe @ p3[e].t())
        outs.append(he @ p2[e])
        start += n
    y = torch.cat(outs)
    y.backward(go.float())
    return y.detach(), xr.grad, p1.grad, p2.grad, p3.grad


def test_dropless_mlp_composition_tracks_autograd():
    """dropless_mlp_fwd_bwd against the float32 per-expert loop: experts and the three weight tensors have distinct
    magnitudes, one expert is empty, one has a single row; checked per expert so that a weight taken from the wrong
    expert, w2 used transposed, or w1/w3 swapped shows."""
    E, D, H = 5, 64, 96
    sizes = [40, 0, 1, 23, 64]
    T = sum(sizes)
    x, go = seeded((T, D), 1), seeded((T, D), 5, std=1e-3)
    mag = (2.0 ** torch.arange(E)).reshape(E, 1, 1)
    w1 = (seeded((E, H, D), 2, std=0.05).float() * mag).bfloat16()
    w3 = (seeded((E, H, D), 3, std=0.15).float() * mag.flip(0)).bfloat16()
    w2 = seeded((E, H, D), 4, std=0.1)
    res = O.dropless_mlp_fwd_bwd(x, w1, w2, w3, sizes, go, O.recipe("rowwise"))
    y, gx, g1, g2, g3 = _dropless_autograd(x, w1, w2, w3, sizes, go)

    assert res["y"].shape == (T, D) and res["grad_x"].shape == (T, D)
    for k in ("grad_w1", "grad_w2", "grad_w3"):
        assert res[k].shape == (E, H, D)
        assert torch.count_nonzero(res[k][1]) == 0, "the empty expert's weight gradient is zero"
    start = 0
    for e, n in enumerate(sizes):
        if n:
            rows = slice(start, start + n)
            assert _cos(res["y"][rows], y[rows]) > 0.996, (e, "y", _cos(res["y"][rows], y[rows]))
            assert _cos(res["grad_x"][rows], gx[rows]) > _COS_BWD, (e, "grad_x", _cos(res["grad_x"][rows], gx[rows]))
            assert 0.96 < _norm_ratio(res["grad_x"][rows], gx[rows]) < 1.04
            for name, got, want in (("grad_w1", res["grad_w1"][e], g1[e]), ("grad_w2", res["grad_w2"][e], g2[e]),
                                    ("grad_w3", res["grad_w3"][e], g3[e])):
                assert _cos(got, want) > _COS_BWD, (e, name, _cos(got, want))
                assert 0.96 < _norm_ratio(got, want) < 1.04, (e, name)
        start += n
    # the construction separates the mistakes: other experts' and the transposed w2's results are far away
    assert abs(_cos(g1[0], g3[0])) < 0.5 and abs(_cos(g1[0], g1[4])) < 0.5


def test_dropless_mlp_exact_on_representable_inputs():
    """With silu's argument driven far positive (silu(v) = v to bf16 precision for v >= 32) and small-integer data
    the whole expert MLP is exact in float8 under power-of-two scales: y = ((x w1^T) * (x w3^T)) w2 per expert.
    Any indexing slip between experts changes an integer."""
    E, D, H = 3, 16, 16
    sizes = [3, 0, 5]
    T = sum(sizes)
    g = torch.Generator().manual_seed(0)
    x = torch.zeros(T, D); x[:, 0] = 1.0
    x[:, 1:4] = torch.randint(0, 2, (T, 3), generator=g).float()
    w1 = torch.zeros(E, H, D); w1[:, :, 0] = 32.0            # x1 = 32 for every row and hidden unit
    w3 = torch.randint(-2, 3, (E, H, D), generator=g).float() * torch.tensor([1.0, 2.0, 4.0]).reshape(E, 1, 1)
    w2 = torch.randint(-1, 2, (E, H, D), generator=g).float()
    res = O.dropless_mlp_fwd_bwd(x.bfloat16(), w1.bfloat16(), w2.bfloat16(), w3.bfloat16(), sizes, None, O.recipe("rowwise"))
    start, outs = 0, []
    for e, n in enumerate(sizes):
        xe = x[start:start + n]
        x1 = xe @ w1[e].t()
        assert torch.equal(torch.nn.functional.silu(x1.bfloat16()).float(), x1)  # silu is the identity here
        outs.append((x1 * (xe @ w3[e].t())) @ w2[e])
        start += n
    want = torch.cat(outs)
    assert float(want.abs().max()) <= 2.0**15
    assert torch.equal(res["y"].float(), want.bfloat16().float())


def test_magnitude_codes_bound_the_swiglu_gradients():
    """The property the sparse amax of the gate gradients rests on, against torch's own bf16 autograd: for every bf16
    pattern of x1 and a spread of gh and x3 values, the code of each gradient is at most the sum of the inputs' codes
    plus its margin (checked where inputs and gradient are finite and the gradient is not in the denormal range);
    and the codes are a lower bound on log2 |x| within 0.0861."""
    import numpy as np

    pats = torch.from_numpy(np.arange(65536, dtype=np.uint16).view(np.int16).copy()).view(torch.bfloat16)
    lx = O.bf16_magnitude_code(pats)
    finite = (lx < 0x7F80) & (lx >= 0x0080)
    log2 = torch.log2(pats.double().abs()[finite])
    est = lx[finite].double() / 128 - 127
    assert (est <= log2 + 1e-12).all() and (log2 <= est + 0.0861).all()
    others = torch.tensor([1.0, -3.0, 0.37, 1e-3, 255.0, 1.99, 1e-30, 3e20, -7.5e-4, 0.0078125], dtype=torch.bfloat16)
    # The code of a product exceeds the sum of the factors' codes the most when both mantissas sit near sqrt(2) - 1
    # (a piecewise-linear logarithm under-estimates most in the middle of a binade: the gap is 21.96 of the margin's
    # 24 units there); around 2 - sqrt(2) the mantissa of the product wraps.  Those mantissas, on several exponents,
    # for gh and for x3 (x1 runs over every pattern anyway).
    worst = torch.tensor([m * e for m in (1.4140625, 1.4765625, 1.171875, 1.5859375, 1.40625, 1.421875)
                          for e in (1.0, -2.0 ** -10, 2.0 ** 7, 2.0 ** -20)], dtype=torch.bfloat16)
    assert torch.equal(worst.float()[:4], torch.tensor([1.4140625, -1.4140625 * 2.0 ** -10, 1.4140625 * 128, 1.4140625 * 2.0 ** -20]))
    for gv in torch.cat([others, worst]):
        for bv in torch.cat([others[:6], worst[::4], worst[1::4]]):
            x1 = pats.clone()
            x3 = torch.full_like(x1, bv.item())
            gh = torch.full_like(x1, gv.item())
            g1, g3 = O.swiglu_backward(x1, x3, gh)
            lg, la, lb = O.bf16_magnitude_code(gh), O.bf16_magnitude_code(x1), O.bf16_magnitude_code(x3)
            ok_in = (la < 0x7F80) & (lb < 0x7F80) & (lg < 0x7F80)
            for grad, s, which in ((g1, lg + torch.maximum(la, lb), 0), (g3, lg + torch.maximum(la, lb), 1), (g1, lg + lb, 0), (g3, lg + la, 1)):
                lgr = O.bf16_magnitude_code(grad)
                bound = O.swiglu_gradient_code_bounds(s)[which]
                ok = ok_in & (lgr < 0x7F80) & (lgr >= 0x0400)
                assert not (ok & (lgr > bound)).any(), (gv.item(), bv.item(), which)


def test_rowseg_codes_layout():
    x = torch.zeros((3, 130), dtype=torch.bfloat16)
    x[0, 5], x[1, 64], x[2, 129], x[2, 0] = -2.0, 0.5, 3.0, float("inf")
    codes = O.rowseg_max_codes(x).view(3, 3)  # [segment][row]
    two, half, three = 0x4000, 0x3F00, 0x4040
    assert codes.tolist() == [[two, 0, 0x7F80], [0, half, 0], [0, 0, three]]
    both = O.rowseg_max_codes(x, torch.full_like(x, 1.0)).view(3, 3)
    assert both.tolist() == [[two, 0x3F80, 0x7F80], [0x3F80, 0x3F80, 0x3F80], [0x3F80, 0x3F80, three]]

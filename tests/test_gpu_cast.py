"""Parity of the HIP cast kernels with the CPU oracle: fp8 bytes and float32 scales bit-exact."""

import numpy as np
import pytest
import torch

from helpers import E4M3, E5M2, all_bf16_patterns, assert_bytes_equal, assert_scale_equal, bits32, seeded, u8
from oracle import c_oracle as C
from oracle import float8_oracle as O

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import ops  # noqa: E402

SCALES = [1.0, 0.37, 2.0**-3, 448 / 3.14159, 1e-3, 57344 / 0.0113, 4.48e14, 3.0e-5]


@pytest.fixture(params=[False, True], ids=["hwcvt", "swcvt"])
def cvt_mode(request):
    old = ops.FORCE_SW_CVT
    ops.FORCE_SW_CVT = request.param
    yield request.param
    ops.FORCE_SW_CVT = old


@pytest.mark.parametrize("fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
def test_exhaustive_bf16_patterns(dev, fp8, cvt_mode):
    """All 65536 bf16 bit patterns x 8 scales: bytes equal torch-CPU's saturating RNE cast, row-major and
    transposed; this is where the hardware converter's rounding, subnormal, -0 and NaN behaviour is proven."""
    x = all_bf16_patterns().reshape(256, 256)
    xd = x.to(dev)
    for s in SCALES:
        st = torch.tensor(s, dtype=torch.float32)
        ref = O.cast_with_scale(x, st, fp8)
        q, q_t, s_out = ops.cast_tensorwise(xd, fp8, want_rowmajor=True, want_transposed=True, scale=st.to(dev))
        assert_bytes_equal(q, ref, what=f"scale {s} row-major")
        assert_bytes_equal(q_t, ref.t(), what=f"scale {s} transposed")
        assert bits32(s_out)[0] == bits32(st.reshape(1))[0]


@pytest.mark.parametrize("fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
def test_exhaustive_against_c_oracle(dev, fp8):
    """Same sweep against the independent bit-level C restatement (no torch converter involved)."""
    x = all_bf16_patterns()
    bits = x.view(torch.int16).numpy().view(np.uint16)
    code = C.E4M3 if fp8 is E4M3 else C.E5M2
    for s in (1.0, 0.37, 142.6):
        st = torch.tensor(s, dtype=torch.float32)
        ref = torch.from_numpy(C.cast_bf16_bits(bits, float(st), code)).reshape(256, 256)
        q, _, _ = ops.cast_tensorwise(x.reshape(256, 256).to(dev), fp8, scale=st.to(dev))
        assert_bytes_equal(q, ref, what=f"C oracle scale {s}")


SHAPES = [(1, 16), (3, 48), (17, 16), (100, 272), (128, 128), (129, 144), (300, 4096), (2048, 512), (257, 11008)]


@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
@pytest.mark.parametrize("pow2", [False, True], ids=["", "pow2"])
def test_tensorwise_dynamic(dev, shape, fp8, pow2, cvt_mode):
    x = seeded(shape, seed=shape[0] * 7 + shape[1], std=1.0)
    ref_q, ref_s = O.cast(x, fp8, O.TENSORWISE, None, pow2)
    q, q_t, s = ops.cast_tensorwise(x.to(dev), fp8, pow2=pow2, want_rowmajor=True, want_transposed=True)
    assert_scale_equal(s, ref_s, "tensorwise scale")
    assert_bytes_equal(q, ref_q, what="row-major")
    rows = shape[0]
    assert q_t.shape == (shape[1], ops.pad16(rows))
    assert_bytes_equal(q_t[:, :rows], ref_q.t(), what="transposed")
    assert int(u8(q_t[:, rows:]).max() if q_t.shape[1] > rows else 0) == 0, "padding must be zero bytes"


@pytest.mark.parametrize("shape", [(1, 16), (1, 4096), (7, 528), (16, 4096), (64, 1024), (33, 1040)],
                         ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
@pytest.mark.parametrize("pow2", [False, True], ids=["", "pow2"])
def test_tensorwise_small_single_launch(dev, shape, fp8, pow2, cvt_mode):
    """Up to 65536 elements with only the row-major copy wanted: the cast takes the amax itself (one launch).
    Bytes and scale equal the oracle's and those of the two-kernel route (amax partials, then cast); float32
    input, NaN, an all-zero tensor and a padded output pitch included."""
    x = seeded(shape, seed=shape[0] * 13 + shape[1], std=0.7)
    ref_q, ref_s = O.cast(x, fp8, O.TENSORWISE, None, pow2)
    xd = x.to(dev)
    q, q_t, s = ops.cast_tensorwise(xd, fp8, pow2=pow2)  # the single-launch route
    assert q_t is None
    assert_scale_equal(s, ref_s, "scale")
    assert_bytes_equal(q, ref_q, what="row-major")
    q2, _, s2 = ops.cast_tensorwise(xd, fp8, pow2=pow2, slots=ops.amax_partials(xd))  # the two-kernel route
    assert torch.equal(u8(q), u8(q2)) and torch.equal(s, s2)
    # float32 input and a wider output pitch
    x32 = x.float() * 1.0009765625
    ref_q32, ref_s32 = O.cast(x32, fp8, O.TENSORWISE, None, pow2)
    q32, _, s32 = ops.cast_tensorwise(x32.to(dev), fp8, pow2=pow2, pitch=shape[1] + 32)
    assert q32.stride(0) == shape[1] + 32
    assert_scale_equal(s32, ref_s32, "scale (float32 input)")
    assert_bytes_equal(q32, ref_q32, what="row-major (float32 input)")
    # NaN and all zeros behave as on the two-kernel route
    for special in (torch.zeros(shape, dtype=torch.bfloat16), x.clone()):
        if special.abs().max() > 0:
            special.view(-1)[special.numel() // 2] = float("nan")
        sd = special.to(dev)
        qa, _, sa = ops.cast_tensorwise(sd, fp8, pow2=pow2)
        qb, _, sb = ops.cast_tensorwise(sd, fp8, pow2=pow2, slots=ops.amax_partials(sd))
        assert torch.equal(u8(qa), u8(qb)) and torch.equal(sa.view(torch.int32), sb.view(torch.int32))


@pytest.mark.parametrize("std", [0.02, 1e-3, 50.0, 1e-20])
def test_tensorwise_magnitudes(dev, std):
    x = seeded((333, 528), seed=11, std=std)
    for fp8 in (E4M3, E5M2):
        ref_q, ref_s = O.cast(x, fp8)
        q, q_t, s = ops.cast_tensorwise(x.to(dev), fp8, want_transposed=True)
        assert_scale_equal(s, ref_s)
        assert_bytes_equal(q, ref_q)
        assert_bytes_equal(q_t[:, :333], ref_q.t())


def test_tensorwise_outliers_saturation(dev):
    """0.1 % of entries x100 (the outlier workload): amax comes from an outlier, the clamp is exercised."""
    g = torch.Generator().manual_seed(1004)
    x = torch.randn(512, 1280, generator=g)
    pos = torch.randperm(x.numel(), generator=g)[: x.numel() // 1000]
    x.view(-1)[pos] *= 100
    x = x.bfloat16()
    for fp8 in (E4M3, E5M2):
        ref_q, ref_s = O.cast(x, fp8)
        q, _, s = ops.cast_tensorwise(x.to(dev), fp8)
        assert_scale_equal(s, ref_s)
        assert_bytes_equal(q, ref_q)


def test_tensorwise_special_values(dev):
    base = seeded((64, 64), seed=5)
    cases = {}
    z = torch.zeros(64, 64, dtype=torch.bfloat16)
    cases["all_zero"] = z
    n = base.clone(); n[3, 7] = float("nan"); cases["one_nan"] = n
    i = base.clone(); i[10, 1] = float("inf"); cases["one_inf"] = i
    m = base.clone(); m[0, 0] = -0.0; m[0, 1] = 3.3895e38; cases["huge"] = m
    for name, x in cases.items():
        for fp8 in (E4M3, E5M2):
            ref_q, ref_s = O.cast(x, fp8)
            q, q_t, s = ops.cast_tensorwise(x.to(dev), fp8, want_transposed=True)
            assert_scale_equal(s, ref_s, name)
            assert_bytes_equal(q, ref_q, what=name)
            assert_bytes_equal(q_t, ref_q.t(), what=name + " transposed")


def test_tensorwise_float32_input(dev):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(200, 336, generator=g) * 0.02
    for fp8 in (E4M3, E5M2):
        ref_q, ref_s = O.cast(x, fp8)
        q, q_t, s = ops.cast_tensorwise(x.to(dev), fp8, want_transposed=True)
        assert_scale_equal(s, ref_s)
        assert_bytes_equal(q, ref_q)
        assert_bytes_equal(q_t[:, :200], ref_q.t())


def test_amax_partials_and_scale(dev):
    for n in (1, 7, 8, 1000, 8191, 1 << 20, (1 << 22) + 5):
        x = seeded((n,), seed=n, std=3.0)
        slots, used = ops.amax_partials(x.to(dev))
        got = slots[:used].view(torch.float32).max().cpu()
        assert float(got) == float(x.abs().max().float()), n
        for fp8 in (E4M3, E5M2):
            for pow2 in (False, True):
                out = ops.scale_from_partials(slots, used, fp8, pow2).cpu()
                assert_scale_equal(out[0], O.amax_to_scale(x.abs().max(), fp8, pow2), f"n={n}")
                assert float(out[1]) == float(x.abs().max().float())


def test_amax_partials_batch_equals_separate_calls(dev):
    """One launch over several tensors leaves, per tensor, exactly the partials of its own launch (ragged sizes,
    a tail shorter than a vector, float32 as well as bf16, the maximum in the last element)."""
    sizes = (5, 8, 8191, 1 << 20, (1 << 22) + 3, 4096 * 11008, 1000, 64)
    for dt in (torch.bfloat16, torch.float32):
        xs = [seeded((n,), seed=100 + n % 97, std=1.0 + i).to(dt) for i, n in enumerate(sizes)]
        xs[4][-1] = 1e4
        xs[0][4] = -77.0
        xd = [x.to(dev) for x in xs]
        for count in (1, 3, len(xd)):
            got = ops.amax_partials_batch(xd[:count])
            assert len(got) == count
            for x, xdev, (slots, used) in zip(xs, xd, got):
                ref_slots, ref_used = ops.amax_partials(xdev)
                assert used == ref_used
                assert torch.equal(slots[:used], ref_slots[:used])
                assert float(slots[:used].view(torch.float32).max().cpu()) == float(x.abs().max().float())
    with pytest.raises(ValueError):
        ops.amax_partials_batch([xd[0]] * 9)
    with pytest.raises(ValueError):
        ops.amax_partials_batch([xd[0].float(), xd[1].bfloat16()])


def test_scale_every_bf16_amax(dev):
    """Scale for every positive finite bf16 amax value (one row each) - the f64 route on the GPU."""
    vals = all_bf16_patterns()
    vals = vals[(vals > 0) & torch.isfinite(vals)]
    x = torch.zeros(vals.numel(), 16, dtype=torch.bfloat16)
    x[:, 3] = vals
    for fp8 in (E4M3, E5M2):
        for pow2 in (False, True):
            _, s = ops.cast_rowwise(x.to(dev), fp8, pow2=pow2)
            ref = O.amax_to_scale(vals, fp8, pow2)
            assert_scale_equal(s, ref, f"{fp8} pow2={pow2}")


ROW_SHAPES = [(1, 16), (5, 48), (64, 1024), (100, 2048), (33, 4096), (17, 5120), (9, 11008), (5, 27648)]


@pytest.mark.parametrize("shape", ROW_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("pow2", [False, True], ids=["", "pow2"])
def test_rowwise(dev, shape, pow2, cvt_mode):
    x = seeded(shape, seed=shape[1] + 1, std=0.7)
    x[0, :] = 0  # an all-zero row: amax clamps at 1e-12
    if shape[0] > 2:
        x[2, 5] = float("nan")
    for fp8 in (E4M3, E5M2):
        ref_q, ref_s = O.cast(x, fp8, O.AXISWISE, -1, pow2)
        q, s = ops.cast_rowwise(x.to(dev), fp8, pow2=pow2)
        assert_scale_equal(s, ref_s, "rowwise scale")
        assert_bytes_equal(q, ref_q, what="rowwise bytes")


COL_SHAPES = [(1, 16), (16, 16), (100, 272), (255, 128), (256, 4096), (1000, 144), (4100, 512)]


@pytest.mark.parametrize("shape", COL_SHAPES, ids=lambda s: f"{s[0]}x{s[1]}")
@pytest.mark.parametrize("pow2", [False, True], ids=["", "pow2"])
def test_colwise_transposed(dev, shape, pow2, cvt_mode):
    x = seeded(shape, seed=shape[0] + 3, std=0.05)
    x[:, 1] = 0
    if shape[0] > 4:
        x[4, 2] = float("nan")
    rows = shape[0]
    for fp8 in (E4M3, E5M2):
        ref_q, ref_s = O.cast(x, fp8, O.AXISWISE, 0, pow2)
        q_t, s = ops.cast_colwise_t(x.to(dev), fp8, pow2=pow2)
        assert_scale_equal(s, ref_s, "colwise scale")
        assert_bytes_equal(q_t[:, :rows], ref_q.t(), what="colwise bytes")
        if q_t.shape[1] > rows:
            assert int(u8(q_t[:, rows:]).max()) == 0


@pytest.mark.parametrize("shape", [(100, 272), (256, 4096), (1000, 144)], ids=lambda s: f"{s[0]}x{s[1]}")
def test_operand_pitches(dev, shape):
    """Outputs with a row pitch wider than the row: same bytes in the view, nothing written outside it, and a GEMM
    on the padded operands equal to the GEMM on the packed ones."""
    rows, cols = shape
    x = seeded(shape, seed=rows + 11, std=0.3)
    xd = x.to(dev)
    ref_q, ref_s = O.cast(x, E4M3, O.TENSORWISE, None, False)
    q, q_t, s = ops.cast_tensorwise(xd, E4M3, want_transposed=True, pitch=cols + 128, pitch_t=ops.pad16(rows) + 272)
    assert q.stride(0) == cols + 128 and q_t.stride(0) == ops.pad16(rows) + 272
    assert_scale_equal(s, ref_s)
    assert_bytes_equal(q, ref_q, what="row-major view")
    assert_bytes_equal(q_t[:, :rows], ref_q.t(), what="transposed view")
    if q_t.shape[1] > rows:
        assert int(u8(q_t[:, rows:]).max()) == 0
    ref_q, ref_s = O.cast(x, E4M3, O.AXISWISE, -1, True)
    qr, sr = ops.cast_rowwise(xd, E4M3, pow2=True, pitch=cols + 16)
    assert_scale_equal(sr, ref_s)
    assert_bytes_equal(qr, ref_q, what="rowwise view")
    ref_q, ref_s = O.cast(x, E4M3, O.AXISWISE, 0, True)
    qc, sc = ops.cast_colwise_t(xd, E4M3, pow2=True, pitch_t=ops.pad16(rows) + 128)
    assert_scale_equal(sc, ref_s)
    assert_bytes_equal(qc[:, :rows], ref_q.t(), what="colwise view")
    # the GEMMs take the pitch from the view
    packed, _, _ = ops.cast_tensorwise(xd, E4M3)
    w = seeded((256, cols), seed=5, std=0.1).to(E4M3).to(dev)
    one = torch.ones(1, device=dev)
    assert torch.equal(ops.gemm_fp8(q, one, w, one), ops.gemm_fp8(packed, one, w, one))


def test_colwise_float32_input(dev):
    g = torch.Generator().manual_seed(8)
    x = torch.randn(300, 160, generator=g)
    ref_q, ref_s = O.cast(x, E4M3, O.AXISWISE, 0, True)
    q_t, s = ops.cast_colwise_t(x.to(dev), E4M3, pow2=True)
    assert_scale_equal(s, ref_s)
    assert_bytes_equal(q_t[:, :300], ref_q.t())
    ref_q, ref_s = O.cast(x, E5M2, O.AXISWISE, -1, False)
    q, s = ops.cast_rowwise(x.to(dev), E5M2)
    assert_scale_equal(s, ref_s)
    assert_bytes_equal(q, ref_q)


def test_determinism(dev):
    x = seeded((1024, 2048), seed=77).to(dev)
    a = ops.cast_tensorwise(x, E4M3, want_transposed=True)
    b = ops.cast_tensorwise(x, E4M3, want_transposed=True)
    assert torch.equal(a[0].view(torch.uint8), b[0].view(torch.uint8))
    assert torch.equal(a[1].view(torch.uint8), b[1].view(torch.uint8))
    assert torch.equal(a[2], b[2])


def test_full_size_properties(dev):
    """At the 7B MLP activation size (16384 x 4096): the transposed copy is the transpose of the row-major
    copy, the scale equals the oracle's scale for the same amax, and a row sample matches the oracle bytes."""
    g = torch.Generator(device="cpu").manual_seed(1002)
    x = torch.randn(16384, 4096, generator=g).bfloat16()
    xd = x.to(dev)
    q, q_t, s = ops.cast_tensorwise(xd, E4M3, want_transposed=True)
    assert torch.equal(q_t.view(torch.uint8), q.view(torch.uint8).t().contiguous())
    ref_s = O.amax_to_scale(x.abs().max(), E4M3)
    assert_scale_equal(s, ref_s)
    rows = torch.arange(0, 16384, 257)
    assert_bytes_equal(q[rows.to(dev)], O.cast_with_scale(x[rows], ref_s, E4M3), what="row sample")


def test_argument_errors(dev):
    from olmo_core_amd.exceptions import MI8KernelError

    x = torch.zeros(4, 24, dtype=torch.bfloat16, device=dev)
    with pytest.raises(MI8KernelError):
        ops.cast_tensorwise(x, E4M3)  # cols not a multiple of 16
    with pytest.raises(RuntimeError):
        ops.cast_tensorwise(torch.zeros(4, 16, dtype=torch.bfloat16), E4M3)  # CPU tensor: no CPU path
    with pytest.raises(TypeError):
        ops.cast_rowwise(torch.zeros(4, 16, dtype=torch.float16, device=dev), E4M3)

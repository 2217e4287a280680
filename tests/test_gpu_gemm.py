"""Parity of the scaled fp8 GEMM with the oracle's emulated matmul (tolerance stated in helpers.py) and
exactness on integer-valued operands."""

import pytest
import torch

from helpers import E4M3, E5M2, assert_gemm_close, seeded
from oracle import float8_oracle as O

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import ops  # noqa: E402


def _variants():
    return list(range(len(ops.gemm_variants())))


def _gemm(a, sa, b, sb, variant, **kw):
    """Run one variant; returns None where the variant documents that it does not take the shape."""
    from olmo_core_amd.exceptions import MI8KernelError

    try:
        return ops.gemm_fp8(a, sa, b, sb, variant=variant, **kw)
    except MI8KernelError as e:
        if "direct-to-LDS variant needs" in str(e) or "few-rows variant takes" in str(e):
            return None
        raise


def _int_operand(shape, seed, dtype):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(-2, 3, shape, generator=g).float().to(dtype)


EXACT_SHAPES = [(32, 32, 64), (1, 16, 16), (33, 48, 144), (256, 256, 128), (300, 272, 1040), (257, 513, 4096), (512, 768, 16),
                (264, 520, 384), (256, 256, 256), (1024, 768, 1152), (2304, 2816, 128),
                # a few rows of A: the kernel that streams B once (K split over eight waves, ragged N and K)
                (1, 4096, 4096), (7, 1000, 2064), (16, 24, 16), (17, 40, 1040), (48, 1032, 4096), (64, 528, 11008)]


@pytest.mark.parametrize("mnk", EXACT_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_integer_operands_exact(dev, mnk):
    """Operands in {-2..2}: every product and partial sum is an integer below 2^24, so fp32 accumulation in any
    order is exact and the output must equal the integer matmul exactly - any wrong index, dropped k-chunk or
    mis-mapped accumulator register changes the result."""
    M, N, K = mnk
    one = torch.ones(1, device=dev)
    for da, db in ((E4M3, E4M3), (E5M2, E4M3), (E4M3, E5M2), (E5M2, E5M2)):
        a = _int_operand((M, K), 1, da)
        b = _int_operand((N, K), 2, db)
        ref = a.float() @ b.float().t()
        for v in _variants():
            out = _gemm(a.to(dev), one, b.to(dev), one, v, out_dtype=torch.float32)
            if out is None:
                continue
            assert torch.equal(out.cpu(), ref), f"variant {ops.gemm_variants()[v]} {da} x {db}: max diff {(out.cpu() - ref).abs().max()}"


@pytest.mark.parametrize("mnk", [(520, 776, 256), (2088, 1032, 384), (256, 264, 128)], ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("vec", [False, True], ids=["single-scales", "scale-vectors"])
def test_persistent_kernel_pitched_output(dev, mnk, vec):
    """The persistent kernel writes its tiles through buffer stores addressed from the tile's origin: an output with a
    row pitch wider than N, M and N that are not multiples of 256 (the last tile row / column is shifted back over the
    previous one).  Integer operands and power-of-two scales: exact; the columns past N keep what they held."""
    M, N, K = mnk
    a, b = _int_operand((M, K), 70 + M, E4M3), _int_operand((N, K), 71 + N, E5M2)
    g = torch.Generator().manual_seed(72)
    if vec:
        sa, sb = 2.0 ** torch.randint(-3, 4, (M,), generator=g).float(), 2.0 ** torch.randint(-3, 4, (N,), generator=g).float()
        want = a.float() @ b.float().t() / sa[:, None] / sb[None, :]
    else:
        sa, sb = torch.tensor([4.0]), torch.tensor([0.5])
        want = a.float() @ b.float().t() / 2.0
    kM16 = ops.gemm_variants().index("256x256_dma_w4x128_m16x128")
    wide = torch.full((M, N + 24), 7.0, dtype=torch.bfloat16, device=dev)
    res = ops.gemm_fp8(a.to(dev), sa.to(dev), b.to(dev), sb.to(dev), out=wide[:, :N], variant=kM16)
    assert res.data_ptr() == wide.data_ptr()
    assert torch.equal(wide[:, :N].float().cpu(), want.bfloat16().float())
    assert bool((wide[:, N:] == 7.0).all())


@pytest.mark.parametrize("M", [1, 5, 16, 31, 64])
def test_few_rows_scales_and_outputs(dev, M):
    """The default route for M <= 64: every mix of single scales and scale vectors, both output types, padded row
    pitches; integer operands and power-of-two scales make the expected result exact."""
    N, K, lda, ldb, ldc = 200, 400, 448, 416, 208
    g = torch.Generator().manual_seed(40 + M)
    a = torch.zeros(M, lda)
    a[:, :K] = torch.randint(-2, 3, (M, K), generator=g).float()
    a[:, K:] = 3.0  # bytes past K must not be read into the sum
    b = torch.zeros(N, ldb)
    b[:, :K] = torch.randint(-2, 3, (N, K), generator=g).float()
    b[:, K:] = 3.0
    ref = a[:, :K] @ b[:, :K].t()
    aq, bq = a.to(E5M2).to(dev)[:, :K], b.to(E4M3).to(dev)[:, :K]
    sa_v = (2.0 ** torch.randint(-3, 4, (M,), generator=g).float())
    sb_v = (2.0 ** torch.randint(-3, 4, (N,), generator=g).float())
    for sa, sb in ((torch.tensor([4.0]), torch.tensor([0.5])), (sa_v, sb_v), (sa_v, torch.tensor([2.0])),
                   (torch.tensor([0.25]), sb_v)):
        want = ref / (sa[:, None] if sa.numel() > 1 else sa) / (sb[None, :] if sb.numel() > 1 else sb)
        for dt in (torch.float32, torch.bfloat16):
            out = torch.full((M, ldc), 7.0, device=dev, dtype=dt)
            res = ops.gemm_fp8(aq, sa.to(dev), bq, sb.to(dev), out_dtype=dt, out=out[:, :N])
            assert res.data_ptr() == out.data_ptr()
            assert torch.equal(out[:, :N].float().cpu(), want.to(dt).float())
            assert bool((out[:, N:] == 7.0).all())  # nothing stored past column N


@pytest.mark.parametrize("mnk", [(100, 200, 1040), (257, 130, 4096), (64, 72, 256), (130, 1000, 2048)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("splits", [2, 3, 8])
def test_split_k_exact(dev, mnk, splits):
    """K cut into slices that are summed separately and added in slice order: integer operands make every slice
    and their sum exact, so a slice that is dropped, counted twice or cut at the wrong byte changes the result.
    Scale vectors of powers of two, both output types, an output with padded rows."""
    M, N, K = mnk
    splits = min(splits, (K + 127) // 128)
    g = torch.Generator().manual_seed(M + splits)
    a, b = _int_operand((M, K), 11, E5M2), _int_operand((N, K), 12, E4M3)
    sa = (2.0 ** torch.randint(-3, 4, (M,), generator=g).float())
    sb = (2.0 ** torch.randint(-3, 4, (N,), generator=g).float())
    ref = (a.float() @ b.float().t())
    for sa_t, sb_t in ((torch.ones(1), torch.ones(1)), (sa, sb)):
        want = ref / (sa_t[:, None] if sa_t.numel() > 1 else sa_t) / (sb_t[None, :] if sb_t.numel() > 1 else sb_t)
        for dt in (torch.float32, torch.bfloat16):
            out = torch.full((M, N + 8), 7.0, device=dev, dtype=dt)
            ops.gemm_fp8(a.to(dev), sa_t.to(dev), b.to(dev), sb_t.to(dev), out_dtype=dt, out=out[:, :N], splits=splits)
            assert torch.equal(out[:, :N].float().cpu(), want.to(dt).float()), (dt, sa_t.numel())
            assert bool((out[:, N:] == 7.0).all())
    # the library's own choice for the shape gives the same numbers
    auto = ops.gemm_fp8(a.to(dev), sa.to(dev), b.to(dev), sb.to(dev), out_dtype=torch.float32)
    assert torch.equal(auto.cpu(), ref / sa[:, None] / sb[None, :])


def test_split_k_matches_single_pass_on_real_data(dev):
    """Random operands: the sliced sum differs from the single-pass sum only by fp32 summation order."""
    M, N, K = 384, 1024, 4096
    a, b = seeded((M, K), 5).to(E4M3).to(dev), seeded((N, K), 6).to(E4M3).to(dev)
    one = torch.ones(1, device=dev)
    whole = ops.gemm_fp8(a, one, b, one, out_dtype=torch.float32, splits=1)
    cut = ops.gemm_fp8(a, one, b, one, out_dtype=torch.float32, splits=8)
    again = ops.gemm_fp8(a, one, b, one, out_dtype=torch.float32, splits=8)
    assert torch.equal(cut, again)  # fixed summation order
    assert float((cut - whole).abs().max()) <= 1e-4 * float(whole.abs().max())


def test_integer_operands_exact_padded_pitch(dev):
    """Row pitch larger than K (the zero-padded transposed copies): only the first K bytes of a row count."""
    M, N, K, ld = 100, 80, 112, 128
    a = torch.zeros(M, ld, dtype=E4M3); a[:, :K] = _int_operand((M, K), 3, E4M3); a[:, K:] = 1.0
    b = torch.zeros(N, ld, dtype=E4M3); b[:, :K] = _int_operand((N, K), 4, E4M3); b[:, K:] = 1.0
    ref = a[:, :K].float() @ b[:, :K].float().t()
    one = torch.ones(1, device=dev)
    for v in _variants():
        out = _gemm(a.to(dev), one, b.to(dev), one, v, k=K, out_dtype=torch.float32)
        if out is not None:
            assert torch.equal(out.cpu(), ref)


PARITY_SHAPES = [(64, 96, 128), (2048, 1024, 512), (300, 272, 1040), (128, 4096, 4096), (1000, 11008, 256), (520, 264, 2048)]


@pytest.mark.parametrize("mnk", PARITY_SHAPES, ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("gran", ["tensorwise", "axiswise"])
def test_against_emulated_mm(dev, mnk, gran):
    M, N, K = mnk
    x = seeded((M, K), seed=M + K, std=1.0)
    w = seeded((N, K), seed=N + 1, std=0.02)
    if gran == "tensorwise":
        a8, sa = O.cast(x, E4M3)
        b8, sb = O.cast(w, E4M3)
        ref = O.emulated_mm_f32(a8, sa, b8.t(), sb)
        sa_d, sb_d = sa.reshape(1).to(dev), sb.reshape(1).to(dev)
    else:
        a8, sa = O.cast(x, E4M3, O.AXISWISE, -1, True)
        b8, sb = O.cast(w, E4M3, O.AXISWISE, -1, True)
        ref = O.emulated_mm_f32(a8, sa, b8.t(), sb.t())
        sa_d, sb_d = sa.reshape(-1).to(dev), sb.reshape(-1).to(dev)
    for v in _variants():
        out = _gemm(a8.to(dev), sa_d, b8.to(dev), sb_d, v)
        if out is None:
            continue
        assert out.dtype == torch.bfloat16
        assert_gemm_close(out, ref, f"variant {v}")
        out32 = _gemm(a8.to(dev), sa_d, b8.to(dev), sb_d, v, out_dtype=torch.float32)
        if out32 is None:  # this variant only writes bf16
            continue
        assert_gemm_close(out32, ref, f"variant {v} f32")
        # bf16 output is the rounding of the fp32 output
        assert torch.equal(out32.bfloat16(), out)


def test_bf16_integer_exact_all_variants(dev):
    """bf16 output path (LDS-staged stores in the pipelined variant): integer results below 256 are exact in
    bf16, so the stored tile must equal the integer matmul element for element."""
    M, N, K = 520, 776, 128
    g = torch.Generator().manual_seed(9)
    a = (torch.randint(0, 2, (M, K), generator=g).float()).to(E4M3)
    b = (torch.randint(-1, 2, (N, K), generator=g).float()).to(E4M3)
    ref = a.float() @ b.float().t()
    assert ref.abs().max() < 256
    sa = (2.0 ** torch.randint(-2, 3, (M,), generator=g).float()).to(dev)
    sb = (2.0 ** torch.randint(-2, 3, (N,), generator=g).float()).to(dev)
    want = ref / sa.cpu()[:, None] / sb.cpu()[None, :]
    for v in _variants():
        out = _gemm(a.to(dev), sa, b.to(dev), sb, v)
        if out is not None:
            assert torch.equal(out.float().cpu(), want.bfloat16().float()), ops.gemm_variants()[v]


@pytest.mark.parametrize("K", [128, 256, 384])
def test_many_short_tiles_per_workgroup_exact(dev, K):
    """More tiles than six per compute unit, one to three K steps each, scale vectors: the persistent kernels
    switch tiles (operand prefetch, scale hand-over, epilogue) every few steps.  Integer data and power-of-two
    scales make the expected bf16 output exact."""
    M, N = 8192, 12288
    g = torch.Generator().manual_seed(31 + K)
    a = (torch.randint(0, 2, (M, K), generator=g).float())
    b = (torch.randint(-1, 2, (N, K), generator=g).float())
    a[:, K // 2:] = 0  # keeps |sum| below 256 for every K
    ref = a @ b.t()
    assert ref.abs().max() < 256
    sa = (2.0 ** torch.randint(-2, 3, (M,), generator=g).float())
    sb = (2.0 ** torch.randint(-2, 3, (N,), generator=g).float())
    want = (ref / sa[:, None] / sb[None, :]).bfloat16()
    out = ops.gemm_fp8(a.to(E4M3).to(dev), sa.to(dev), b.to(E4M3).to(dev), sb.to(dev))
    assert torch.equal(out.cpu(), want)
    one = torch.ones(1, device=dev)
    out1 = ops.gemm_fp8(a.to(E4M3).to(dev), one, b.to(E4M3).to(dev), one)
    assert torch.equal(out1.cpu(), ref.bfloat16())


def test_scaled_mm_library_crosscheck(dev):
    """Tensorwise case against torch-CPU's own _scaled_mm (library routine)."""
    x = seeded((96, 256), 1)
    w = seeded((160, 256), 2, std=0.02)
    a8, sa = O.cast(x, E4M3)
    b8, sb = O.cast(w, E4M3)
    ref = torch._scaled_mm(a8, b8.t(), scale_a=sa.reciprocal(), scale_b=sb.reciprocal(), out_dtype=torch.float32)
    out = ops.gemm_fp8(a8.to(dev), sa.reshape(1).to(dev), b8.to(dev), sb.reshape(1).to(dev), out_dtype=torch.float32)
    assert_gemm_close(out, ref)


def test_mixed_dtypes_gradient_shapes(dev):
    """e5m2 x e4m3 with a long, padded K: the grad_weight call shape."""
    M_tok, N, K = 1000, 272, 144
    go = seeded((M_tok, N), 5, std=1e-3)
    x = seeded((M_tok, K), 6)
    go8, sg = O.cast(go, E5M2)
    x8, sx = O.cast(x, E4M3)
    ref = O.emulated_mm_f32(go8.t(), sg, x8, sx)
    ld = ops.pad16(M_tok)
    a = torch.zeros(N, ld, dtype=E5M2); a[:, :M_tok] = go8.t()
    b = torch.zeros(K, ld, dtype=E4M3); b[:, :M_tok] = x8.t()
    out = ops.gemm_fp8(a.to(dev), sg.reshape(1).to(dev), b.to(dev), sx.reshape(1).to(dev), out_dtype=torch.float32)
    assert_gemm_close(out, ref)


def test_full_size_row_sample(dev):
    """7B MLP up-projection at full size (16384 x 11008 x 4096): a sample of output rows against the oracle."""
    M, N, K = 16384, 11008, 4096
    x = seeded((M, K), 1002)
    w = seeded((N, K), 1003, std=0.02)
    xq, _, sx = ops.cast_tensorwise(x.to(dev), E4M3)
    wq, _, sw = ops.cast_tensorwise(w.to(dev), E4M3)
    out = ops.gemm_fp8(xq, sx, wq, sw)
    rows = torch.arange(5, M, 1021)
    ref = O.emulated_mm_f32(xq[rows.to(dev)].cpu(), sx.cpu()[0], wq.cpu().t(), sw.cpu()[0])
    assert_gemm_close(out[rows.to(dev)], ref, "row sample")
    # linearity in the scales: doubling a scale halves the output exactly (power of two)
    out2 = ops.gemm_fp8(xq, sx * 2, wq, sw)
    assert torch.equal(out2[rows.to(dev)].float() * 2, out[rows.to(dev)].float())


@pytest.mark.parametrize("shape", [(16384, 4096, 11008), (11008, 4096, 16384), (4096, 11008, 16384)],
                         ids=lambda s: "x".join(map(str, s)))
def test_full_size_gradient_shapes_row_sample(dev, shape):
    """The grad_input and grad_weight GEMMs of the 7B MLP at full size (e5m2 left operand, as grad_output is cast):
    a sample of output rows against the oracle, for the default kernel and every persistent variant that
    takes the shape held to the same bar."""
    M, N, K = shape
    a = seeded((M, K), 2001, std=1e-3)
    b = seeded((N, K), 2002)
    aq, _, sa = ops.cast_tensorwise(a.to(dev), E5M2)
    bq, _, sb = ops.cast_tensorwise(b.to(dev), E4M3)
    out = ops.gemm_fp8(aq, sa, bq, sb)
    rows = torch.arange(3, M, max(M // 13, 1))
    ref = O.emulated_mm_f32(aq[rows.to(dev)].cpu(), sa.cpu()[0], bq.cpu().t(), sb.cpu()[0])
    assert_gemm_close(out[rows.to(dev)], ref, "row sample")
    names = ops.gemm_variants()
    for v, name in enumerate(names):
        if "dma" in name and "k64" not in name:
            other = ops.gemm_fp8(aq, sa, bq, sb, variant=v)
            # (the fp32 summation order inside a 128-byte K step differs between the MFMA shapes)
            assert_gemm_close(other[rows.to(dev)], ref, name)


def test_argument_errors(dev):
    from olmo_core_amd.exceptions import MI8KernelError

    a = torch.zeros(16, 24, dtype=E4M3, device=dev)
    one = torch.ones(1, device=dev)
    with pytest.raises(MI8KernelError):
        ops.gemm_fp8(a, one, a, one)  # K not a multiple of 16
    with pytest.raises(TypeError):
        ops.gemm_fp8(a.view(torch.uint8), one, a, one)
    with pytest.raises(ValueError):
        ops.gemm_fp8(torch.zeros(16, 32, dtype=E4M3, device=dev), torch.ones(3, device=dev), a, one)
    b = torch.zeros(16, 256, dtype=E4M3, device=dev)
    with pytest.raises(MI8KernelError, match="splits"):
        ops.gemm_fp8(b, one, b, one, splits=3)  # more slices than 128-byte K steps
    L = ops._C.lib()
    assert L.mi8_gemm_splitk_workspace_bytes(100, 30, 4) == 4 * 100 * 32 * 4
    assert L.mi8_gemm_splitk_suggest(16384, 11008, 4096) == 1 and L.mi8_gemm_splitk_suggest(256, 4096, 11008) > 1
    small = torch.empty(64, dtype=torch.uint8, device=dev)
    out = torch.empty(16, 16, dtype=torch.bfloat16, device=dev)
    rc = L.mi8_gemm_fp8_splitk(b.data_ptr(), 0, 256, b.data_ptr(), 0, 256, 16, 16, 256, one.data_ptr(), 0, one.data_ptr(), 0,
                               out.data_ptr(), 0, 16, 2, small.data_ptr(), small.numel(), 0)
    assert rc != 0 and b"workspace" in L.mi8_last_error()


@pytest.mark.parametrize("shape", [(512, 768, 256), (1024, 512, 1152), (300, 272, 144), (64, 512, 256), (2048, 2048, 128),
                                   (256, 1024, 4096), (128, 4096, 2816)],
                         ids=lambda s: "x".join(map(str, s)))
@pytest.mark.parametrize("vec", [False, True], ids=["single-scales", "scale-vectors"])
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32], ids=["bf16", "f32"])
def test_accumulating_gemm_equals_gemm_plus_add(dev, shape, vec, out_dtype):
    """out += product: the bits of `out + gemm(...)` on tensors of the output type (the new term rounded first, the
    sum formed in float32 and rounded once), on the persistent kernel (full 256-tiles), on the general one, and for
    shapes with few tiles and a long K, which the plain call sums in slices of K (the last two shapes)."""
    M, N, K = shape
    a, b = seeded((M, K), 31, std=1e-3), seeded((N, K), 32)
    if vec:
        aq, sa = ops.cast_rowwise(a.to(dev), E4M3, pow2=True)
        bq, sb = ops.cast_rowwise(b.to(dev), E4M3, pow2=True)
    else:
        aq, _, sa = ops.cast_tensorwise(a.to(dev), E5M2)
        bq, _, sb = ops.cast_tensorwise(b.to(dev), E4M3)
    first = (seeded((M, N), 33, std=1e-3 * K ** 0.5).float()).to(out_dtype).to(dev)
    first[0, 0] = float("inf")
    first[1, 1] = -0.0
    term = ops.gemm_fp8(aq, sa, bq, sb, out_dtype=out_dtype)
    want = first + term
    got = first.clone()
    res = ops.gemm_fp8(aq, sa, bq, sb, out_dtype=out_dtype, out=got, accumulate=True)
    assert res.data_ptr() == got.data_ptr()
    assert torch.equal(got.view(torch.int16 if out_dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if out_dtype == torch.bfloat16 else torch.int32))
    # a view with a row pitch: only the addressed columns change
    if out_dtype == torch.bfloat16:
        wide = torch.full((M, N + 64), 7.0, dtype=out_dtype, device=dev)
        wide[:, :N] = first
        ops.gemm_fp8(aq, sa, bq, sb, out_dtype=out_dtype, out=wide[:, :N], accumulate=True)
        assert torch.equal(wide[:, :N], want) and bool((wide[:, N:] == 7.0).all())
    with pytest.raises(ValueError):
        ops.gemm_fp8(aq, sa, bq, sb, out_dtype=out_dtype, accumulate=True)

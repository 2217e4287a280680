"""Ragged grouped float8 kernels (dropless-MoE expert layer) against the oracle's per-expert loop."""

import pytest
import torch

from helpers import E4M3, assert_bytes_equal, assert_gemm_close, assert_scale_equal, gemm_errors, seeded, u8
from oracle import float8_oracle as O
from oracle import moe_oracle as MO

pytestmark = pytest.mark.gpu

from olmo_core_amd.float8 import ops  # noqa: E402
from olmo_core_amd.nn import DroplessMoEMLP, ParallelDroplessMLP  # noqa: E402

SIZE_CASES = [
    [3, 2],
    [5, 0, 9, 2],
    [0, 0, 7],
    [130, 1, 0, 255, 128],
    [300, 17, 0, 0, 411, 64],
    # more groups than a wave has lanes: the tile -> group search carries its sums from one 64-group chunk to the next
    [(i * 37) % 23 if i % 5 else 0 for i in range(150)] + [200],
]


def _case_id(sizes):
    return "-".join(map(str, sizes)) if len(sizes) <= 8 else f"{len(sizes)}groups"


def _padded_starts(sizes):
    starts, tiles = [], 0
    for m in sizes:
        starts.append(128 * tiles)
        tiles += (m + 127) // 128
    return starts


@pytest.mark.parametrize("sizes", SIZE_CASES, ids=_case_id)
def test_grouped_colwise_cast_bit_exact(dev, sizes):
    T, C = sum(sizes), 144
    x = seeded((T, C), 3, std=0.3)
    x[:, 1] = 0
    q_t, scale = ops.grouped_cast_colwise_t(x.to(dev), torch.tensor(sizes), E4M3, pow2=True)
    assert q_t.shape == (C, ops.grouped_padded_rows(T, len(sizes)))
    start = 0
    for e, (m, p0) in enumerate(zip(sizes, _padded_starts(sizes))):
        if m == 0:
            continue
        ref_q, ref_s = O.cast(x[start:start + m], E4M3, O.AXISWISE, 0, True)
        assert_scale_equal(scale[e], ref_s, f"group {e} scales")
        assert_bytes_equal(q_t[:, p0:p0 + m], ref_q.t(), what=f"group {e} bytes")
        pad_end = p0 + 128 * ((m + 127) // 128)
        if pad_end > p0 + m:
            assert int(u8(q_t[:, p0 + m:pad_end]).max()) == 0, "segment padding must be zero"
        start += m


@pytest.mark.parametrize("pow2", [True, False], ids=["pow2", "exact"])
@pytest.mark.parametrize("sizes", SIZE_CASES, ids=_case_id)
def test_rows_and_grouped_colwise_cast_bit_exact(dev, sizes, pow2):
    """The two-product cast gives the oracle's per-row cast of the whole tensor and its per-expert per-column cast,
    and is byte-identical to the two single-product entry points."""
    T, C = sum(sizes), 272
    x = seeded((T, C), 11, std=0.3)
    x[:, 1] = 0
    x[T // 2] = 0
    xd = x.to(dev)
    q, rs, q_t, cs = ops.grouped_cast_rows_and_colwise_t(xd, torch.tensor(sizes), E4M3, pow2=pow2)
    ref_q, ref_s = O.cast(x, E4M3, O.AXISWISE, -1, pow2)
    assert_scale_equal(rs, ref_s.reshape(-1), "row scales")
    assert_bytes_equal(q, ref_q, what="row-major bytes")
    q_t1, cs1 = ops.grouped_cast_colwise_t(xd, torch.tensor(sizes), E4M3, pow2=pow2)
    start = 0
    for e, (m, p0) in enumerate(zip(sizes, _padded_starts(sizes))):
        if m == 0:
            continue
        ref_qc, ref_sc = O.cast(x[start:start + m], E4M3, O.AXISWISE, 0, pow2)
        assert_scale_equal(cs[e], ref_sc, f"group {e} column scales")
        assert_bytes_equal(q_t[:, p0:p0 + m], ref_qc.t(), what=f"group {e} transposed bytes")
        assert torch.equal(u8(q_t[:, p0:p0 + 128 * ((m + 127) // 128)]), u8(q_t1[:, p0:p0 + 128 * ((m + 127) // 128)]))
        assert torch.equal(cs[e], cs1[e])
        start += m


@pytest.mark.parametrize("sizes", SIZE_CASES, ids=_case_id)
def test_grouped_swiglu_with_amax_matches_separate_kernels(dev, sizes):
    """The group-aware SwiGLU kernels write the bytes of the flat ones, and the cast that takes their amax
    workspace gives the bytes and scales of the cast that computes the amax itself (forward and backward)."""
    T, C = sum(sizes), 272
    x1, x2, gh = (seeded((T, C), s, std=1.0).to(dev) for s in (21, 22, 23))
    sz = torch.tensor(sizes)
    h_ref, _ = ops.swiglu_fwd(x1, x2, want_amax=False)
    h, ws = ops.grouped_swiglu_fwd(x1, x2, sz)
    assert torch.equal(h.view(torch.int16), h_ref.view(torch.int16))
    want = ops.grouped_cast_rows_and_colwise_t(h_ref, sz, E4M3, pow2=True)
    got = ops.grouped_cast_rows_and_colwise_t(h, sz, E4M3, pow2=True, amax=ws)
    g1_ref, g2_ref, _, _ = ops.swiglu_bwd(x1, x2, gh, want_amax=False)
    g1, g2, ws1, ws2 = ops.grouped_swiglu_bwd(x1, x2, gh, sz)
    assert torch.equal(g1.view(torch.int16), g1_ref.view(torch.int16))
    assert torch.equal(g2.view(torch.int16), g2_ref.view(torch.int16))
    pairs = [(want, got)]
    for g_ref, g, w in ((g1_ref, g1, ws1), (g2_ref, g2, ws2)):
        pairs.append((ops.grouped_cast_rows_and_colwise_t(g_ref, sz, E4M3, pow2=True),
                      ops.grouped_cast_rows_and_colwise_t(g, sz, E4M3, pow2=True, amax=w)))
    for want, got in pairs:
        (q, rs, q_t, cs), (q2, rs2, q_t2, cs2) = want, got
        assert torch.equal(u8(q), u8(q2)) and torch.equal(rs, rs2)
        for e, (m, p0) in enumerate(zip(sizes, _padded_starts(sizes))):
            if m:
                seg = slice(p0, p0 + 128 * ((m + 127) // 128))
                assert torch.equal(u8(q_t[:, seg]), u8(q_t2[:, seg])) and torch.equal(cs[e], cs2[e])


@pytest.mark.parametrize("sizes", SIZE_CASES, ids=_case_id)
def test_grouped_gemm_exact_integers(dev, sizes):
    """Integer operands: the grouped forward GEMM must reproduce the per-expert integer matmul exactly, for both
    weight layouts (stacked rows / transposed with a column offset per expert)."""
    E, T, K, N = len(sizes), sum(sizes), 48, 80
    g = torch.Generator().manual_seed(4)
    a = torch.randint(-2, 3, (T, K), generator=g).float()
    w = torch.randint(-2, 3, (E, N, K), generator=g).float()
    ref = torch.cat([a[s:s + m] @ w[e].t() for e, (s, m) in enumerate(zip([sum(sizes[:i]) for i in range(E)], sizes))]) if T else None
    sz = torch.tensor(sizes).to(dev)
    ones_t, ones_n = torch.ones(T, device=dev), torch.ones(E * N, device=dev)
    b = w.reshape(E * N, K).to(E4M3).to(dev)
    out = ops.grouped_gemm_fp8(a.to(E4M3).to(dev), ones_t, b, ones_n, sz, n=N, k=K, b_group_stride=N * K,
                               sb_group_stride=N, out_dtype=torch.float32)
    assert torch.equal(out.cpu(), ref)
    # transposed-grouped layout: [N, E*K] with expert e at column offset e*K
    bt = w.permute(1, 0, 2).reshape(N, E * K).contiguous().to(E4M3).to(dev)
    out2 = ops.grouped_gemm_fp8(a.to(E4M3).to(dev), ones_t, bt, ones_n, sz, n=N, k=K, b_group_stride=K,
                                sb_group_stride=N, out_dtype=torch.float32)
    assert torch.equal(out2.cpu(), ref)


@pytest.mark.parametrize("sizes", SIZE_CASES, ids=_case_id)
def test_grouped_wgrad_exact_integers(dev, sizes):
    E, T, N, Kl = len(sizes), sum(sizes), 48, 80
    g = torch.Generator().manual_seed(5)
    go = torch.randint(-2, 3, (T, N), generator=g).float().bfloat16()
    x = torch.randint(-2, 3, (T, Kl), generator=g).float().bfloat16()
    sz = torch.tensor(sizes).to(dev)
    # quantise with the grouped cast; power-of-two scales keep small integers exact
    got, sgo = ops.grouped_cast_colwise_t(go.to(dev), sz, E4M3, pow2=True)
    xt, sx = ops.grouped_cast_colwise_t(x.to(dev), sz, E4M3, pow2=True)
    out = ops.grouped_wgrad_fp8(got, sgo, xt, sx, sz, tokens=T, out_dtype=torch.float32).cpu()
    start = 0
    for e, m in enumerate(sizes):
        ref = go[start:start + m].float().t() @ x[start:start + m].float()
        assert torch.equal(out[e], ref), f"group {e} (size {m})"
        start += m


# group-size lists for the full-tile (256 x 256, persistent) kernels: T >= 256 with groups that end inside a
# tile, empty groups, a group larger than two tiles, a last tile that is shifted back to stay inside the matrix
BIG_SIZE_CASES = [
    [256, 256],
    [300, 17, 0, 0, 411, 64],
    [1, 255, 513, 0, 3],
    [0, 1000, 0],
    [5] * 70,
]


def _group_starts(sizes):
    return [sum(sizes[:i]) for i in range(len(sizes))]


@pytest.mark.parametrize("sizes", BIG_SIZE_CASES, ids=lambda s: "-".join(map(str, s[:6])))
@pytest.mark.parametrize("n,k", [(256, 128), (320, 384)])
def test_grouped_gemm_full_tiles_exact_integers(dev, sizes, n, k):
    """bf16 output, N >= 256, K % 128 == 0: integer operands give integer sums that fp32 holds exactly, so the
    result must equal the per-expert matmul rounded once to bf16; per-row and per-column power-of-two scales
    must come out exactly as well."""
    E, T = len(sizes), sum(sizes)
    g = torch.Generator().manual_seed(6)
    a = torch.randint(-2, 3, (T, k), generator=g).float()
    w = torch.randint(-2, 3, (E, n, k), generator=g).float()
    sa = torch.tensor([1.0, 2.0, 0.5, 4.0]).repeat((T + 3) // 4)[:T].contiguous()
    sb = torch.tensor([1.0, 0.25, 8.0]).repeat((E * n + 2) // 3)[:E * n].contiguous()
    ref = torch.cat([a[s:s + m] @ w[e].t() / sb[e * n:(e + 1) * n] for e, (s, m) in enumerate(zip(_group_starts(sizes), sizes))])
    ref = (ref / sa[:, None]).bfloat16()
    sz = torch.tensor(sizes).to(dev)
    b = w.reshape(E * n, k).to(E4M3).to(dev)
    out = ops.grouped_gemm_fp8(a.to(E4M3).to(dev), sa.to(dev), b, sb.to(dev), sz, n=n, k=k, b_group_stride=n * k,
                               sb_group_stride=n, out_dtype=torch.bfloat16)
    assert torch.equal(out.cpu(), ref)
    bt = w.permute(1, 0, 2).reshape(n, E * k).contiguous().to(E4M3).to(dev)
    out2 = ops.grouped_gemm_fp8(a.to(E4M3).to(dev), sa.to(dev), bt, sb.to(dev), sz, n=n, k=k, b_group_stride=k,
                                sb_group_stride=n, out_dtype=torch.bfloat16)
    assert torch.equal(out2.cpu(), ref)


@pytest.mark.parametrize("sizes", BIG_SIZE_CASES, ids=lambda s: "-".join(map(str, s[:6])))
def test_grouped_wgrad_full_tiles_exact_integers(dev, sizes):
    E, T, N, Kl = len(sizes), sum(sizes), 320, 272
    g = torch.Generator().manual_seed(7)
    go = torch.randint(-2, 3, (T, N), generator=g).float().bfloat16()
    x = torch.randint(-2, 3, (T, Kl), generator=g).float().bfloat16()
    sz = torch.tensor(sizes).to(dev)
    got, sgo = ops.grouped_cast_colwise_t(go.to(dev), sz, E4M3, pow2=True)
    xt, sx = ops.grouped_cast_colwise_t(x.to(dev), sz, E4M3, pow2=True)
    out = ops.grouped_wgrad_fp8(got, sgo, xt, sx, sz, tokens=T, out_dtype=torch.bfloat16).cpu()
    out32 = ops.grouped_wgrad_fp8(got, sgo, xt, sx, sz, tokens=T, out_dtype=torch.float32).cpu()
    for e, (s, m) in enumerate(zip(_group_starts(sizes), sizes)):
        ref = go[s:s + m].float().t() @ x[s:s + m].float()
        assert torch.equal(out32[e], ref), f"group {e} (size {m}), general kernel"
        assert torch.equal(out[e], ref.bfloat16()), f"group {e} (size {m})"


@pytest.mark.parametrize("sizes", BIG_SIZE_CASES + [[4000, 0, 123, 2500]], ids=lambda s: "-".join(map(str, s[:6])))
def test_full_tile_kernels_match_general_kernels(dev, sizes):
    """Random data, arbitrary (not power-of-two) scales: the persistent full-tile kernels (bf16 output) and the
    general kernels (taken for fp32 output) accumulate in the same K order, so their results must agree
    bit for bit after one rounding to bf16."""
    E, T, n, k = len(sizes), sum(sizes), 320, 384
    g = torch.Generator().manual_seed(8)
    a = torch.randn(T, k, generator=g).to(E4M3).to(dev)
    w = torch.randn(E * n, k, generator=g).to(E4M3).to(dev)
    sa = (torch.rand(T, generator=g) + 0.5).to(dev)
    sb = (torch.rand(E * n, generator=g) + 0.5).to(dev)
    sz = torch.tensor(sizes).to(dev)
    kw = dict(n=n, k=k, b_group_stride=n * k, sb_group_stride=n)
    o16 = ops.grouped_gemm_fp8(a, sa, w, sb, sz, out_dtype=torch.bfloat16, **kw)
    o32 = ops.grouped_gemm_fp8(a, sa, w, sb, sz, out_dtype=torch.float32, **kw)
    assert torch.equal(o16, o32.bfloat16())
    go = torch.randn(T, n, generator=g).bfloat16().to(dev)
    x = torch.randn(T, k, generator=g).bfloat16().to(dev)
    got, sgo = ops.grouped_cast_colwise_t(go, sz, E4M3, pow2=False)
    xt, sx = ops.grouped_cast_colwise_t(x, sz, E4M3, pow2=False)
    w16 = ops.grouped_wgrad_fp8(got, sgo, xt, sx, sz, tokens=T, out_dtype=torch.bfloat16)
    w32 = ops.grouped_wgrad_fp8(got, sgo, xt, sx, sz, tokens=T, out_dtype=torch.float32)
    assert torch.equal(w16, w32.bfloat16())


def _moe_case(dev, E, D, H, sizes, seed=0):
    T = sum(sizes)
    x = seeded((T, D), seed + 1)
    go = seeded((T, D), seed + 2, std=1e-3)
    mlp = DroplessMoEMLP(d_model=D, hidden_size=H, num_experts=E, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(seed + 3)
    with torch.no_grad():
        for p in mlp.parameters():
            p.copy_((torch.randn(p.shape, generator=g) * 0.02).bfloat16())
    w1, w2, w3 = (p.detach().clone().view(E, H, D) for p in (mlp.w1, mlp.w2, mlp.w3))
    ref = O.dropless_mlp_fwd_bwd(x, w1, w2, w3, sizes, go, O.recipe("rowwise"))
    mlp = mlp.to(dev)
    xd = x.to(dev).requires_grad_(True)
    y = mlp(xd, torch.tensor(sizes).to(dev))
    y.backward(go.to(dev))
    return ref, y, xd.grad, mlp


def test_dropless_mlp_shape_contract(dev):
    """x [5,128], tokens_per_expert [3,2] -> [5,128] (reference: src/test/nn/moe/mlp_test.py:30-39)."""
    mlp = DroplessMoEMLP(d_model=128, hidden_size=256, num_experts=2, init_device="cuda", dtype=torch.bfloat16)
    x = torch.randn(5, 128, device=dev, dtype=torch.bfloat16)
    out = mlp(x, torch.tensor([3, 2], device=dev))
    assert out.shape == (5, 128)


@pytest.mark.parametrize("sizes", [[3, 2], [40, 0, 90, 7], [300, 17, 0, 0, 411, 64]], ids=_case_id)
@pytest.mark.parametrize("dims", [(128, 256), (256, 384), (128, 320)], ids=lambda d: f"{d[0]}x{d[1]}")
def test_dropless_mlp_against_oracle(dev, sizes, dims):
    E, (D, H) = len(sizes), dims
    if D >= 256 and sum(sizes) < 256:
        pytest.skip("the larger dimensions are there for the full-tile kernels, which need 256 rows")
    ref, y, gx, mlp = _moe_case(dev, E, D, H, sizes)
    # Compositions through re-quantised bf16 intermediates: cosine bar kept, max-error bar doubled (see
    # tests/test_gpu_mlp.py).  y itself goes through the re-quantised h; with the small H of the second case
    # its contraction averages over few fp8 codes, so it is held to the composition bar there.
    if H <= 256:
        assert_gemm_close(y, ref["y"], "y")
    for name, got, want in (
        ("y", y, ref["y"]),
        ("grad_x", gx, ref["grad_x"]),
        ("grad_w1", mlp.w1.grad.view(E, H, D), ref["grad_w1"]),
        ("grad_w2", mlp.w2.grad.view(E, H, D), ref["grad_w2"]),
        ("grad_w3", mlp.w3.grad.view(E, H, D), ref["grad_w3"]),
    ):
        rel, cos = gemm_errors(got, want)
        assert rel <= 2e-2 and cos >= 0.9999, (name, rel, cos)
    for e, m in enumerate(sizes):
        if m == 0:
            assert torch.count_nonzero(mlp.w1.grad.view(E, H, D)[e]) == 0
            assert torch.count_nonzero(mlp.w2.grad.view(E, H, D)[e]) == 0


@pytest.mark.parametrize("tokens,top_k", [(96, 2), (700, 4)])
def test_routed_layer_against_oracle(dev, tokens, top_k):
    """Router output -> sort -> gather -> experts -> weighted scatter (reference ParallelDroplessMLP,
    src/olmo_core/nn/moe/parallel_mlp.py:102-183, :851-871) against the oracle's composition: NumPy-loop
    permutation around the per-expert float8 emulation."""
    E, D, H = 8, 256, 384
    g = torch.Generator().manual_seed(11)
    x = seeded((tokens, D), 12)
    logits = torch.randn(tokens, E, generator=g)
    logits[:, 5] = -1e9  # an expert nobody picks
    scores = logits.softmax(-1)
    expert_weights, expert_indices = torch.topk(scores, top_k, dim=-1)
    expert_weights = expert_weights.bfloat16()
    sizes = O.batched_histc(expert_indices.reshape(1, -1), E)[0]
    go = seeded((tokens, D), 13, std=1e-2)

    mlp = DroplessMoEMLP(d_model=D, hidden_size=H, num_experts=E, dtype=torch.bfloat16)
    with torch.no_grad():
        for p_ in mlp.parameters():
            p_.copy_((torch.randn(p_.shape, generator=g) * 0.02).bfloat16())
    w1, w2, w3 = (p_.detach().clone().view(E, H, D) for p_ in (mlp.w1, mlp.w2, mlp.w3))

    # oracle: permutation loops + per-expert emulated float8 MLP (forward and grad_x through the same ops)
    indices, bin_ids, bins = MO.indices_and_bins(expert_indices, E)
    xs = MO.gather(x, indices, None, top_k)
    ref = O.dropless_mlp_fwd_bwd(xs, w1, w2, w3, sizes.tolist(), None, O.recipe("rowwise"))
    want = MO.scatter(ref["y"], indices, expert_weights.reshape(-1), top_k)

    layer = ParallelDroplessMLP(mlp=mlp.to(dev), top_k=top_k)
    xd = x.to(dev).requires_grad_(True)
    wd = expert_weights.to(dev).requires_grad_(True)
    out = layer(xd, wd, expert_indices.to(dev), sizes.to(dev))
    assert out.shape == x.shape
    rel, cos = gemm_errors(out, want)
    assert rel <= 2e-2 and cos >= 0.9999, (rel, cos)
    out.backward(go.to(dev))
    # gradients: the oracle's chain, scatter^T = weighted gather, then the experts' backward, then gather^T = scatter
    gys = MO.gather(go, indices, expert_weights.reshape(-1), top_k)
    refb = O.dropless_mlp_fwd_bwd(xs, w1, w2, w3, sizes.tolist(), gys, O.recipe("rowwise"))
    want_gx = MO.scatter(refb["grad_x"], indices, None, top_k)
    rel, cos = gemm_errors(xd.grad, want_gx)
    assert rel <= 3e-2 and cos >= 0.9995, ("grad_x", rel, cos)
    want_gw = MO.scatter_wgrad(ref["y"], go, indices, top_k).reshape(tokens, top_k)
    rel, cos = gemm_errors(wd.grad, want_gw)
    assert rel <= 3e-2 and cos >= 0.9995, ("grad_expert_weights", rel, cos)
    assert torch.count_nonzero(mlp.w1.grad.view(E, H, D)[5]) == 0


@pytest.mark.parametrize("sizes,dims", [([40, 0, 90, 7], (128, 256)), ([300, 17, 0, 0, 411, 64], (256, 384)),
                                        ([33, 150, 1], (128, 320))], ids=["4e-128x256", "6e-256x384", "3e-128x320"])
def test_dropless_mlp_stage_by_stage_against_oracle(dev, sizes, dims):
    """Every stage of the expert MLP against the oracle of that stage fed with the device's own bf16 input of the
    stage (stage_checks.check_dropless_stages), expert by expert.  A hidden size that is not a multiple of 128 is
    included: the transposed weight copies pad every expert to 128 columns."""
    from stage_checks import check_dropless_stages

    E, (D, H) = len(sizes), dims
    T = sum(sizes)
    mlp = DroplessMoEMLP(d_model=D, hidden_size=H, num_experts=E, dtype=torch.bfloat16)
    g = torch.Generator().manual_seed(3)
    with torch.no_grad():
        for i, p in enumerate(mlp.parameters()):
            p.copy_((torch.randn(p.shape, generator=g) * 0.02 * (1 + i)).bfloat16())
    check_dropless_stages(dev, mlp, seeded((T, D), 1), seeded((T, D), 2, std=1e-3), sizes, experts=range(E))


@pytest.mark.parametrize("tokens,top_k", [(96, 2), (700, 4)])
def test_routed_layer_fused_gather_equals_separate_gather(dev, tokens, top_k):
    """ParallelDroplessMLP with the gather fused into the quantisation of the expert inputs gives the bits of the
    layer that gathers first (outputs, grad_x, the router-weight gradient and every expert weight gradient)."""
    E, D, H = 8, 256, 384
    g = torch.Generator().manual_seed(21)
    x = seeded((tokens, D), 22)
    logits = torch.randn(tokens, E, generator=g)
    logits[:, 3] = -1e9
    expert_weights, expert_indices = torch.topk(logits.softmax(-1), top_k, dim=-1)
    sizes = O.batched_histc(expert_indices.reshape(1, -1), E)[0]
    go = seeded((tokens, D), 23, std=1e-2)
    mlp = DroplessMoEMLP(d_model=D, hidden_size=H, num_experts=E, dtype=torch.bfloat16)
    with torch.no_grad():
        for p_ in mlp.parameters():
            p_.copy_((torch.randn(p_.shape, generator=g) * 0.02).bfloat16())
    mlp = mlp.to(dev)
    results = []
    for fuse in (True, False):
        layer = ParallelDroplessMLP(mlp=mlp, top_k=top_k, fuse_gather=fuse)
        for p_ in mlp.parameters():
            p_.grad = None
        xd = x.to(dev).requires_grad_(True)
        wd = expert_weights.bfloat16().to(dev).requires_grad_(True)
        out = layer(xd, wd, expert_indices.to(dev), sizes.to(dev))
        out.backward(go.to(dev))
        results.append([out.detach(), xd.grad, wd.grad] + [p_.grad.clone() for p_ in mlp.parameters()])
    for name, a, b in zip(("out", "grad_x", "grad_expert_weights", "grad_w1", "grad_w2", "grad_w3"), *results):
        assert torch.equal(a, b), name


@pytest.mark.parametrize("sizes,n,k", [([300, 17, 0, 411, 64], 512, 256), ([5, 0, 9, 2], 48, 64), ([700, 1, 0, 323], 256, 1024),
                                       ([256, 256], 320, 128)], ids=["full-tiles", "small", "full-tiles-k1024", "n320"])
def test_accumulating_grouped_gemm_equals_gemm_plus_add(dev, sizes, n, k):
    T, E = sum(sizes), len(sizes)
    x = seeded((T, k), 41, std=1e-3)
    w = seeded((E * n, k), 42, std=0.05)
    sz = torch.tensor(sizes).to(dev)
    xq, sx = ops.cast_rowwise(x.to(dev), E4M3, pow2=True)
    wq, sw = ops.cast_rowwise(w.to(dev), E4M3, pow2=True)
    kw = dict(n=n, k=k, b_group_stride=n * wq.stride(0), sb_group_stride=n)
    term = ops.grouped_gemm_fp8(xq, sx, wq, sw, sz, **kw)
    first = seeded((T, n), 43, std=1e-3).to(dev)
    want = first + term
    got = ops.grouped_gemm_fp8(xq, sx, wq, sw, sz, accumulate_into=first.clone(), **kw)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_kept_expert_weight_operands(dev):
    """keep_float8_weights: the float8 copies of the expert weights are made once and reused until a weight changes;
    results are the bits of a module that quantises on every call."""
    E, D, H, sizes = 4, 256, 384, [300, 0, 170, 42]
    T = sum(sizes)
    x, go = seeded((T, D), 51).to(dev), seeded((T, D), 52, std=1e-3).to(dev)
    sz = torch.tensor(sizes).to(dev)
    g = torch.Generator().manual_seed(53)
    mods = []
    for keep in (False, True):
        m = DroplessMoEMLP(d_model=D, hidden_size=H, num_experts=E, dtype=torch.bfloat16, keep_float8_weights=keep)
        g.manual_seed(53)
        with torch.no_grad():
            for p_ in m.parameters():
                p_.copy_((torch.randn(p_.shape, generator=g) * 0.02).bfloat16())
        mods.append(m.to(dev))
    plain, kept = mods
    assert plain.weight_operands() is None

    def run(m):
        for p_ in m.parameters():
            p_.grad = None
        xd = x.clone().requires_grad_(True)
        y = m(xd, sz)
        y.backward(go)
        return [y.detach(), xd.grad] + [p_.grad.clone() for p_ in m.parameters()]

    for a, b in zip(run(plain), run(kept)):
        assert torch.equal(a, b)
    first = kept.weight_operands()
    assert first is kept.weight_operands(), "unchanged weights: the same copies are handed out"
    for a, b in zip(run(plain), run(kept)):  # second call on kept copies
        assert torch.equal(a, b)
    with torch.no_grad():  # an optimizer step: in-place updates move the version counters
        for m in mods:
            m.w1.mul_(1.5)
            m.w2.add_(0.01)
    assert kept.weight_operands() is not first
    for a, b in zip(run(plain), run(kept)):
        assert torch.equal(a, b)


DUAL_SIZE_CASES = [[300, 17, 0, 411, 64], [256], [1, 0, 0, 255, 513], [0, 1000, 0], [5] * 70, [700, 1, 0, 323, 2048, 9]]


@pytest.mark.parametrize("sizes", DUAL_SIZE_CASES, ids=lambda s: "-".join(map(str, s[:6])))
@pytest.mark.parametrize("n,k1,k2", [(256, 256, 256), (320, 512, 256), (512, 256, 1024)])
def test_grouped_dual_gemm_exact_integers(dev, sizes, n, k1, k2):
    """out = a1 . B1_e^T / sa1 / sb1_e + a2 . B2_e^T / sa2 / sb2_e in one accumulation.  Small-integer operands and
    power-of-two scales (different for the two products, per row and per column): every partial sum is exact in
    float32, so the result must equal the float64 evaluation rounded once to bf16 - any wrong operand window, scale
    vector, group or segment switch changes an integer."""
    E, T = len(sizes), sum(sizes)
    g = torch.Generator().manual_seed(16)
    a1 = torch.randint(-2, 3, (T, k1), generator=g).float()
    a2 = torch.randint(-2, 3, (T, k2), generator=g).float()
    w1 = torch.randint(-2, 3, (E, n, k1), generator=g).float()
    w2 = torch.randint(-2, 3, (E, n, k2), generator=g).float()
    pick = lambda vals, count, seed: torch.tensor(vals)[torch.randint(0, len(vals), (count,), generator=torch.Generator().manual_seed(seed))]  # noqa: E731
    sa1, sa2 = pick([1.0, 2.0, 0.5, 4.0, 64.0], T, 1), pick([1.0, 0.25, 8.0, 2.0 ** -7], T, 2)
    sb1, sb2 = pick([1.0, 0.25, 8.0], E * n, 3), pick([2.0, 0.5, 16.0, 2.0 ** 9], E * n, 4)
    starts = _group_starts(sizes)
    ref = torch.cat([
        (a1[s:s + m].double() @ w1[e].double().t()) / sb1[e * n:(e + 1) * n].double() / sa1[s:s + m, None].double()
        + (a2[s:s + m].double() @ w2[e].double().t()) / sb2[e * n:(e + 1) * n].double() / sa2[s:s + m, None].double()
        for e, (s, m) in enumerate(zip(starts, sizes))
    ]).float().bfloat16()
    sz = torch.tensor(sizes).to(dev)
    kmax = max(k1, k2)
    # operands of both products in buffers of one row pitch, as the entry point requires
    a_buf = torch.zeros((2, T, kmax), dtype=E4M3)
    a_buf[0, :, :k1], a_buf[1, :, :k2] = a1.to(E4M3), a2.to(E4M3)
    b_buf = torch.zeros((2, E * n, kmax), dtype=E4M3)
    b_buf[0, :, :k1], b_buf[1, :, :k2] = w1.reshape(E * n, k1).to(E4M3), w2.reshape(E * n, k2).to(E4M3)
    a_buf, b_buf = a_buf.to(dev), b_buf.to(dev)
    if not ops.grouped_gemm_dual_supported(T, n, k1, k2):
        with pytest.raises(Exception):
            ops.grouped_gemm_fp8_dual(a_buf[0, :, :k1], sa1.to(dev), b_buf[0, :, :k1], sb1.to(dev), a_buf[1, :, :k2], sa2.to(dev),
                                      b_buf[1, :, :k2], sb2.to(dev), sz, n=n, k1=k1, k2=k2, b_group_stride=n * kmax, sb_group_stride=n)
        return
    out = ops.grouped_gemm_fp8_dual(a_buf[0, :, :k1], sa1.to(dev), b_buf[0, :, :k1], sb1.to(dev), a_buf[1, :, :k2], sa2.to(dev),
                                    b_buf[1, :, :k2], sb2.to(dev), sz, n=n, k1=k1, k2=k2, b_group_stride=n * kmax, sb_group_stride=n)
    assert torch.equal(out.cpu(), ref)


@pytest.mark.parametrize("sizes", [[300, 17, 0, 411, 64], [700, 1, 0, 323, 2048, 9]], ids=lambda s: "-".join(map(str, s[:6])))
def test_grouped_dual_gemm_against_separate_products(dev, sizes):
    """Random operands through the product's casts (power-of-two scales): the single launch agrees with the sum of the
    two separate grouped GEMMs taken in float32 (same K order per product, one rounding instead of three) to within
    a bf16 rounding of each term, and with the float64 product of the dequantised operands at the single-GEMM bar."""
    E, T, n, k = len(sizes), sum(sizes), 512, 768
    sz = torch.tensor(sizes).to(dev)
    g1, g2 = seeded((T, k), 51, std=1e-3).to(dev), seeded((T, k), 52, std=3e-3).to(dev)
    w1, w2 = seeded((E * k, n), 53, std=0.02).to(dev), seeded((E * k, n), 54, std=0.3).to(dev)
    equal = torch.full((E,), k, dtype=torch.int64, device=dev)
    g1q, s1 = ops.cast_rowwise(g1, E4M3, pow2=True)
    g2q, s2 = ops.cast_rowwise(g2, E4M3, pow2=True)
    w1t, c1 = ops.grouped_cast_colwise_t(w1, equal, E4M3, pow2=True)  # [n, E * k]: group e's K columns, one scale per (e, column)
    w2t, c2 = ops.grouped_cast_colwise_t(w2, equal, E4M3, pow2=True)
    kw = dict(n=n, b_group_stride=k, sb_group_stride=n)
    got = ops.grouped_gemm_fp8_dual(g1q, s1, w1t, c1, g2q, s2, w2t, c2, sz, k1=k, k2=k, **kw)
    p1 = ops.grouped_gemm_fp8(g1q, s1, w1t, c1, sz, k=k, out_dtype=torch.float32, **kw)
    p2 = ops.grouped_gemm_fp8(g2q, s2, w2t, c2, sz, k=k, out_dtype=torch.float32, **kw)
    want = (p1 + p2)
    err = (got.float() - want).abs().max() / want.abs().max()
    assert float(err) <= 2.0 ** -8, float(err)  # one bf16 rounding of the sum
    # float64 on the host from the dequantised operands, group by group
    starts = _group_starts(sizes)
    for e, (s, m) in enumerate(zip(starts, sizes)):
        if m == 0:
            continue
        ref = 0
        for q, sr, wt, sc in ((g1q, s1, w1t, c1), (g2q, s2, w2t, c2)):
            a = q[s:s + m].float().double().cpu() / sr[s:s + m, None].double().cpu()
            b = wt[:, e * k:(e + 1) * k].float().double().cpu() / sc[e][:, None].double().cpu()
            ref = ref + a @ b.t()
        assert_gemm_close(got[s:s + m], ref, f"group {e}")

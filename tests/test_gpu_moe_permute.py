"""HIP token-permutation kernels against the NumPy-loop oracle (the loops of src/test/ops/moe_test.py:46-66 and
:125-145, restated in oracle/moe_oracle.py), on the reference's own parametrisations."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as M

pytestmark = pytest.mark.gpu

from olmo_core_amd.ops import moe as ops  # noqa: E402

# (sl, hs, ne, top_k): the grid of src/test/ops/moe_test.py:11-33 (every second size to keep the loops short)
REFERENCE_CASES = [
    (4, 2, 2, 1), (4, 2, 2, 2), (4, 2, 2, 4),
    (1024, 1536, 4, 1), (1024, 1536, 4, 4), (1024, 1536, 64, 2), (1024, 1536, 128, 4),
    (16384, 768, 4, 2), (16384, 768, 64, 1), (16384, 768, 128, 4),
]
SMALL_CASES = [(4, 2, 2, 1), (4, 2, 2, 2), (4, 2, 2, 4), (100, 24, 7, 3), (257, 136, 5, 2), (512, 2048, 64, 8)]
RTOL = 5e-3  # the reference's tolerance for sums whose order is not fixed (moe_test.py:147-155)


def _case(sl, hs, ne, top_k, dtype, seed=0):
    g = torch.Generator().manual_seed(seed + sl + top_k)
    x = torch.randn((sl, hs), generator=g).to(dtype)
    top_expert = torch.randint(0, ne, (sl, top_k), generator=g)
    indices, bin_ids, bins = M.indices_and_bins(top_expert, ne)
    weights = torch.rand((sl * top_k,), generator=g).to(dtype)
    return x, indices, bin_ids, bins, weights


def _close(got, want, exact):
    if exact:
        assert torch.equal(got.cpu(), want)
    else:
        np.testing.assert_allclose(got.float().cpu().numpy(), want.float().numpy(), rtol=RTOL, atol=1e-6)


@pytest.mark.parametrize("sl,hs,ne,top_k", REFERENCE_CASES, ids=lambda v: str(v))
def test_binned_gather_and_scatter_reference_grid(dev, sl, hs, ne, top_k):
    """test_binned_gather / test_binned_scatter of the reference: capacity factor 1, fp16."""
    ec = (sl * top_k) // ne
    x, indices, _, bins, weights = _case(sl, hs, ne, top_k, torch.float16)
    out = ops.binned_gather(x.to(dev), indices.to(dev), bins.to(dev), ec, top_k)
    expected = M.binned_gather(x, indices, None, bins, ec, top_k)
    assert torch.all(torch.eq(out.cpu(), expected))
    got = ops.binned_scatter(out, indices.to(dev), weights.to(dev), bins.to(dev), top_k)
    want = M.binned_scatter(expected, indices, weights, bins, top_k)
    _close(got, want, exact=top_k <= 2)  # a two-term float32 sum has one rounding whatever the order


@pytest.mark.parametrize("sl,hs,ne,top_k", SMALL_CASES + [(16384, 768, 64, 2)], ids=lambda v: str(v))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32], ids=["bf16", "f16", "f32"])
def test_dropless_gather_scatter_wgrad(dev, sl, hs, ne, top_k, dtype):
    x, indices, bin_ids, bins, weights = _case(sl, hs, ne, top_k, dtype, seed=1)
    d = lambda t: t.to(dev)  # noqa: E731
    y = ops._gather(d(x), d(indices), None, top_k)
    assert torch.equal(y.cpu(), M.gather(x, indices, None, top_k))
    yw = ops._gather(d(x), d(indices), d(weights), top_k)
    assert torch.equal(yw.cpu(), M.gather(x, indices, weights, top_k))
    yc = y.cpu()
    _close(ops._scatter(y, d(indices), d(weights), top_k), M.scatter(yc, indices, weights, top_k), exact=top_k <= 2)
    _close(ops._scatter(y, d(indices), None, top_k), M.scatter(yc, indices, None, top_k), exact=top_k <= 2)
    grad = torch.randn((sl, hs), generator=torch.Generator().manual_seed(2)).to(dtype)
    wg = ops._scatter_wgrad(y, d(grad), d(indices), top_k)
    want = M.scatter_wgrad(yc, grad, indices, top_k)
    np.testing.assert_allclose(wg.float().cpu().numpy(), want.float().numpy(), rtol=2e-2, atol=2e-2 * hs ** 0.5)


@pytest.mark.parametrize("ec", [1, 5, 40])
def test_binned_capacity_and_weight_gradient(dev, ec):
    sl, hs, ne, top_k = 96, 40, 8, 2
    x, indices, _, bins, weights = _case(sl, hs, ne, top_k, torch.bfloat16, seed=5)
    d = lambda t: t.to(dev)  # noqa: E731
    yw = ops._binned_gather(d(x), d(indices), d(weights), d(bins), ec, top_k)
    assert torch.equal(yw.cpu(), M.binned_gather(x, indices, weights, bins, ec, top_k))
    y = M.binned_gather(x, indices, None, bins, ec, top_k)
    got = ops._binned_scatter(d(y), d(indices), d(weights), d(bins), top_k)
    assert torch.equal(got.cpu(), M.binned_scatter(y, indices, weights, bins, top_k))
    grad = torch.randn((sl, hs), generator=torch.Generator().manual_seed(6)).bfloat16()
    wg = ops._binned_scatter_wgrad(d(y), d(grad), d(indices), d(bins), top_k)
    want = M.binned_scatter_wgrad(y, grad, indices, bins, top_k)
    np.testing.assert_allclose(wg.float().cpu().numpy(), want.float().numpy(), rtol=2e-2, atol=0.15)
    dropped = want == 0  # dropped slots are exactly zero on both sides
    assert torch.count_nonzero(wg.cpu()[dropped]) == 0


def test_fp8_rows_are_moved_as_bytes(dev):
    sl, hs, ne, top_k = 300, 256, 16, 4
    x, indices, _, bins, _ = _case(sl, hs, ne, top_k, torch.bfloat16, seed=7)
    q = (x * 8).to(torch.float8_e4m3fn)
    out = ops._gather(q.to(dev), indices.to(dev), None, top_k)
    assert torch.equal(out.cpu().view(torch.uint8), q.view(torch.uint8)[indices.long() // top_k])


def test_autograd_matches_reference_structure(dev):
    """gather's backward is the unweighted scatter; scatter's backward is the weighted gather plus the weight
    gradient (src/olmo_core/ops/moe.py:42-50, :84-112)."""
    sl, hs, ne, top_k = 64, 48, 4, 2
    x, indices, bin_ids, bins, weights = _case(sl, hs, ne, top_k, torch.float32, seed=8)
    d = lambda t: t.to(dev)  # noqa: E731
    xd = d(x).requires_grad_(True)
    wd = d(weights).requires_grad_(True)
    y = ops.gather(xd, d(indices), d(bin_ids), d(bins), top_k)
    out = ops.scatter(y, d(indices), d(bin_ids), wd, d(bins), top_k)
    go = torch.randn((sl, hs), generator=torch.Generator().manual_seed(3))
    out.backward(d(go))
    # dense restatement: out[t] = sum_j w[t*k+j] * x[t]  ->  dx[t] = go[t] * sum_j w[t,j], dw[t,j] = <x[t], go[t]>
    wsum = weights.view(sl, top_k).sum(1, keepdim=True)
    np.testing.assert_allclose(out.detach().cpu().numpy(), (x * wsum).numpy(), rtol=1e-5, atol=1e-6)
    np.testing.assert_allclose(xd.grad.cpu().numpy(), (go * wsum).numpy(), rtol=1e-5, atol=1e-6)
    want_w = (x * go).sum(1, keepdim=True).expand(sl, top_k).reshape(-1)
    np.testing.assert_allclose(wd.grad.cpu().numpy(), want_w.numpy(), rtol=1e-4, atol=1e-4)


def test_errors(dev):
    x = torch.zeros(4, 8)
    with pytest.raises(RuntimeError, match="GPU"):
        ops._gather(x, torch.zeros(4, dtype=torch.int32), None, 1)
    with pytest.raises(ValueError):
        ops._gather(x.to(dev), torch.zeros(3, dtype=torch.int32, device=dev), None, 1)
    # an index outside the slot range is dropped, not followed
    bad = torch.tensor([0, 1, 99, -5], dtype=torch.int32, device=dev)
    out = ops._gather(torch.ones(4, 8, device=dev), bad, None, 1)
    assert out.cpu().sum(1).tolist() == [8.0, 8.0, 0.0, 0.0]


@pytest.mark.parametrize("sl,hs,ne,top_k", [(100, 32, 7, 3), (257, 144, 5, 2), (700, 256, 8, 4), (2048, 512, 64, 8)],
                         ids=lambda v: str(v))
@pytest.mark.parametrize("pow2", [True, False], ids=["pow2", ""])
def test_gather_fused_with_the_grouped_cast(dev, sl, hs, ne, top_k, pow2):
    """gather -> quantise in one call: bytes and scales equal the two-call route (gather, then the grouped
    two-product cast) and the oracle (NumPy-loop gather, then the per-expert casts), the gathered bf16 tensor is never
    written.  An expert without tokens and an out-of-range slot index (a dropped token: a row of zeros) included."""
    from helpers import E4M3, assert_bytes_equal, assert_scale_equal, u8
    from olmo_core_amd.float8 import ops as f8
    from oracle import float8_oracle as O

    x, indices, _, bins, _ = _case(sl, hs, ne, top_k, torch.bfloat16, seed=3)
    if ne >= 5:  # route everything away from expert 2
        g = torch.Generator().manual_seed(9)
        top_expert = torch.randint(0, ne - 1, (sl, top_k), generator=g)
        top_expert[top_expert >= 2] += 1
        indices, _, bins = M.indices_and_bins(top_expert, ne)
    sizes = torch.diff(bins.long(), prepend=torch.zeros(1, dtype=torch.long))
    d = lambda t: t.to(dev)  # noqa: E731
    q, srow, q_t, scol = f8.gather_cast_rows_and_colwise_t(d(x), d(indices), top_k, d(sizes), E4M3, pow2=pow2)

    xs_dev = ops._gather(d(x), d(indices), None, top_k)
    q2, srow2, q_t2, scol2 = f8.grouped_cast_rows_and_colwise_t(xs_dev, d(sizes), E4M3, pow2=pow2)
    assert torch.equal(u8(q), u8(q2)) and torch.equal(srow.cpu(), srow2.cpu())

    xs = M.gather(x, indices, None, top_k)
    start = seg = 0
    for e, n in enumerate(sizes.tolist()):
        if n:
            xe = xs[start:start + n]
            ref_r, ref_sr = O.cast(xe, E4M3, O.AXISWISE, -1, pow2)
            ref_c, ref_sc = O.cast(xe, E4M3, O.AXISWISE, 0, pow2)
            assert_scale_equal(srow[start:start + n], ref_sr, f"expert {e}: row scales")
            assert_scale_equal(scol[e], ref_sc, f"expert {e}: column scales")
            assert_scale_equal(scol[e], scol2[e], f"expert {e}: column scales vs two-call route")
            assert_bytes_equal(q[start:start + n], ref_r, what=f"expert {e}: per-row bytes")
            assert_bytes_equal(q_t[:, seg:seg + n], ref_c.t(), what=f"expert {e}: per-column bytes")
            pad = (n + 127) // 128 * 128
            assert torch.equal(u8(q_t[:, seg:seg + pad]), u8(q_t2[:, seg:seg + pad])), f"expert {e}: transposed copy"
            seg += pad
        start += n

    # weighted: the rows of the weighted gather, quantised
    w = torch.rand((sl * top_k,), generator=torch.Generator().manual_seed(5)).to(torch.bfloat16)
    qw, srw, qtw, scw = f8.gather_cast_rows_and_colwise_t(d(x), d(indices), top_k, d(sizes), E4M3, pow2=pow2, weights=d(w))
    xw_dev = ops._gather(d(x), d(indices), d(w), top_k)
    assert torch.equal(xw_dev.cpu(), M.gather(x, indices, w, top_k))
    q2w, sr2w, qt2w, sc2w = f8.grouped_cast_rows_and_colwise_t(xw_dev, d(sizes), E4M3, pow2=pow2)
    assert torch.equal(u8(qw), u8(q2w)) and torch.equal(srw.cpu(), sr2w.cpu())
    seg = 0
    for e, n in enumerate(sizes.tolist()):
        if n:
            pad = (n + 127) // 128 * 128
            assert torch.equal(u8(qtw[:, seg:seg + pad]), u8(qt2w[:, seg:seg + pad])), f"expert {e}: weighted, transposed copy"
            assert_scale_equal(scw[e], sc2w[e], f"expert {e}: weighted, column scales")
            seg += pad

    # a slot index that points nowhere reads as a row of zeros (zero bytes; scale of an all-zero row)
    bad = indices.clone()
    bad[0] = sl * top_k + 5
    qb, srb, _, _ = f8.gather_cast_rows_and_colwise_t(d(x), d(bad), top_k, d(sizes), E4M3, pow2=pow2)
    assert int(u8(qb[0]).max()) == 0
    assert_scale_equal(srb[0:1], O.amax_to_scale(torch.zeros(1, 1, dtype=torch.bfloat16), E4M3, pow2))
    assert torch.equal(u8(qb[1:]), u8(q[1:]))

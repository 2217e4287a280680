"""The NumPy-loop oracle of the MoE permutation ops against an independent vectorised formulation, permutation
identities and the reference's known answers (CPU only)."""

import numpy as np
import pytest
import torch

from oracle import float8_oracle as O
from oracle import moe_oracle as M


def _case(sl, hs, ne, top_k, seed=0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((sl, hs), generator=g).to(dtype)
    top_expert = torch.randint(0, ne, (sl, top_k), generator=g)
    indices, bin_ids, bins = M.indices_and_bins(top_expert, ne)
    weights = torch.rand((sl * top_k,), generator=g).to(dtype)
    return x, top_expert, indices, bin_ids, bins, weights


def test_batched_histc_known_answer():
    """src/test/ops/moe_test.py:158-164"""
    x = torch.tensor([[0, 1, 1], [2, 0, 0]])
    assert torch.equal(O.batched_histc(x, 5), torch.tensor([[1, 2, 0, 0, 0], [2, 0, 1, 0, 0]]))


def test_indices_and_bins():
    top_expert = torch.tensor([[2, 0], [1, 2], [0, 0]])
    indices, bin_ids, bins = M.indices_and_bins(top_expert, 4)
    assert bin_ids.tolist() == [0, 0, 0, 1, 2, 2]
    assert indices.tolist() == [1, 4, 5, 2, 0, 3]  # stable: slot order inside an expert
    assert bins.tolist() == [3, 4, 6, 6]
    assert indices.dtype == torch.int32 and bins.dtype == torch.int32


@pytest.mark.parametrize("sl,hs,ne,top_k", [(4, 2, 2, 1), (4, 2, 2, 2), (64, 24, 4, 4), (128, 16, 16, 2)])
def test_gather_scatter_against_index_arithmetic(sl, hs, ne, top_k):
    x, _, indices, _, bins, weights = _case(sl, hs, ne, top_k)
    idx = indices.long()
    # gather: row i <- x[idx[i] // k] * w[idx[i]]
    want = (x.float()[idx // top_k] * weights.float()[idx][:, None]).to(x.dtype)
    assert torch.equal(M.gather(x, indices, weights, top_k), want)
    assert torch.equal(M.gather(x, indices, None, top_k), x[idx // top_k])
    # scatter: tmp[idx[i]] = y[i] * w[idx[i]]; out = sum over slots
    y = M.gather(x, indices, None, top_k)
    tmp = torch.zeros((sl * top_k, hs))
    tmp[idx] = (y.float() * weights.float()[idx][:, None]).to(x.dtype).float()
    want = tmp.view(sl, top_k, hs).sum(1).to(x.dtype)
    got = M.scatter(y, indices, weights, top_k)
    np.testing.assert_allclose(got.float().numpy(), want.float().numpy(), rtol=5e-3)
    # identity: scattering the gathered rows with unit weights gives top_k * x
    unit = M.scatter(y, indices, None, top_k)
    np.testing.assert_allclose(unit.float().numpy(), (top_k * x.float()).to(x.dtype).float().numpy(), rtol=5e-3)
    # weight gradient: slot s gets <y[row of s], grad[s // k]>
    grad = torch.randn((sl, hs), generator=torch.Generator().manual_seed(9)).to(x.dtype)
    inv = torch.empty_like(idx)
    inv[idx] = torch.arange(idx.numel())
    want = (y.double()[inv] * grad.double().repeat_interleave(top_k, 0)).sum(1)
    np.testing.assert_allclose(M.scatter_wgrad(y, grad, indices, top_k).double().numpy(), want.numpy(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("sl,hs,ne,top_k,ec", [(4, 2, 2, 1, 2), (64, 8, 4, 2, 32), (64, 8, 4, 2, 5), (32, 16, 8, 4, 40)])
def test_binned_against_dropless(sl, hs, ne, top_k, ec):
    """The binned layout is the dropless one cut into per-expert bins of `ec` rows: rows beyond the expert's
    count are zero, tokens beyond the capacity are dropped."""
    x, _, indices, bin_ids, bins, weights = _case(sl, hs, ne, top_k, seed=3)
    flat = M.gather(x, indices, weights, top_k)
    binned = M.binned_gather(x, indices, weights, bins, ec, top_k)
    assert binned.shape == (ne, ec, hs)
    start = 0
    kept = torch.zeros(sl * top_k, dtype=torch.bool)
    for e in range(ne):
        n = int(bins[e]) - start
        m = min(n, ec)
        assert torch.equal(binned[e, :m], flat[start:start + m])
        assert torch.count_nonzero(binned[e, m:]) == 0
        kept[indices[start:start + m].long()] = True
        start = int(bins[e])
    # scatter of the binned rows == dropless scatter with the dropped slots' weights set to zero
    y = M.binned_gather(x, indices, None, bins, ec, top_k)
    got = M.binned_scatter(y, indices, weights, bins, top_k)
    w0 = torch.where(kept, weights.float(), torch.zeros(())).to(weights.dtype)
    want = M.scatter(M.gather(x, indices, None, top_k), indices, w0, top_k)
    np.testing.assert_allclose(got.float().numpy(), want.float().numpy(), rtol=5e-3, atol=1e-6)
    grad = torch.randn((sl, hs), generator=torch.Generator().manual_seed(4)).to(x.dtype)
    wg = M.binned_scatter_wgrad(y, grad, indices, bins, top_k)
    wg_flat = M.scatter_wgrad(M.gather(x, indices, None, top_k), grad, indices, top_k)
    assert torch.equal(wg[kept], wg_flat[kept]) and torch.count_nonzero(wg[~kept]) == 0

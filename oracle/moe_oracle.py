"""
CPU restatement of the reference's MoE token-permutation ops.  TEST INFRASTRUCTURE ONLY: imported by tests/ and
nothing else; the product path is the HIP library.

The loops follow the reference's own NumPy oracles and kernels:

* ``binned_gather`` / ``binned_scatter``: the NumPy loops in ``src/test/ops/moe_test.py:46-66`` and ``:125-145``
  (capacity-limited copies), extended with the optional scale of ``src/olmo_core/kernels/moe.py:300-373``.
* ``gather`` / ``scatter`` / ``scatter_wgrad``: ``src/olmo_core/kernels/moe.py:40-139`` (``_padded_copy`` with
  ``padded_bins == bins``), ``:142-192`` (copy to ``[tokens, top_k, hidden]`` then ``sum(dim=1)``) and ``:195-298``.
* ``binned_scatter_wgrad``: ``kernels/moe.py:457-537``.
* ``batched_histc`` lives in ``oracle/float8_oracle.py`` (known answer ``src/test/ops/moe_test.py:158-164``).
* ``indices_and_bins``: ``src/olmo_core/nn/moe/parallel_mlp.py:102-125``.

Rounding points (as in the kernels): a product is formed in float32 from the two operands widened to float32 and
rounded once to the element type; the scatter sums the rounded terms of a token's slots (float32 accumulation in
torch's ``sum``; the order of that sum is not pinned by any reference vector, so sums are compared with the
tolerance the reference's own test uses, rtol 5e-3).

Pinned by: the loops being transcriptions of the reference's test oracles; ``tests/test_oracle_moe.py`` checks
them against an independent vectorised formulation (index arithmetic with torch ``index_select`` / ``index_add``),
against the permutation identities (scatter(gather(x)) == top_k * x for unit weights, gather with top_k == 1 is a
row permutation).
"""

from __future__ import annotations

from typing import Optional, Tuple

import numpy as np
import torch


def _round_to(a: np.ndarray, dtype: torch.dtype) -> np.ndarray:
    """float32 array -> values representable in ``dtype`` (round to nearest even), returned as float32."""
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).to(dtype).float().numpy()


def _f32(t: Optional[torch.Tensor]) -> Optional[np.ndarray]:
    return None if t is None else t.detach().float().cpu().numpy()


def indices_and_bins(expert_indices: torch.Tensor, num_experts: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """top-k expert assignment [tokens, top_k] -> (indices int32, bin_ids int32, bins int32)
    (parallel_mlp.py:102-125: flatten, stable sort, cumulative histogram)."""
    flat = expert_indices.reshape(-1).to(torch.int64)
    bin_ids, indices = torch.sort(flat, stable=True)
    hist = torch.bincount(flat, minlength=num_experts)
    bins = torch.cumsum(hist, 0)
    return indices.int(), bin_ids.int(), bins.int()


def gather(x, indices, weights, top_k):
    x_np, w_np, idx = _f32(x), _f32(weights), indices.cpu().numpy()
    out = np.zeros((idx.shape[0], x_np.shape[1]), dtype=np.float32)
    for i in range(idx.shape[0]):
        scale = np.float32(1.0) if w_np is None else w_np[idx[i]]
        out[i, :] = x_np[idx[i] // top_k, :] * scale
    return torch.from_numpy(_round_to(out, x.dtype)).to(x.dtype)


def scatter(x, indices, weights, top_k):
    x_np, w_np, idx = _f32(x), _f32(weights), indices.cpu().numpy()
    tokens = idx.shape[0] // top_k
    tmp = np.zeros((tokens * top_k, x_np.shape[1]), dtype=np.float32)
    for i in range(idx.shape[0]):
        scale = np.float32(1.0) if w_np is None else w_np[idx[i]]
        tmp[idx[i], :] = x_np[i, :] * scale
    tmp = _round_to(tmp, x.dtype).reshape(tokens, top_k, -1)
    out = tmp.sum(axis=1, dtype=np.float32) if top_k > 1 else tmp.reshape(tokens, -1)
    return torch.from_numpy(_round_to(out, x.dtype)).to(x.dtype)


def scatter_wgrad(x, grad, indices, top_k):
    x_np, g_np, idx = _f32(x), _f32(grad), indices.cpu().numpy()
    out = np.zeros(idx.shape[0], dtype=np.float32)
    for i in range(idx.shape[0]):
        out[idx[i]] = np.dot(x_np[i, :].astype(np.float64), g_np[idx[i] // top_k, :].astype(np.float64))
    return torch.from_numpy(_round_to(out, x.dtype)).to(x.dtype)


def binned_gather(x, indices, weights, bins, ec, top_k):
    x_np, w_np, idx, bins_np = _f32(x), _f32(weights), indices.cpu().numpy(), bins.cpu().numpy()
    ne = bins_np.shape[0]
    out = np.zeros((ne, ec, x_np.shape[1]), dtype=np.float32)
    start = 0
    for i in range(ne):
        end = bins_np[i]
        for j in range(min(ec, end - start)):
            index = idx[start + j]
            scale = np.float32(1.0) if w_np is None else w_np[index]
            out[i, j, :] = x_np[index // top_k, :] * scale
        start = end
    return torch.from_numpy(_round_to(out, x.dtype)).to(x.dtype)


def binned_scatter(x, indices, weights, bins, top_k):
    x_np, w_np, idx, bins_np = _f32(x), _f32(weights), indices.cpu().numpy(), bins.cpu().numpy()
    ne, ec, hs = x_np.shape
    tokens = idx.shape[0] // top_k
    tmp = np.zeros((tokens * top_k, hs), dtype=np.float32)
    start = 0
    for i in range(ne):
        end = bins_np[i]
        for j in range(min(ec, end - start)):
            index = idx[start + j]
            scale = np.float32(1.0) if w_np is None else w_np[index]
            tmp[index, :] = x_np[i, j, :] * scale
        start = end
    tmp = _round_to(tmp, x.dtype).reshape(tokens, top_k, hs)
    out = tmp.sum(axis=1, dtype=np.float32) if top_k > 1 else tmp.reshape(tokens, hs)
    return torch.from_numpy(_round_to(out, x.dtype)).to(x.dtype)


def binned_scatter_wgrad(x, grad, indices, bins, top_k):
    x_np, g_np, idx, bins_np = _f32(x), _f32(grad), indices.cpu().numpy(), bins.cpu().numpy()
    ne, ec, _ = x_np.shape
    out = np.zeros(idx.shape[0], dtype=np.float32)
    start = 0
    for i in range(ne):
        end = bins_np[i]
        for j in range(min(ec, end - start)):
            index = idx[start + j]
            out[index] = np.dot(x_np[i, j, :].astype(np.float64), g_np[index // top_k, :].astype(np.float64))
        start = end
    return torch.from_numpy(_round_to(out, x.dtype)).to(x.dtype)

"""The routing helpers that produce the ragged group sizes of the dropless-MoE expert layer, on the GPU, integer for
integer: the per-expert histogram (reference ``batched_histc``, src/olmo_core/ops/moe.py:289-297, known answer
src/test/ops/moe_test.py:158-164) and ``indices_and_bins`` (src/olmo_core/nn/moe/parallel_mlp.py:102-125) against the
CPU restatements ``oracle.float8_oracle.batched_histc`` / ``oracle.moe_oracle.indices_and_bins``.

``torch.sort`` on the device is not stable, so ``indices`` may order the slots of one expert differently from the
oracle's stable sort; what the reference's contract fixes is that ``indices`` is a permutation of the slots,
that ``expert_indices[indices] == bin_ids`` is sorted, and the histogram / prefix sums - each checked exactly."""

import pytest
import torch

from oracle import float8_oracle as O
from oracle import moe_oracle as MO

pytestmark = pytest.mark.gpu

from olmo_core_amd.nn import DroplessMoEMLP  # noqa: E402
from olmo_core_amd.nn.moe import ParallelDroplessMLP  # noqa: E402
from olmo_core_amd.ops import moe as moe_ops  # noqa: E402


def _zipf_assignment(T=16384, E=64, top_k=8, seed=1005):
    """The expert assignment of the benchmark's configuration 5: N(0,1) logits plus a Zipf(s=1.1) per-expert bias."""
    g = torch.Generator().manual_seed(seed)
    rank = torch.arange(1, E + 1, dtype=torch.float64)
    pmf = rank ** -1.1
    pmf = pmf / pmf.sum()
    logits = torch.randn(T, E, generator=g) + (1.75 * torch.log(pmf)).float()
    return logits.float().softmax(-1).topk(top_k, dim=-1).indices  # [T, top_k] int64


def test_batched_histc_known_answer_on_gpu(dev):
    x = torch.tensor([[0, 1, 1], [2, 0, 0]], device=dev)
    hist = moe_ops.batched_histc(x, 5)
    assert hist.dtype == x.dtype and hist.device == x.device
    assert torch.equal(hist.cpu(), torch.tensor([[1, 2, 0, 0, 0], [2, 0, 1, 0, 0]]))
    assert torch.equal(moe_ops.histc(x.reshape(-1), 5).cpu(), torch.tensor([3, 2, 1, 0, 0]))


@pytest.mark.parametrize("shape", [(16384, 64, 8), (4096, 16, 2), (33, 5, 3), (1, 4, 1)], ids=str)
def test_histogram_and_bins_equal_the_oracle(dev, shape):
    T, E, top_k = shape
    assign = _zipf_assignment(T, E, top_k)
    flat = assign.reshape(-1)
    ref_hist = O.batched_histc(flat.unsqueeze(0), E)[0]
    assert torch.equal(ref_hist, torch.bincount(flat, minlength=E))
    got_hist = moe_ops.histc(flat.to(dev), E)
    assert torch.equal(got_hist.cpu(), ref_hist)
    got_b = moe_ops.batched_histc(assign.to(dev), E)  # one histogram per token: top_k ones
    assert torch.equal(got_b.cpu(), O.batched_histc(assign, E))

    layer = ParallelDroplessMLP(mlp=DroplessMoEMLP(d_model=16, hidden_size=16, num_experts=E), top_k=top_k)
    indices, bin_ids, bins = layer.indices_and_bins(flat.to(dev), got_hist)
    ref_indices, ref_bin_ids, ref_bins = MO.indices_and_bins(assign, E)
    assert indices.dtype == torch.int32 and bins.dtype == torch.int32 and bin_ids.dtype == torch.int32
    assert torch.equal(bins.cpu(), ref_bins), "inclusive prefix sums of the per-expert counts"
    assert torch.equal(bin_ids.cpu(), ref_bin_ids), "sorted expert ids"
    idx = indices.cpu().long()
    assert torch.equal(torch.sort(idx).values, torch.arange(T * top_k)), "indices must be a permutation of the slots"
    assert torch.equal(flat[idx].int(), ref_bin_ids), "indices must sort the expert assignment"
    # inside one expert the slots are the oracle's (as a set): same rows reach the same expert
    bounds = [0] + ref_bins.tolist()
    for e in range(E):
        a = torch.sort(idx[bounds[e]:bounds[e + 1]]).values
        b = ref_indices[bounds[e]:bounds[e + 1]].long()  # the stable sort lists them in slot order
        assert torch.equal(a, b), f"expert {e}: slots differ"


def test_config5_group_sizes(dev):
    """The benchmark's configuration 5: 64 experts, 16384 tokens, top-8, Zipf bias -> 131072 slots, seven experts with
    no token and one with a single token; the device's histogram is what the expert GEMMs receive."""
    assign = _zipf_assignment()
    hist = moe_ops.histc(assign.reshape(-1).to(dev), 64).cpu()
    assert int(hist.sum()) == 131072 and int((hist == 0).sum()) == 7 and int((hist == 1).sum()) >= 1
    assert torch.equal(hist, O.batched_histc(assign.reshape(1, -1), 64)[0])

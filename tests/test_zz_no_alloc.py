"""The entry point that allocates nothing (mi8_cast_tensorwise_static) against the two-call route it is a
variant of (mi8_amax_partials into a caller-owned workspace, then mi8_cast_tensorwise), through the C ABI:
bytes and scale bit-exact, twice in a row with the second input smaller, plus the CPU oracle."""

import ctypes

import pytest
import torch

from helpers import E4M3, E5M2, assert_bytes_equal, assert_scale_equal, bits32, seeded, u8
from olmo_core_amd import _C
from oracle import float8_oracle as O

FP8_CODE = {E4M3: _C.MI8_E4M3, E5M2: _C.MI8_E5M2}


def _pad16(n):
    return (n + 15) // 16 * 16


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _two_call_route(xd, fp8, flags):
    L = _C.lib()
    rows, cols = xd.shape
    slots = torch.empty(_C.AMAX_SLOTS, dtype=torch.int32, device=xd.device)
    used = ctypes.c_int32(0)
    _C.check(L.mi8_amax_partials(xd.data_ptr(), _C.MI8_BF16, rows * cols, slots.data_ptr(), ctypes.byref(used), _stream()))
    q = torch.empty(rows, cols, dtype=torch.uint8, device=xd.device)
    q_t = torch.empty(cols, _pad16(rows), dtype=torch.uint8, device=xd.device)
    s = torch.empty(1, dtype=torch.float32, device=xd.device)
    _C.check(L.mi8_cast_tensorwise(xd.data_ptr(), _C.MI8_BF16, rows, cols, slots.data_ptr(), used.value, None,
                                   FP8_CODE[fp8], flags, q.data_ptr(), cols, q_t.data_ptr(), _pad16(rows),
                                   s.data_ptr(), _stream()))
    return q, q_t, s


def _static_route(xd, fp8, flags, q, q_t, s):
    """Outputs are passed in: between the two calls of the test nothing is allocated on the device."""
    L = _C.lib()
    rows, cols = xd.shape
    _C.check(L.mi8_cast_tensorwise_static(xd.data_ptr(), _C.MI8_BF16, rows, cols, FP8_CODE[fp8], flags, q.data_ptr(),
                                          cols, q_t.data_ptr(), _pad16(rows), s.data_ptr(), _stream()))


@pytest.mark.gpu
@pytest.mark.parametrize("fp8", [E4M3, E5M2], ids=["e4m3", "e5m2"])
@pytest.mark.parametrize("pow2", [False, True], ids=["", "pow2"])
def test_static_cast_equals_workspace_cast_twice_in_a_row(dev, fp8, pow2):
    flags = _C.FLAG_POW2_SCALE if pow2 else 0
    # first call: many partial maxima (2048 slots); second call: a smaller tensor that uses 3 slots only, with a
    # much smaller amax, so that a stale slot of the first call would change its scale
    big = seeded((4100, 4096), seed=11, std=3.0)
    small = seeded((300, 80), seed=12, std=0.01)
    inputs = [big.to(dev), small.to(dev)]
    outs = []
    for xd in inputs:  # every device buffer exists before the first call
        rows, cols = xd.shape
        outs.append((torch.zeros(rows, cols, dtype=torch.uint8, device=dev),
                     torch.zeros(cols, _pad16(rows), dtype=torch.uint8, device=dev),
                     torch.zeros(1, dtype=torch.float32, device=dev)))
    for xd, (q, q_t, s) in zip(inputs, outs):
        _static_route(xd, fp8, flags, q, q_t, s)
    torch.cuda.synchronize()
    for x, xd, (q, q_t, s) in zip((big, small), inputs, outs):
        rq, rq_t, rs = _two_call_route(xd, fp8, flags)
        assert bits32(s)[0] == bits32(rs)[0], "scale differs from the workspace route"
        assert torch.equal(u8(q), u8(rq)), "row-major bytes differ from the workspace route"
        assert torch.equal(u8(q_t), u8(rq_t)), "transposed bytes differ from the workspace route"
        ref_q, ref_s = O.cast(x, fp8, O.TENSORWISE, None, pow2)
        assert_scale_equal(s, ref_s, "scale vs oracle")
        assert_bytes_equal(q.view(fp8), ref_q, what="row-major vs oracle")
        assert_bytes_equal(q_t[:, : x.shape[0]].view(fp8), ref_q.t(), what="transposed vs oracle")


def test_static_cast_refuses_sizes_beyond_its_limit():
    """Argument checks run before any GPU call."""
    L = _C.lib()
    big = (1 << 22) + 16
    assert L.mi8_cast_tensorwise_static(16, _C.MI8_BF16, 16, big, 0, 0, 16, big, None, 0, None, None) == -2
    assert "limit" in _C.last_error()
    assert L.mi8_cast_tensorwise_static(16, _C.MI8_BF16, 1 << 17, 1 << 17, 0, 0, 16, 1 << 17, None, 0, None, None) == -2
    assert L.mi8_cast_tensorwise_static(None, _C.MI8_BF16, 16, 16, 0, 0, None, 16, None, 0, None, None) == -1

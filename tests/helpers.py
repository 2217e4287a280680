"""Shared helpers for the parity tests (CPU oracle vs HIP path)."""

from __future__ import annotations

import numpy as np
import torch

from oracle import float8_oracle as O

E4M3, E5M2 = torch.float8_e4m3fn, torch.float8_e5m2

# tolerance of the GEMM outputs against the fp32-accumulated emulation
MAX_REL_ERR = 1e-2
MIN_COSINE = 0.9999


def seeded(shape, seed, std=1.0, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * std).to(dtype)


def all_bf16_patterns() -> torch.Tensor:
    bits = np.arange(65536, dtype=np.uint16)
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def u8(t: torch.Tensor) -> torch.Tensor:
    return t.contiguous().view(torch.uint8).cpu()


def bits32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().contiguous().view(torch.int32).cpu()


def assert_bytes_equal(got: torch.Tensor, ref: torch.Tensor, what: str = "", fp8: torch.dtype = None):
    """Bit-exact comparison of fp8 bytes; where both sides hold a NaN code only NaN-ness must match
    (the sign/payload of a NaN produced by a multiply differs between x86 and the GPU)."""
    fp8 = fp8 if fp8 is not None else (ref.dtype if ref.dtype in (E4M3, E5M2) else got.dtype)
    assert fp8 in (E4M3, E5M2), "cannot tell which float8 encoding is being compared"
    nan_floor = 0x7D if fp8 == E5M2 else 0x7F  # e5m2 NaN codes 0x7D..0x7F; e4m3fn NaN 0x7F
    got, ref = u8(got), u8(ref)
    assert got.shape == ref.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    neq = got != ref
    if neq.any():
        both_nan = ((got & 0x7F) >= nan_floor) & ((ref & 0x7F) >= nan_floor)
        bad = neq & ~both_nan
        if bad.any():
            idx = bad.nonzero()[:5].tolist()
            raise AssertionError(
                f"{what}: {int(bad.sum())} byte mismatches of {bad.numel()}; first at {idx}: "
                f"got {[int(got[tuple(i)]) for i in idx]} ref {[int(ref[tuple(i)]) for i in idx]}"
            )


def assert_scale_equal(got: torch.Tensor, ref: torch.Tensor, what: str = ""):
    g, r = got.detach().float().cpu().reshape(-1), ref.detach().float().cpu().reshape(-1)
    assert g.shape == r.shape, f"{what}: scale shape {tuple(g.shape)} vs {tuple(r.shape)}"
    same = (bits32(g) == bits32(r)) | (torch.isnan(g) & torch.isnan(r))
    assert bool(same.all()), f"{what}: {int((~same).sum())} scale mismatches, e.g. {g[~same][:4]} vs {r[~same][:4]}"


def gemm_errors(got: torch.Tensor, ref: torch.Tensor):
    g, r = got.detach().double().cpu().reshape(-1), ref.detach().double().cpu().reshape(-1)
    denom = r.abs().max().clamp_min(1e-30)
    rel = float((g - r).abs().max() / denom)
    cos = float(torch.dot(g, r) / (g.norm() * r.norm()).clamp_min(1e-30))
    return rel, cos


def assert_gemm_close(got, ref, what=""):
    rel, cos = gemm_errors(got, ref)
    assert rel <= MAX_REL_ERR and cos >= MIN_COSINE, f"{what}: max rel err {rel:.3e} (<= {MAX_REL_ERR}), cosine {cos:.6f} (>= {MIN_COSINE})"


def spec_for(recipe: str) -> O.LinearSpec:
    return O.recipe(recipe)


def assert_bf16_pointwise_close(got, ref, what="", max_frac=1e-2, ulps=2):
    """A pointwise bf16 result against the host's evaluation of the same formula on the same inputs: the device's
    exp / reciprocal differ from the host's in the last place before a bf16 rounding, so a small fraction of
    elements may differ, each by at most `ulps` bf16 steps of its own magnitude."""
    g, r = got.detach().cpu(), ref.detach().cpu()
    assert g.shape == r.shape and g.dtype == r.dtype == torch.bfloat16, what
    diff = g != r
    frac = float(diff.float().mean())
    assert frac < max_frac, f"{what}: {frac:.4%} of the elements differ (limit {max_frac:.2%})"
    if diff.any():
        gi, ri = g.view(torch.int16).int(), r.view(torch.int16).int()
        # same sign and adjacent bit patterns = adjacent bf16 values
        step = (gi - ri).abs()[diff]
        tiny = (r.float().abs()[diff] < 1e-30) & (g.float().abs()[diff] < 1e-30)
        assert bool(((step <= ulps) | tiny).all()), f"{what}: an element differs by more than {ulps} bf16 steps"

"""Shared checks for the parity tests."""
import torch


def assert_parity(got: torch.Tensor, ref: torch.Tensor, rel: float = 1e-2, what: str = "", tight: float = None,
                  elementwise: float = None):
    """The fp16/bf16 output gate: max relative error <= `rel` against the high-precision
    oracle, with max|ref| as denominator, plus the elementwise form
    |got-ref| <= rel*|ref| + rel*rms(ref).  `tight` optionally asserts a stricter
    max-abs-error / rms(ref) bound that a correct kernel comfortably meets; `elementwise`
    replaces `rel` in the elementwise form only."""
    g = got.detach().to("cpu", torch.float64).reshape(-1)
    r = ref.detach().to("cpu", torch.float64).reshape(-1)
    assert g.shape == r.shape, f"{what}: shape {tuple(got.shape)} vs {tuple(ref.shape)}"
    assert torch.isfinite(g).all(), f"{what}: non-finite output"
    err = (g - r).abs()
    denom = r.abs().max().clamp_min(1e-30)
    rms = r.pow(2).mean().sqrt().clamp_min(1e-30)
    max_rel = float(err.max() / denom)
    assert max_rel <= rel, f"{what}: max rel err {max_rel:.3e} > {rel}"
    e = rel if elementwise is None else elementwise
    bad = err > e * r.abs() + e * rms
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements outside {e}*|ref|+{e}*rms"
    if tight is not None:
        t = float(err.max() / rms)
        assert t <= tight, f"{what}: max abs err / rms = {t:.3e} > {tight}"
    return max_rel


def reference_allclose(got, ref):
    """The reference test-suite's own comparison (tests/test_utils.py:12-27 there)."""
    return torch.allclose(got.float().cpu(), ref.float().cpu(), rtol=1e-4, atol=1e-1)

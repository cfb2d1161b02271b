"""Shared checks for the parity tests."""
import json
import os

import torch


def record_error(what: str, measured: float, gate: float, kind: str = "max_rel"):
    """Every parity assertion reports what it measured: printed (pytest -s / -rP show it) and, when
    MUI_PARITY_LOG names a file, appended there as one JSON line per assertion."""
    line = {"what": what, "kind": kind, "measured": float(measured), "gate": float(gate)}
    print("parity %s: %s = %.3e (gate %.1e)" % (what, kind, measured, gate))
    path = os.environ.get("MUI_PARITY_LOG")
    if path:
        with open(path, "a") as f:
            f.write(json.dumps(line) + "\n")


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
    e = rel if elementwise is None else elementwise
    # smallest factor f for which |got-ref| <= f*|ref| + f*rms(ref) holds everywhere
    elem_needed = float((err / (r.abs() + rms)).max())
    tag = "%s [%s]" % (what, str(got.dtype).replace("torch.", ""))
    record_error(tag, max_rel, rel, "max_err_over_max_ref")
    record_error(tag, elem_needed, e, "elementwise_factor")
    assert max_rel <= rel, f"{what}: max rel err {max_rel:.3e} > {rel}"
    bad = err > e * r.abs() + e * rms
    assert not bool(bad.any()), f"{what}: {int(bad.sum())} elements outside {e}*|ref|+{e}*rms"
    if tight is not None:
        t = float(err.max() / rms)
        assert t <= tight, f"{what}: max abs err / rms = {t:.3e} > {tight}"
    return max_rel


def reference_allclose(got, ref):
    """The reference test-suite's own comparison (tests/test_utils.py:12-27 there)."""
    return torch.allclose(got.float().cpu(), ref.float().cpu(), rtol=1e-4, atol=1e-1)

"""Comparison helpers (test infrastructure only)."""
from __future__ import annotations

import torch


def mismatch_report(actual: torch.Tensor, expected: torch.Tensor, rtol: float, atol: float):
    """Returns (mismatch_fraction, max_abs_err, max_rel_err) under the
    ``|a - e| <= atol + rtol |e|`` rule of torch.isclose."""
    a = actual.detach().to("cpu", torch.float64)
    e = expected.detach().to("cpu", torch.float64)
    err = (a - e).abs()
    bad = ~(err <= atol + rtol * e.abs())
    bad |= torch.isnan(a) | torch.isnan(e)
    rel = err / e.abs().clamp(min=1e-12)
    return bad.double().mean().item(), err.max().item(), rel[e.abs() > atol].max().item() if (e.abs() > atol).any() else 0.0


def assert_close(actual, expected, rtol: float = 1e-2, atol: float = 2e-2, mismatch_ratio: float = 0.0, msg: str = ""):
    """Same acceptance rule as attention_engine/benchmark/bench_utils.py:133-173:
    element-wise isclose, and at most ``mismatch_ratio`` of the elements may
    fall outside the tolerance."""
    assert actual.shape == expected.shape, f"shape {tuple(actual.shape)} vs {tuple(expected.shape)}"
    frac, max_abs, max_rel = mismatch_report(actual, expected, rtol, atol)
    if frac > mismatch_ratio:
        raise AssertionError(
            f"{msg} mismatch fraction {frac:.3e} > {mismatch_ratio:.3e} "
            f"(max abs err {max_abs:.4e}, max rel err {max_rel:.4e}, rtol {rtol}, atol {atol})")

"""Shared helpers for the parity tests."""
import numpy as np
import torch

TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-2, torch.float16: 2e-2}
NAME = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16"}


def to_dev(a: np.ndarray, dtype) -> torch.Tensor:
    """numpy (float64/float32/int) -> device tensor of `dtype`, RNE rounding."""
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype.is_floating_point:
        t = t.to(torch.float32).to(dtype)
    return t.cuda()


def as_f64(t: torch.Tensor) -> np.ndarray:
    """device/host tensor -> float64 numpy (exact widening)."""
    return t.detach().cpu().to(torch.float64).numpy()


def assert_close(got: torch.Tensor, expected: np.ndarray, tol: float, what: str = ""):
    """|got - e| <= max(tol, tol * |e|) elementwise — the rule of the reference's
    conformance runner (InterpretTestRunner.swift:1778)."""
    g = as_f64(got)
    e = np.asarray(expected, dtype=np.float64)
    assert g.shape == e.shape, f"{what}: shape {g.shape} vs {e.shape}"
    both_nan = np.isnan(g) & np.isnan(e)
    err = np.abs(g - e)
    lim = np.maximum(tol, tol * np.abs(e))
    bad = ~(err <= lim) & ~both_nan
    if bad.any():
        i = np.unravel_index(np.argmax(np.where(bad, err / lim, 0)), g.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {g.size} outside tol {tol}; worst at {i}: "
                             f"got {g[i]!r} expected {e[i]!r}")

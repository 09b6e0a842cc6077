"""Shared helpers for the parity tests (not collected by pytest)."""
import torch


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.double().flatten()
    b = b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-300))


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.double() - b.double()).abs().max())


# Tolerances of the parity contract for O, dQ, dK, dV against fp32/fp64 attention on the
# dequantized inputs: max-abs <= 2e-2 and cosine >= 0.999.
MAX_ABS_TOL = 2e-2
COS_TOL = 0.999


def assert_close(name, got, want, max_abs_tol=MAX_ABS_TOL, cos_tol=COS_TOL):
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    ma, cs = max_abs(got, want), cosine(got, want)
    assert ma <= max_abs_tol and cs >= cos_tol, f"{name}: max-abs {ma:.3e} (tol {max_abs_tol}), cosine {cs:.6f} (tol {cos_tol})"
    return ma, cs

"""Shared helpers for the parity tests (not collected by pytest)."""
import torch


def cosine(a: torch.Tensor, b: torch.Tensor) -> float:
    a = a.double().flatten()
    b = b.double().flatten()
    return float((a @ b) / (a.norm() * b.norm()).clamp_min(1e-300))


def max_abs(a: torch.Tensor, b: torch.Tensor) -> float:
    return float((a.double() - b.double()).abs().max())


# Tolerances of the parity contract against fp64 attention on the dequantized inputs:
#   O            max-abs <= 2e-2 and cosine >= 0.999   (|O| <= max|V|, values of order one)
#   dQ, dK, dV   max-abs <= 2e-2 * max(1, max|reference|) and cosine >= 0.999
# The gradients are not of order one (with 20x outlier channels |dQ| reaches ~60), and a 16-bit
# output alone carries a rounding error of 2^-9 of its magnitude (bf16), so their absolute bound
# scales with the largest reference value; the cosine bound does not move.
MAX_ABS_TOL = 2e-2
COS_TOL = 0.999


def assert_close(name, got, want, max_abs_tol=MAX_ABS_TOL, cos_tol=COS_TOL, scaled=False):
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    ma, cs = max_abs(got, want), cosine(got, want)
    tol = max_abs_tol * (max(1.0, float(want.abs().max())) if scaled else 1.0)
    assert ma <= tol and cs >= cos_tol, f"{name}: max-abs {ma:.3e} (tol {tol:.3e}), cosine {cs:.6f} (tol {cos_tol})"
    return ma, cs

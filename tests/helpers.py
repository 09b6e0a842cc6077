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
#   dQ, dK, dV   for EVERY element  |got - want| <= 2e-2 + ulp * (|want| + spread),  and cosine >= 0.999, where
#                ulp    = 2^-7 for bf16, 2^-10 for fp16: the rounding step of the 16-bit format (half a unit in
#                         the last place is 2^-9 / 2^-12 of the value; the bound leaves two bits),
#                want   = the closed-form backward in fp64 given what the kernel is given: the saved 16-bit O
#                         (delta = rowsum(O o dO) comes from it, as in the reference, quant_flash_attn.py:97-99),
#                spread = the 2-norm of the terms of the sum that forms the element (oracle.attn_bwd(spread=True)):
#                         the probabilities and dS enter the matrix pipe rounded to 16 bits, and the error of a
#                         sum of terms rounded that way grows with this norm, not with the (cancelled) result.
# The gradients are not of order one (with 20x outlier channels |dQ| reaches ~60): the bound is element-wise, a
# small element gets no allowance from a large neighbour.  Measured against the EXACT gradients (O not rounded)
# no implementation that receives a 16-bit O can meet 2e-2: that rounding alone moves dK by 4e-2 at N = 384
# (fp64 evaluation of the same formulas), which is why `want` takes the saved O.
MAX_ABS_TOL = 2e-2
COS_TOL = 0.999
REL_TOL = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}


def assert_close(name, got, want, max_abs_tol=MAX_ABS_TOL, cos_tol=COS_TOL, scaled=False, rel=None, spread=None):
    """scaled=False: max|got - want| <= max_abs_tol.  scaled=True (gradients, and outputs that are not of order
    one): |got - want| <= max_abs_tol + rel * (|want| + spread) element-wise, rel from got's dtype unless given."""
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    cs = cosine(got, want)
    err = (got.double() - want.double()).abs()
    if scaled:
        r = REL_TOL.get(got.dtype, 2.0 ** -7) if rel is None else rel
        size = want.double().abs() if spread is None else want.double().abs() + spread.double()
        excess = err - (max_abs_tol + r * size)
        worst = int(excess.argmax())
        ok = bool(excess.max() <= 0)
        detail = (f"worst element: |got - want| {float(err.flatten()[worst]):.3e} at |want| + spread "
                  f"{float(size.flatten()[worst]):.3e} (bound {max_abs_tol:.1e} + {r:.1e} * that)")
    else:
        ok = bool(err.max() <= max_abs_tol)
        detail = f"max-abs {float(err.max()):.3e} (tol {max_abs_tol:.3e})"
    # A reference whose typical element lies below the absolute bar has no direction to compare at the contract's
    # resolution: nearly one-hot softmax rows leave dQ as the small difference of large terms (two dominant keys
    # give dQ_i = sm * dS_i1 * (k_1 - k_2) with the keys' common part cancelled), where the 16-bit operands'
    # rounding is a few percent of the result while every element is 25 times inside the element-wise bound.
    if float(want.double().pow(2).mean().sqrt()) < max_abs_tol:
        cos_tol = -1.0
    assert ok and cs >= cos_tol, f"{name}: {detail}, cosine {cs:.6f} (tol {cos_tol})"
    return float(err.max()), cs


def rounded_output_floor(qh, kh, v, do, o_ref, lse_ref, out_dtype, causal, sm):
    """dQ, dK from the exact formulas (quant_flash_attn.py:153-164) in fp64, but with delta = rowsum(O o dO) taken
    from O ROUNDED to the 16-bit output format -- what every backward is handed (the reference sums the rounded
    O in fp16 as well, :97-99).  Where softmax rows are nearly one-hot, dS = P o (dP - delta) cancels down to that
    rounding, and no kernel can be closer to the exact gradients than these values are."""
    Nq, Nk = qh.shape[-2], kh.shape[-2]
    s = (qh @ kh.transpose(-1, -2)) * sm
    if causal:
        s = s.masked_fill(torch.arange(Nk)[None, :] > torch.arange(Nq)[:, None], float("-inf"))
    p = torch.exp(s - lse_ref.double()[..., None])
    delta = (o_ref.to(out_dtype).double() * do.double()).sum(-1, keepdim=True)
    ds = p * (do.double() @ v.double().transpose(-1, -2) - delta)
    return (ds @ kh) * sm, (ds.transpose(-1, -2) @ qh) * sm

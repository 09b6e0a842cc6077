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
# cosine bar for a reference whose RMS lies below the absolute bar (see assert_close): 0.99 still rejects a result that
# is zero, has the wrong sign or misses a tenth of the reference in any direction
SMALL_COS_TOL = 0.99
REL_TOL = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}


def assert_close(name, got, want, max_abs_tol=MAX_ABS_TOL, cos_tol=COS_TOL, scaled=False, rel=None, spread=None,
                 small_cos_tol=SMALL_COS_TOL):
    """scaled=False: max|got - want| <= max_abs_tol.  scaled=True (gradients, and outputs that are not of order
    one): |got - want| <= max_abs_tol + rel * (|want| + spread) element-wise; rel is the rounding step of got's dtype
    and must be given when got is not a 16-bit tensor (there is no default to fall back on)."""
    assert torch.isfinite(got.float()).all(), f"{name}: non-finite values"
    cs = cosine(got, want)
    err = (got.double() - want.double()).abs()
    if scaled:
        assert rel is not None or got.dtype in REL_TOL, f"{name}: pass rel= for a {got.dtype} result"
        r = REL_TOL[got.dtype] if rel is None else rel
        size = want.double().abs() if spread is None else want.double().abs() + spread.double()
        excess = err - (max_abs_tol + r * size)
        worst = int(excess.argmax())
        ok = bool(excess.max() <= 0)
        detail = (f"worst element: |got - want| {float(err.flatten()[worst]):.3e} at |want| + spread "
                  f"{float(size.flatten()[worst]):.3e} (bound {max_abs_tol:.1e} + {r:.1e} * that)")
    else:
        ok = bool(err.max() <= max_abs_tol)
        detail = f"max-abs {float(err.max()):.3e} (tol {max_abs_tol:.3e})"
    # A reference whose typical element lies below the absolute bar is compared at a coarser angle, never at none:
    # nearly one-hot softmax rows leave dQ as the small difference of large terms (two dominant keys
    # give dQ_i = sm * dS_i1 * (k_1 - k_2) with the keys' common part cancelled), where the 16-bit operands'
    # rounding is a few percent of the result while every element is 25 times inside the element-wise bound
    # (measured: 0.9978); a result of zero, which the absolute bar alone would let through there, has cosine 0.
    rms = float(want.double().pow(2).mean().sqrt())
    if rms < 1e-3 * max_abs_tol:
        cos_tol = -1.0   # a reference that is zero at the bar's resolution has no direction; the absolute bar holds got to zero
    elif rms < max_abs_tol:
        cos_tol = min(cos_tol, small_cos_tol)
    assert ok and cs >= cos_tol, f"{name}: {detail}, cosine {cs:.6f} (tol {cos_tol}), RMS of the reference {rms:.3e}"
    return float(err.max()), cs


def rounded_output_floor(qh, kh, v, do, o_ref, lse_ref, out_dtype, causal, sm):
    """dQ, dK from the exact formulas (quant_flash_attn.py:153-164) in fp64, but with delta = rowsum(O o dO) taken
    from O ROUNDED to the 16-bit output format -- what every backward is handed (the reference sums the rounded
    O in fp16 as well, :97-99).  Where softmax rows are nearly one-hot, dS = P o (dP - delta) cancels down to that
    rounding, and no kernel can be closer to the exact gradients than these values are."""
    Nq, Nk = qh.shape[-2], kh.shape[-2]
    s = (qh @ kh.transpose(-1, -2)) * sm
    if causal:   # aligned to the last key, as in the kernels and the oracle
        s = s.masked_fill(torch.arange(Nk)[None, :] > torch.arange(Nq)[:, None] + (Nk - Nq), float("-inf"))
    p = torch.exp(s - lse_ref.double()[..., None])
    delta = (o_ref.to(out_dtype).double() * do.double()).sum(-1, keepdim=True)
    ds = p * (do.double() @ v.double().transpose(-1, -2) - delta)
    return (ds @ kh) * sm, (ds.transpose(-1, -2) @ qh) * sm

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
# The direction test is waived only for an error that is small in absolute terms: RMS(got - want) <= SMALL_ERR_FRAC
# of the absolute bar (see assert_close).  A result of zero, or of the wrong sign, passes that only where the reference
# itself lies below that size.
SMALL_ERR_FRAC = 0.15
REL_TOL = {torch.bfloat16: 2.0 ** -7, torch.float16: 2.0 ** -10}


def assert_close(name, got, want, max_abs_tol=MAX_ABS_TOL, cos_tol=COS_TOL, scaled=False, rel=None, spread=None):
    """scaled=False: max|got - want| <= max_abs_tol.  scaled=True (gradients, and outputs that are not of order
    one): |got - want| <= max_abs_tol + rel * (|want| + spread) element-wise; rel is the rounding step of got's dtype
    and must be given when got is not a 16-bit tensor (there is no default to fall back on).
    Direction: cosine >= cos_tol, or else RMS(got - want) <= SMALL_ERR_FRAC * max_abs_tol, or else (spread given)
    RMS(got - want) <= rel * RMS(spread)."""
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
    # A cosine below the bar is accepted only when the error itself is small in absolute terms.  Nearly one-hot
    # softmax rows leave dQ as the small difference of large terms (two dominant keys give
    # dQ_i = sm * dS_i1 * (k_1 - k_2) with the keys' common part cancelled): the reference's RMS is then 5e-3,
    # the 16-bit operands' rounding leaves an error of 7e-4 -- thirty times inside the element-wise bound -- and the
    # cosine comes out at 0.98.  What this exception does NOT let through is a result of zero or of the wrong sign
    # for a reference above 3e-3, which the element-wise bound alone would.
    # Likewise where the spread is given and the error's RMS stays below one rounding step of the spread's RMS: a single
    # query against 700 keys leaves dQ at a hundredth of its terms, and what the 8-bit operands lose of those terms
    # is then a third of the result (cosine 0.97) although it is half a percent of what was summed.
    err_rms = float(err.pow(2).mean().sqrt())
    rms = float(want.double().pow(2).mean().sqrt())
    direction_ok = cs >= cos_tol or err_rms <= SMALL_ERR_FRAC * max_abs_tol
    if scaled and spread is not None:
        direction_ok = direction_ok or err_rms <= r * float(spread.double().pow(2).mean().sqrt())
    assert ok and direction_ok, (f"{name}: {detail}, cosine {cs:.6f} (tol {cos_tol}), RMS of the error {err_rms:.3e}, "
                                 f"of the reference {rms:.3e}")
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

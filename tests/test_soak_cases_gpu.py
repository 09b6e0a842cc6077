"""Seeded cases that a random soak of 6 000 forward + backward problems left OUTSIDE the usual bars, kept as tests of
what the kernels do there (the soak itself is not part of the suite).  Two kinds:

  * three "offset" problems whose largest dK error passes the element-wise bound  2e-2 + 2^-7 (|want| + spread)  by
    2 to 10 %.  P, dS and the dequantized operand enter the matrix pipe rounded to 8 bits, so an element's error has a
    standard deviation of about 2^-9 of its spread and the bound sits at four of them; among 10^5 elements one
    reaches 4.5.  Held here to 1.25 x the bound at every element, to the bound itself at all but 1 in 10^4, and to an
    RMS error of one standard deviation;
  * "spike" / "ramp" problems whose dQ cancels down to an RMS of 5e-3 .. 3e-2 (a few dominant keys): every element is
    ten times inside the element-wise bound while the cosine comes out between 0.97 and 0.999.  Held to the
    element-wise bound and to an RMS error of 15 % of the absolute bar, or of one rounding step of the summed terms'
    RMS where those are a hundred times the result (helpers.assert_close's rule for directions).

The problems are generated exactly as the soak generated them (same generator seeds)."""
import math
import random

import pytest
import torch

from helpers import MAX_ABS_TOL, REL_TOL, assert_close, max_abs
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _soak_case(seed, index):
    """The index-th problem of the soak with this seed (the draws of the earlier problems are replayed)."""
    rng = random.Random(seed)
    for it in range(index + 1):
        D = rng.choice((64, 128, 256, 256))
        dt = rng.choice((torch.bfloat16, torch.float16))
        causal = rng.random() < 0.6
        B, H = rng.choice(((1, 1), (1, 2), (2, 2), (1, 5), (3, 3)))
        Nk = rng.choice((64, 128, 192, 256, 320, 384, 100, 333, 129, 65, 500, 31, 33, 700, 1, 17))
        if causal:
            Nq = rng.choice([x for x in (Nk, Nk, 1, 17, 31, 32, 33, 64, 97, 128, 200, 256) if x <= Nk])
        else:
            Nq = rng.choice((Nk, 128, 256, 97, 17, 1))
        kind = rng.choice(("normal", "normal", "ramp", "spike", "offset", "tiny"))
    g = torch.Generator().manual_seed(seed * 100000 + index)
    q = torch.randn(B, H, Nq, D, generator=g)
    k = torch.randn(B, H, Nk, D, generator=g)
    v = torch.randn(B, H, Nk, D, generator=g)
    do = torch.randn(B, H, Nq, D, generator=g)
    if kind == "ramp":
        q = q * 0.2 + 1.0
        k = k * 0.2 + torch.linspace(-1, 2, Nk).view(1, 1, Nk, 1)
    elif kind == "spike":
        q = q * 0.3 + 1.0
        idx = torch.randint(0, Nk, (max(1, Nk // 50),), generator=g)
        k = k * 0.3
        k[:, :, idx] += 3.0
    elif kind == "offset":
        q = q + torch.randn(B, H, Nq, 1, generator=g) * 2
        k = k + torch.randn(B, H, Nk, 1, generator=g) * 2
    elif kind == "tiny":
        q, k = q * 1e-3, k * 1e-3
    return kind, D, dt, causal, (q.to(dt), k.to(dt), v.to(dt), do.to(dt))


def _run(qfa, q, k, v, do, causal, sm):
    qq, kq = qfa.quantize_pair_for_attention(q.to(DEV), k.to(DEV))
    o, lse = qfa.attn_fwd_quantized(qq, kq, v.to(DEV), causal, sm)
    dq, dk, dv = qfa.attn_bwd_quantized(qq, kq, v.to(DEV), o, do.to(DEV), lse, causal, sm)
    qh = oracle.dequantize_per_token(qq.codes.cpu(), qq.scale.cpu(), qq.zero_point.cpu(), torch.float64)
    kh = oracle.dequantize_per_token(kq.codes.cpu(), kq.scale.cpu(), kq.zero_point.cpu(), torch.float64)
    o_ref, lse_ref = oracle.attn_fwd(qh, kh, v, causal, sm)
    want, spreads = oracle.attn_bwd(qh, kh, v, do, causal, sm, o=o.cpu(), spread=True)
    assert_close("O", o.cpu(), o_ref)
    assert max_abs(lse.cpu(), lse_ref) < 2.0 ** -8 * max(1.0, float(lse_ref.abs().max()) / 64)
    return (dq.cpu(), dk.cpu(), dv.cpu()), want, spreads


@pytest.mark.parametrize("seed,index", [(11, 269), (11, 1839), (11, 2620)])
def test_largest_dk_error_of_offset_problems(qfa, seed, index):
    kind, D, dt, causal, (q, k, v, do) = _soak_case(seed, index)
    assert kind == "offset" and dt == torch.bfloat16
    got, want, spreads = _run(qfa, q, k, v, do, causal, 1.0 / math.sqrt(D))
    for name, g, w, sp in zip(("dQ", "dK", "dV"), got, want, spreads):
        err = (g.double() - w).abs()
        bound = MAX_ABS_TOL + REL_TOL[dt] * (w.abs() + sp)
        assert bool((err <= 1.25 * bound).all()), f"{name}: an element is more than a quarter over the bound"
        assert float((err > bound).double().mean()) <= 1e-4, f"{name}: more than 1 element in 10^4 over the bound"
        assert float(err.pow(2).mean().sqrt()) <= 2.0 ** -9 * float((w.abs() + sp).pow(2).mean().sqrt()) + 1e-3, name
        assert float((g.double() * w).sum() / (g.double().norm() * w.norm())) >= 0.999, name


@pytest.mark.parametrize("seed,index", [(7, 30), (7, 771), (7, 2196), (11, 95), (11, 2404), (11, 483)])
def test_cancelled_dq_of_spike_and_ramp_problems(qfa, seed, index):
    kind, D, dt, causal, (q, k, v, do) = _soak_case(seed, index)
    assert kind in ("spike", "ramp")
    got, want, spreads = _run(qfa, q, k, v, do, causal, 1.0 / math.sqrt(D))
    assert float(want[0].pow(2).mean().sqrt()) < 3e-2, "dQ of these problems is meant to be nearly cancelled"
    for name, g, w, sp in zip(("dQ", "dK", "dV"), got, want, spreads):
        assert_close(name, g, w, scaled=True, spread=sp)

"""Pins the CPU oracle of the attention forward / backward (oracle/oracle.py).

Checks against library routines (torch.softmax, logsumexp, scaled_dot_product_attention,
autograd, gradcheck), closed-form special cases, and the exact integer identity behind the
INT8 score path.  Also runs the plumbing configuration (B1 H4 N256 D64 fp32, non-causal) end to
end on the CPU: quantize q and k, attention forward, compared with fp32 dequantized attention.
"""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs


def _rand(*shape, seed=0, dtype=torch.float64):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed), dtype=dtype)


@pytest.mark.parametrize("causal", [False, True])
def test_fwd_matches_sdpa_and_softmax(causal):
    q, k, v = _rand(2, 3, 40, 16, seed=1), _rand(2, 3, 40, 16, seed=2), _rand(2, 3, 40, 16, seed=3)
    sm = 0.37
    o, lse = oracle.attn_fwd(q, k, v, causal, sm)
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=causal, scale=sm)
    assert torch.allclose(o, ref, atol=1e-12, rtol=1e-10)
    s = q @ k.transpose(-1, -2) * sm
    if causal:
        s = s + torch.full((40, 40), float("-inf"), dtype=s.dtype).triu(1)
    assert torch.allclose(lse, torch.logsumexp(s, -1), atol=1e-12)
    assert torch.allclose(o, torch.softmax(s, -1) @ v, atol=1e-12)


def test_fwd_special_cases():
    v = _rand(1, 1, 9, 4, seed=4)
    zeros = torch.zeros(1, 1, 9, 4, dtype=torch.float64)
    # uniform scores: non-causal O = mean of V, LSE = ln N ; causal O = running mean, LSE = ln(i+1)
    o, lse = oracle.attn_fwd(zeros, zeros, v, False, 1.0)
    assert torch.allclose(o, v.mean(-2, keepdim=True).expand_as(o)) and torch.allclose(lse, torch.full_like(lse, math.log(9)))
    o, lse = oracle.attn_fwd(zeros, zeros, v, True, 1.0)
    run_mean = v.cumsum(-2) / torch.arange(1, 10, dtype=torch.float64)[:, None]
    assert torch.allclose(o, run_mean) and torch.allclose(lse[0, 0], torch.arange(1, 10, dtype=torch.float64).log())
    # causal row 0 only sees key 0
    q, k = _rand(1, 1, 9, 4, seed=5), _rand(1, 1, 9, 4, seed=6)
    o, _ = oracle.attn_fwd(q, k, v, True, 0.5)
    assert torch.allclose(o[..., 0, :], v[..., 0, :])
    # causal with fewer queries than keys: the rows are the last rows of the square case; and against the library
    # mask built independently (tril with a diagonal offset)
    q9, k9 = _rand(1, 1, 9, 4, seed=5), _rand(1, 1, 9, 4, seed=6)
    o_sq, lse_sq = oracle.attn_fwd(q9, k9, v, True, 0.5)
    o_r, lse_r = oracle.attn_fwd(q9[..., 5:, :], k9, v, True, 0.5)
    assert torch.allclose(o_r, o_sq[..., 5:, :]) and torch.allclose(lse_r, lse_sq[..., 5:])
    keep = torch.ones(4, 9, dtype=torch.bool).tril(diagonal=5)
    ref = F.scaled_dot_product_attention(q9[..., 5:, :], k9, v, attn_mask=keep, scale=0.5)
    assert torch.allclose(o_r, ref)
    dq_r, dk_r, dv_r = oracle.attn_bwd(q9[..., 5:, :], k9, v, torch.ones(1, 1, 4, 4, dtype=torch.float64), True, 0.5)
    g = torch.zeros(1, 1, 9, 4, dtype=torch.float64)
    g[..., 5:, :] = 1.0
    dq_s, dk_s, dv_s = oracle.attn_bwd(q9, k9, v, g, True, 0.5)
    assert torch.allclose(dq_r, dq_s[..., 5:, :]) and torch.allclose(dk_r, dk_s) and torch.allclose(dv_r, dv_s)
    # Nq != Nk, non causal: shapes and a one-key limit
    o, lse = oracle.attn_fwd(q[..., :3, :], k[..., :1, :], v[..., :1, :], False, 0.5)
    assert torch.allclose(o, v[..., :1, :].expand(1, 1, 3, 4))


@pytest.mark.parametrize("causal", [False, True])
def test_bwd_closed_form_matches_autograd(causal):
    q, k, v, do = (_rand(2, 2, 24, 8, seed=s) for s in (7, 8, 9, 10))
    dq, dk, dv = oracle.attn_bwd(q, k, v, do, causal, 0.41)
    aq, ak, av = oracle.attn_bwd_autograd(q, k, v, do, causal, 0.41)
    for a, b in ((dq, aq), (dk, ak), (dv, av)):
        assert torch.allclose(a, b, atol=1e-12, rtol=1e-9)
    # and SDPA's own backward
    q2, k2, v2 = (t.clone().requires_grad_(True) for t in (q, k, v))
    F.scaled_dot_product_attention(q2, k2, v2, is_causal=causal, scale=0.41).backward(do)
    assert torch.allclose(dq, q2.grad, atol=1e-11) and torch.allclose(dk, k2.grad, atol=1e-11)
    assert torch.allclose(dv, v2.grad, atol=1e-11)


def test_fwd_gradcheck():
    q, k, v = (_rand(1, 1, 5, 3, seed=s).requires_grad_(True) for s in (11, 12, 13))
    assert torch.autograd.gradcheck(lambda a, b, c: oracle.attn_fwd(a, b, c, True, 0.7)[0], (q, k, v), atol=1e-8)


def test_delta_closed_form():
    o, do = _rand(2, 2, 6, 4, seed=14), _rand(2, 2, 6, 4, seed=15)
    assert torch.allclose(oracle.bwd_delta(o, do), torch.einsum("bhnd,bhnd->bhn", o, do))


@pytest.mark.parametrize("config,D", [("offset", 128), ("uniform", 64), ("outlier", 128)])
def test_integer_cross_term_identity(config, D):
    """A - zk*rq - zq*rk + D*zq*zk == sum_d (qc - zq)(kc - zk), exactly, and the dequantized
    dot product equals scale_q * scale_k * that integer."""
    q, k, _, _ = make_inputs(config, 1, 2, 96, D, seed=3)
    qc, _, zq, sq, rq = oracle.quantize_per_token(q)
    kc, _, zk, sk, rk = oracle.quantize_per_token(k)
    got = oracle.int_scores(qc, zq, kc, zk)
    brute = ((qc.long() - zq.long())[..., :, None, :] * (kc.long() - zk.long())[..., None, :, :]).sum(-1)
    assert torch.equal(got, brute)
    assert got.abs().max() < 2 ** 23 and (qc.long() @ kc.long().transpose(-1, -2)).abs().max() <= 2 ** 21
    qh = oracle.dequantize_per_token(qc, sq, zq, torch.float64)
    kh = oracle.dequantize_per_token(kc, sk, zk, torch.float64)
    dots = qh @ kh.transpose(-1, -2)
    assert torch.allclose(dots, got.double() * sq.double() * sk.double().transpose(-1, -2), rtol=1e-12, atol=1e-12)
    assert torch.equal(rq, qc.int().sum(-1, keepdim=True)) and torch.equal(rk, kc.int().sum(-1, keepdim=True))


def test_legacy_shared_kv_matches_sdpa_autograd():
    """quant_flash_attn.py semantics: K == V == dequant(kv); dkv = dK + dV is what autograd gives a
    single kv leaf used twice (test_accuracy.py:76-81)."""
    q = _rand(1, 2, 7, 16, seed=20)
    kv = _rand(1, 2, 33, 16, seed=21)
    do = _rand(1, 2, 7, 16, seed=22)
    codes, scale, zp, _, _ = oracle.quantize_per_token(kv.float())
    o, _ = oracle.legacy_fwd(q, codes, scale, zp, 0.25)
    dq, dkv = oracle.legacy_bwd(q, codes, scale, zp, do, 0.25)
    kvh = oracle.dequantize_per_token(codes, scale, zp, torch.float64).requires_grad_(True)
    q2 = q.clone().requires_grad_(True)
    ref = F.scaled_dot_product_attention(q2, kvh, kvh, is_causal=False, scale=0.25)
    ref.backward(do)
    assert torch.allclose(o, ref, atol=1e-12)
    assert torch.allclose(dq, q2.grad, atol=1e-11) and torch.allclose(dkv, kvh.grad, atol=1e-11)


def test_plumbing_config_on_cpu():
    """B=1 H=4 N=256 D=64 fp32 non-causal, seed 0: quantize q and k, forward, vs fp32 dequantized
    attention and vs the un-quantized attention at the reference's own tolerance (atol 1e-1)."""
    torch.manual_seed(0)
    q, k, v = torch.randn(1, 4, 256, 64), torch.randn(1, 4, 256, 64), torch.randn(1, 4, 256, 64)
    sm = 1.0 / math.sqrt(64)
    qc, _, zq, sq, _ = oracle.quantize_per_token(q)
    kc, _, zk, sk, _ = oracle.quantize_per_token(k)
    # the configuration text writes zp = round(-min/scale) - 128; the reference rounds
    # -128 - min/scale (asymmetric_quant.py:89-90): same value unless the fp32 subtraction crosses a tie
    alt = oracle.roundf_half_away((-q.amin(-1, keepdim=True) / sq).numpy()) - 128
    assert (torch.from_numpy(alt).to(torch.int8) != zq).float().mean() < 0.02
    qh, kh = oracle.dequantize_per_token(qc, sq, zq), oracle.dequantize_per_token(kc, sk, zk)
    # integer path -> same scores as the dequantized fp32 path
    s_int = oracle.int_scores(qc, zq, kc, zk).double() * sq.double() * sk.double().transpose(-1, -2) * sm
    o_int = torch.softmax(s_int, -1) @ v.double()
    o32 = F.scaled_dot_product_attention(qh, kh, v, scale=sm)
    o64, _ = oracle.attn_fwd(qh, kh, v, False, sm)
    # (qh, kh are fp32-rounded dequantized values; the integer path is exact: agreement to ~1e-7)
    assert torch.allclose(o_int, o64, atol=1e-6)
    assert (o32.double() - o64).abs().max() < 1e-5
    # quantization error against the un-quantized attention stays inside the reference's tolerance
    ref = F.scaled_dot_product_attention(q, k, v, scale=sm)
    assert torch.allclose(o32, ref, atol=1e-1, rtol=0)
    # the timed CPU baseline path returns the same thing
    assert torch.allclose(oracle.reference_cpu_path(q, k, v, False, sm), o32, atol=1e-6)

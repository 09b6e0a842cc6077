"""Seeded random sweeps of shapes, dtypes and score distributions through the C ABI against the CPU oracle.
The distributions are chosen to move the softmax reference around: scores that grow along the keys ("ramp"),
a few keys far above the rest ("spike"), large and tiny magnitudes.  Bars as in the other parity tests
(O max-abs <= 2e-2 * max(1, max|ref|), cosine >= 0.999, LSE 2^-8 relative to max(1, max|LSE|/64)); gradient
cosines are only required where the softmax is not nearly one-hot (the 16-bit rounding of O alone moves small
dQ there)."""
import math
import random

import pytest
import torch

from helpers import assert_close, max_abs
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _scores(kind, q, k, Nk, g):
    if kind == "ramp":
        return q * 0.2 + 1.5, k * 0.2 + torch.linspace(-2, 4, Nk).view(1, 1, Nk, 1)
    if kind == "spike":
        idx = torch.randint(0, Nk, (max(1, Nk // 50),), generator=g)
        k = k * 0.3
        k[:, :, idx] += 5.0
        return q * 0.3 + 2.0, k
    if kind == "big":
        return q * 6.0, k * 3.0
    if kind == "tiny":
        return q * 1e-3, k * 1e-3
    return q, k


def _forward_sweep(qfa, seed, dims, iters):
    rng = random.Random(seed)
    for it in range(iters):
        D = rng.choice(dims)
        dt = rng.choice((torch.bfloat16, torch.float16))
        causal = rng.random() < 0.5
        B, H = rng.choice(((1, 1), (1, 2), (2, 2)))
        Nk = rng.choice((64, 128, 192, 256, 320, 384, 448, 512, 640, 100, 333, 700, 129, 65))
        Nq = Nk if causal else rng.choice((Nk, 128, 256, 97, 384, 17))
        kind = rng.choice(("normal", "ramp", "spike", "big", "tiny"))
        g = torch.Generator().manual_seed(it)
        q = torch.randn((B, H, Nq, D), generator=g)
        k = torch.randn((B, H, Nk, D), generator=g)
        v = torch.randn((B, H, Nk, D), generator=g).to(dt)
        q, k = (t.to(dt) for t in _scores(kind, q, k, Nk, g))
        sm = 1.0 / math.sqrt(D)
        qq, kq = qfa.quantize_for_attention(q.to(DEV)), qfa.quantize_for_attention(k.to(DEV))
        o, lse = qfa.attn_fwd_quantized(qq, kq, v.to(DEV), causal, sm)
        qh = oracle.dequantize_per_token(qq.codes.cpu(), qq.scale.cpu(), qq.zero_point.cpu(), torch.float64)
        kh = oracle.dequantize_per_token(kq.codes.cpu(), kq.scale.cpu(), kq.zero_point.cpu(), torch.float64)
        o_ref, lse_ref = oracle.attn_fwd(qh, kh, v, causal, sm)
        case = f"case {it}: {kind} B{B} H{H} Nq{Nq} Nk{Nk} D{D} {dt} causal={causal}"
        assert_close(case + " O", o.cpu(), o_ref)
        assert max_abs(lse.cpu(), lse_ref) < 2.0 ** -8 * max(1.0, float(lse_ref.abs().max()) / 64), case


def test_forward_random_sweep(qfa):
    _forward_sweep(qfa, 1234, (64, 128), 96)


def test_forward_random_sweep_head_dim_256(qfa):
    _forward_sweep(qfa, 2560, (256,), 40)


def test_shared_kv_random_sweep(qfa):
    rng = random.Random(4321)
    for it in range(64):
        D = rng.choice((64, 128, 256))
        B, H = rng.choice(((1, 1), (1, 3), (2, 2)))
        Nq = rng.choice((1, 5, 16, 17, 32, 33, 48, 64, 97, 130))
        Nk = rng.choice((1, 31, 32, 33, 64, 100, 500, 689, 1025))
        kind = rng.choice(("normal", "offset", "ramp", "big"))
        g = torch.Generator().manual_seed(1000 + it)
        q = torch.randn((B, H, Nq, D), generator=g)
        kv = torch.randn((B, H, Nk, D), generator=g)
        do = torch.randn((B, H, Nq, D), generator=g).half()
        if kind == "offset":
            q, kv = q + 1.0, kv - 0.7
        elif kind == "ramp":
            q, kv = q * 0.2 + 1.0, kv * 0.3 + torch.linspace(-1, 3, Nk).view(1, 1, Nk, 1)
        elif kind == "big":
            q = q * 4.0
        q, kv = q.half(), kv.half()
        sm = 1.0 / math.sqrt(D)
        codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV))
        o, lse = qfa.attn_fwd_shared_kv(q.to(DEV), codes, scale, zp, sm)
        dq, dkv = qfa.attn_bwd_shared_kv(q.to(DEV), codes, scale, zp, o, do.to(DEV), lse, sm)
        c, s_, z = codes.cpu(), scale.cpu(), zp.cpu()
        o_ref, lse_ref = oracle.legacy_fwd(q, c, s_, z, sm)
        (dq_ref, dkv_ref), (nq, nkv) = oracle.legacy_bwd(q, c, s_, z, do, sm, o=o.cpu(), spread=True)
        case = f"case {it}: {kind} B{B} H{H} Nq{Nq} Nk{Nk} D{D}"
        assert_close(case + " O", o.cpu(), o_ref, scaled=True)
        assert max_abs(lse.cpu(), lse_ref) < 2.0 ** -8 * max(1.0, float(lse_ref.abs().max()) / 64), case
        # with a single key P = 1 and dS = 0: dQ is exactly zero and its cosine undefined
        assert_close(case + " dQ", dq.cpu(), dq_ref, scaled=True, spread=nq, cos_tol=-1 if Nk == 1 else 0.999)
        assert_close(case + " dKV", dkv.cpu(), dkv_ref, scaled=True, spread=nkv)
        assert torch.isfinite(dq).all() and torch.isfinite(dkv).all(), case


def _backward_sweep(qfa, seed, dims, iters):
    rng = random.Random(seed)
    for it in range(iters):
        D = rng.choice(dims)
        dt = rng.choice((torch.bfloat16, torch.float16))
        causal = rng.random() < 0.6
        B, H = rng.choice(((1, 1), (1, 2), (2, 2), (3, 3), (2, 5), (1, 16), (4, 5)))
        Nk = rng.choice((64, 128, 192, 256, 320, 384, 100, 333, 129, 65, 500))
        Nq = Nk if causal else rng.choice((Nk, 128, 256, 97, 17))
        kind = rng.choice(("normal", "ramp", "spike", "big"))
        g = torch.Generator().manual_seed(5000 + it)
        q = torch.randn((B, H, Nq, D), generator=g)
        k = torch.randn((B, H, Nk, D), generator=g)
        v = torch.randn((B, H, Nk, D), generator=g).to(dt)
        do = torch.randn((B, H, Nq, D), generator=g).to(dt)
        q, k = _scores(kind, q, k, Nk, g)
        if kind == "big":
            q, k = q * 0.5, k * (2.0 / 3.0)
        q, k = q.to(dt), k.to(dt)
        sm = 1.0 / math.sqrt(D)
        qq, kq = qfa.quantize_for_attention(q.to(DEV)), qfa.quantize_for_attention(k.to(DEV))
        o, lse = qfa.attn_fwd_quantized(qq, kq, v.to(DEV), causal, sm)
        dq, dk, dv = qfa.attn_bwd_quantized(qq, kq, v.to(DEV), o, do.to(DEV), lse, causal, sm)
        qh = oracle.dequantize_per_token(qq.codes.cpu(), qq.scale.cpu(), qq.zero_point.cpu(), torch.float64)
        kh = oracle.dequantize_per_token(kq.codes.cpu(), kq.scale.cpu(), kq.zero_point.cpu(), torch.float64)
        # the closed forms in fp64 on what the kernel is given, the saved 16-bit O included: where softmax rows are
        # nearly one-hot (ramp, spike, big) dS cancels down to the rounding of that O, for every implementation
        (rq, rk, rv), (nq, nk, nv) = oracle.attn_bwd(qh, kh, v, do, causal, sm, o=o.cpu(), spread=True)
        case = f"case {it}: {kind} B{B} H{H} Nq{Nq} Nk{Nk} D{D} {dt} causal={causal}"
        assert_close(case + " dQ", dq.cpu(), rq, scaled=True, spread=nq)
        assert_close(case + " dK", dk.cpu(), rk, scaled=True, spread=nk)
        assert_close(case + " dV", dv.cpu(), rv, scaled=True, spread=nv)
        assert torch.isfinite(dq).all() and torch.isfinite(dk).all() and torch.isfinite(dv).all(), case


def test_backward_random_sweep(qfa):
    """Forward + backward of the INT8-score kernels; head counts from 1 to 20 so that the causal dispatch
    groups (2 to 8 heads) come out full, partial and absent."""
    _backward_sweep(qfa, 777, (64, 128), 72)


def test_backward_random_sweep_head_dim_256(qfa):
    _backward_sweep(qfa, 2561, (256,), 32)

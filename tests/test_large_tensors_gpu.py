"""Tensors of more than 2^31 elements (more than 4 GiB in bf16): every (batch, head) offset, token index and
byte offset past the 32-bit range.  The kernels treat heads independently and deterministically, so the last
head of the large tensor, which lies wholly beyond element 2^31, must come out BIT-IDENTICAL to a launch on a
contiguous copy of that head alone; one forward check against the fp64 oracle ties the small launch to the
reference arithmetic (quant_flash_attn.py:50-83, asymmetric_quant.py:66-106)."""
import math

import pytest
import torch

from helpers import assert_close
from oracle import oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _head(t, b, h):
    return t[b:b + 1, h:h + 1].contiguous()


def _head_q(qt, b, h):
    return type(qt)(*(_head(t, b, h) for t in qt))


def _randn(shape, dtype, seed, offset=0.0):
    g = torch.Generator(device=DEV).manual_seed(seed)
    x = torch.empty(shape, dtype=dtype, device=DEV)
    for b in range(shape[0]):   # per batch entry: no fp32 temporary of the whole tensor
        x[b] = (torch.randn(shape[1:], generator=g, device=DEV) + offset).to(dtype)
    return x


def test_quantizer_past_2_31_elements(qfa):
    B, H, N, D = 65, 64, 4096, 128
    assert B * H * N * D > 2 ** 31
    x = _randn((B, H, N, D), torch.bfloat16, 1, offset=0.5)
    got = qfa.quantize_for_attention(x)
    for (b, h) in [(0, 0), (32, 1), (B - 1, H - 1)]:
        one = qfa.quantize_for_attention(_head(x, b, h))
        for name, big, small in zip(got._fields, got, one):
            assert torch.equal(_head(big, b, h), small), f"{name}[{b},{h}]"
    o_codes, o_scale, o_zp, o_rowsum = oracle.quantize_per_token_c(_head(x, B - 1, H - 1).cpu())
    last = _head_q(got, B - 1, H - 1)
    assert torch.equal(last.codes.cpu(), o_codes) and torch.equal(last.zero_point.cpu(), o_zp)
    assert torch.equal(last.scale.cpu(), o_scale) and torch.equal(last.rowsum.cpu(), o_rowsum)


@pytest.mark.parametrize("causal", [True, False])
def test_attention_past_2_31_elements(qfa, causal):
    B, H, N, D = 65, 64, 4096, 128
    sm = 1.0 / math.sqrt(D)
    q = _randn((B, H, N, D), torch.bfloat16, 2, offset=0.25)
    k = _randn((B, H, N, D), torch.bfloat16, 3, offset=-0.25)
    v = _randn((B, H, N, D), torch.bfloat16, 4)
    do = _randn((B, H, N, D), torch.bfloat16, 5)
    qq, kq = qfa.quantize_for_attention(q), qfa.quantize_for_attention(k)
    del q, k
    o, lse = qfa.attn_fwd_quantized(qq, kq, v, causal, sm)
    dq, dk, dv = qfa.attn_bwd_quantized(qq, kq, v, o, do, lse, causal, sm)
    torch.cuda.synchronize()
    for (b, h) in [(0, 0), (32, 1), (B - 1, H - 1)]:
        qh, kh, vh, doh = _head_q(qq, b, h), _head_q(kq, b, h), _head(v, b, h), _head(do, b, h)
        o1, lse1 = qfa.attn_fwd_quantized(qh, kh, vh, causal, sm)
        assert torch.equal(_head(o, b, h), o1), f"O[{b},{h}]"
        assert torch.equal(_head(lse, b, h), lse1), f"LSE[{b},{h}]"
        dq1, dk1, dv1 = qfa.attn_bwd_quantized(qh, kh, vh, o1, doh, lse1, causal, sm)
        assert torch.equal(_head(dq, b, h), dq1), f"dQ[{b},{h}]"
        assert torch.equal(_head(dk, b, h), dk1), f"dK[{b},{h}]"
        assert torch.equal(_head(dv, b, h), dv1), f"dV[{b},{h}]"
    # the last head against the oracle (last 1024 query rows: dense fp64 scores)
    b, h = B - 1, H - 1
    qh = oracle.dequantize_per_token(*(t.cpu() for t in _head_q(qq, b, h)[:3]), torch.float64)
    kh = oracle.dequantize_per_token(*(t.cpu() for t in _head_q(kq, b, h)[:3]), torch.float64)
    rows = slice(N - 1024, N)
    s = (qh[..., rows, :] @ kh.transpose(-1, -2)) * sm
    if causal:
        s = s.masked_fill(torch.arange(N)[None, :] > torch.arange(N - 1024, N)[:, None], float("-inf"))
    assert_close("O last head", _head(o, b, h).cpu()[..., rows, :], torch.softmax(s, -1) @ _head(v, b, h).cpu().double())


def test_shared_kv_past_2_31_elements(qfa):
    """The reference's benchmark shape (compute_flops.py:96): 3.1e9 key elements."""
    Z, H, Nq, Nkv, D = 512, 16, 16, 3000, 128
    assert Z * H * Nkv * D > 2 ** 31
    sm = 1.0 / math.sqrt(D)
    q = _randn((Z, H, Nq, D), torch.float16, 6)
    kv = _randn((Z, H, Nkv, D), torch.float16, 7)
    do = _randn((Z, H, Nq, D), torch.float16, 8)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv)
    del kv
    from quant_flash_attn_amd.quant_flash_attn import attn_bwd_shared_kv, attn_fwd_shared_kv
    o, lse = attn_fwd_shared_kv(q, codes, scale, zp, sm)
    dq, dkv = attn_bwd_shared_kv(q, codes, scale, zp, o, do, lse, sm)
    torch.cuda.synchronize()
    # a launch on the last 32 batch entries alone (512 heads: enough workgroups that the keys of a query
    # block are not split over several, as in the large launch) must reproduce their part bit for bit
    tail = slice(Z - 32, Z)
    args = (q[tail], codes[tail], scale[tail], zp[tail])
    o1, lse1 = attn_fwd_shared_kv(*args, sm)
    assert torch.equal(o[tail], o1) and torch.equal(lse[tail], lse1), "forward"
    dq1, dkv1 = attn_bwd_shared_kv(*args, o1, do[tail], lse1, sm)
    assert torch.equal(dq[tail], dq1), "dQ"
    assert torch.equal(dkv[tail], dkv1), "dKV"
    z, h = Z - 1, H - 1
    o_ref, _ = oracle.legacy_fwd(_head(q, z, h).cpu(), _head(codes, z, h).cpu(), _head(scale, z, h).cpu(),
                                 _head(zp, z, h).cpu(), sm)
    assert_close("O last head", _head(o, z, h).cpu(), o_ref, scaled=True)

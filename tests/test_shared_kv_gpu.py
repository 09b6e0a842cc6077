"""GPU parity of the shared-KV kernels (the reference's own operator: one quantized tensor serves
as K and V, Q stays in 16-bit float, quant_flash_attn.py:22-83) against the CPU oracle's literal
restatement in fp64.  Tolerances: O max-abs <= 2e-2 * max(1, max|O_ref|) and cosine >= 0.999, LSE
to 2^-8.  (V is the K tensor here, so with outlier channels |O| reaches ~60 and the rounding of a
16-bit output alone is 2^-11 of that; the bound scales with the largest reference value as it does
for the gradients.)"""
import math

import pytest
import torch

from helpers import REL_TOL, COS_TOL, assert_close, max_abs
from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LSE_TOL = 2.0 ** -8


def _inputs(config, B, H, Nq, Nk, D, dtype, seed):
    N = max(Nq, Nk)
    q, k, _, _ = make_inputs(config, B, H, N, D, seed=seed, dtype=dtype)
    return q[:, :, :Nq].contiguous(), k[:, :, :Nk].contiguous()


CASES = [
    # B, H, Nq, Nk, D, config, dtype, scale dtype
    (1, 2, 16, 32, 128, "normal", torch.float16, torch.float16),      # one tile, one wave busy
    (1, 2, 16, 128, 128, "normal", torch.float16, torch.float16),     # one tile per wave
    (2, 3, 16, 3000, 128, "normal", torch.float16, torch.float16),    # reference benchmark shape (compute_flops.py:96)
    (2, 3, 16, 3000, 64, "offset", torch.float16, torch.float16),
    (1, 2, 1, 1, 128, "normal", torch.float16, torch.float16),        # single query, single key
    (1, 2, 5, 33, 64, "uniform", torch.float16, torch.float32),       # ragged tail of one key
    (2, 2, 97, 689, 128, "offset", torch.bfloat16, torch.float32),    # four query blocks, ragged both ways
    (1, 2, 17, 1023, 128, "outlier", torch.float16, torch.float16),
    (1, 4, 32, 512, 64, "normal", torch.bfloat16, torch.bfloat16),
    (1, 2, 128, 4096, 128, "normal", torch.bfloat16, torch.float16),  # scale converted by the wrapper
    (2, 2, 16, 3000, 256, "normal", torch.float16, torch.float16),    # head_dim 256 (compute_flops.py:94)
    (1, 2, 37, 333, 256, "offset", torch.bfloat16, torch.float32),
    (1, 1, 3, 9000, 256, "uniform", torch.float16, torch.float16),    # split over keys
]


@pytest.mark.parametrize("B,H,Nq,Nk,D,config,dtype,sdtype", CASES)
def test_shared_kv_forward_vs_oracle(qfa, B, H, Nq, Nk, D, config, dtype, sdtype):
    q, kv = _inputs(config, B, H, Nq, Nk, D, dtype, seed=Nq + Nk + D)
    sm = 1.0 / math.sqrt(D)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV), scale_dtype=sdtype)
    o, lse = qfa.attn_fwd_shared_kv(q.to(DEV), codes, scale, zp, sm)
    torch.cuda.synchronize()
    o_ref, lse_ref = oracle.legacy_fwd(q, codes.cpu(), scale.cpu(), zp.cpu(), sm)
    assert o.dtype == dtype and o.shape == (B, H, Nq, D) and lse.shape == (B, H, Nq)
    assert_close("O", o.cpu(), o_ref, scaled=True)
    assert max_abs(lse.cpu(), lse_ref) < LSE_TOL


BWD_CASES = [
    # B, H, Nq, Nk, D, config, scale dtype
    (1, 2, 16, 32, 128, "normal", torch.float16),
    (1, 2, 16, 160, 128, "normal", torch.float16),       # tiles on every wave, a second one on wave 0
    (2, 3, 16, 3000, 128, "normal", torch.float16),      # reference benchmark shape (compute_flops.py:96)
    (2, 3, 16, 3000, 64, "offset", torch.float16),
    (1, 2, 1, 1, 128, "normal", torch.float16),
    (1, 2, 5, 33, 64, "uniform", torch.float32),
    (2, 2, 32, 689, 128, "offset", torch.float32),
    (1, 2, 17, 1023, 128, "outlier", torch.float16),
    (1, 4, 32, 512, 64, "normal", torch.float16),
    # more than 32 queries: dQ kernel + dKV kernel
    (2, 2, 97, 689, 128, "normal", torch.float16),       # reference test shape (test_accuracy.py:44), small batch
    (1, 3, 33, 100, 64, "offset", torch.float32),        # one query past a block, one key chunk
    (1, 2, 128, 1000, 128, "uniform", torch.float16),
    (2, 2, 64, 129, 64, "outlier", torch.float32),       # second key chunk holds a single key
    # head_dim 256 (compute_flops.py:94): one pass up to 16 queries; beyond, the two kernels (two waves share
    # a tile in the dKV kernel)
    (2, 2, 16, 3000, 256, "normal", torch.float16),
    (1, 2, 70, 161, 256, "offset", torch.float32),
    (1, 1, 1, 1, 256, "normal", torch.float16),
]


@pytest.mark.parametrize("B,H,Nq,Nk,D,config,sdtype", BWD_CASES)
def test_shared_kv_backward_vs_oracle(qfa, B, H, Nq, Nk, D, config, sdtype):
    """dQ and dKV = dV + dK (quant_flash_attn.py:153-161) against fp64 autograd-checked formulas on
    the dequantized tensor and the saved O; element-wise bound of helpers.assert_close and cosine >= 0.999."""
    q, kv = _inputs(config, B, H, Nq, Nk, D, torch.float16, seed=Nq + Nk + D)
    g = torch.Generator().manual_seed(Nk)
    do = torch.randn((B, H, Nq, D), generator=g).to(torch.float16)
    sm = 1.0 / math.sqrt(D)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV), scale_dtype=sdtype)
    o, lse = qfa.attn_fwd_shared_kv(q.to(DEV), codes, scale, zp, sm)
    dq, dkv = qfa.attn_bwd_shared_kv(q.to(DEV), codes, scale, zp, o, do.to(DEV), lse, sm)
    torch.cuda.synchronize()
    (dq_ref, dkv_ref), (nq, nkv) = oracle.legacy_bwd(q, codes.cpu(), scale.cpu(), zp.cpu(), do, sm, o=o.cpu(), spread=True)
    assert dq.shape == (B, H, Nq, D) and dkv.shape == (B, H, Nk, D) and dq.dtype == torch.float16
    # with a single key P = 1 and dS = 0: dQ is exactly zero and its cosine undefined
    assert_close("dQ", dq.cpu(), dq_ref, scaled=True, spread=nq, cos_tol=COS_TOL if Nk > 1 else -1.0)
    assert_close("dKV", dkv.cpu(), dkv_ref, scaled=True, spread=nkv)


@pytest.mark.parametrize("D", [128, 256, 64])
def test_shared_kv_entry_point_autograd(qfa, D):
    """The reference's entry point end to end on its benchmark shapes (compute_flops.py:94-96, small batch):
    forward and backward run the shared-KV kernels and kv_fp16 receives dKV (quant_flash_attn.py:178-237)."""
    B, H, Nq, Nk = 2, 4, 16, 3000
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=11)
    sm = 1.0 / math.sqrt(D)
    qd = q.to(DEV).requires_grad_(True)
    kvd = kv.to(DEV).requires_grad_(True)
    kv_quant = qfa.asymmetric_quant_per_token(kvd.detach())
    o = qfa.quant_flash_attn(qd, kvd, kv_quant, sm)
    do = torch.randn(o.shape, generator=torch.Generator().manual_seed(3)).to(torch.float16)
    o.backward(do.to(DEV))
    codes, scale, zp = (t.cpu() for t in kv_quant)
    o_ref, _ = oracle.legacy_fwd(q, codes, scale, zp, sm)
    dq_ref, dkv_ref = oracle.legacy_bwd(q, codes, scale, zp, do, sm)
    assert_close("O", o.detach().cpu(), o_ref, scaled=True)
    assert_close("dQ", qd.grad.cpu(), dq_ref, scaled=True)
    assert_close("dKV", kvd.grad.cpu(), dkv_ref, scaled=True)
    assert kvd.grad.dtype == torch.float16 and qd.grad.dtype == torch.float16


@pytest.mark.parametrize("do_scale,D", [(1.0, 128), (2.0 ** -22, 128), (1.0, 256)])
def test_shared_kv_entry_point_bf16(qfa, do_scale, D):
    """bf16 tensors through the reference's entry point: forward in the shared-KV kernel (queries rounded to
    binary16), backward in the binary16 kernels with dO scaled into range by a power of two -- also when
    dO is far below binary16's smallest normal number."""
    B, H, Nq, Nk = 2, 3, 16, 700
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.bfloat16, seed=31)
    sm = 1.0 / math.sqrt(D)
    qd = q.to(DEV).requires_grad_(True)
    kvd = kv.to(DEV).requires_grad_(True)
    kv_quant = qfa.asymmetric_quant_per_token(kvd.detach())
    o = qfa.quant_flash_attn(qd, kvd, kv_quant, sm)
    do = (torch.randn(o.shape, generator=torch.Generator().manual_seed(6)) * do_scale).to(torch.bfloat16)
    o.backward(do.to(DEV))
    assert o.dtype == torch.bfloat16 and qd.grad.dtype == torch.bfloat16 and kvd.grad.dtype == torch.bfloat16
    codes, scale, zp = (t.cpu() for t in kv_quant)
    o_ref, _ = oracle.legacy_fwd(q, codes, scale, zp, sm)
    dq_ref, dkv_ref = oracle.legacy_bwd(q, codes, scale, zp, do, sm)
    assert_close("O", o.detach().cpu(), o_ref, scaled=True)
    # gradients compared in units of dO's scale (the absolute bound of the contract assumes dO of order one)
    assert_close("dQ", qd.grad.cpu().double() / do_scale, dq_ref / do_scale, scaled=True, rel=REL_TOL[torch.bfloat16])
    assert_close("dKV", kvd.grad.cpu().double() / do_scale, dkv_ref / do_scale, scaled=True, rel=REL_TOL[torch.bfloat16])


@pytest.mark.parametrize("do_scale,kv_scale,Nq", [(2.0 ** -6, 1.0, 16), (2.0 ** -10, 1.0, 16), (2.0 ** -14, 1.0, 16),
                                                  (1.0, 2.0 ** -6, 16), (2.0 ** -10, 1.0, 70), (1.0, 2.0 ** -6, 70),
                                                  (1.0, 2.0 ** 6, 16), (1.0, 2.0 ** 8, 16), (1.0, 2.0 ** 8, 70)])
def test_shared_kv_entry_point_fp16_small_gradients(qfa, do_scale, kv_scale, Nq):
    """fp16 tensors with ordinary small gradients (and small K = V): the binary16 kernels do not multiply by dO
    itself but by sm_scale * p * (dP - delta) and that times the key scale, which underflow long before dO
    does; the entry point scales dO by a power of two around them.  One pass (16 queries) and the dQ + dKV
    kernels (70 queries); gradients compared in units of dO's scale.  Large K = V (key scales far above 2^-5, with the
    queries scaled down so that the softmax keeps its shape) must lower the power of two instead: the operand
    ds * scale_j would overflow binary16 otherwise."""
    B, H, Nk, D = 2, 3, 3000, 128
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=41)
    kv = (kv.float() * kv_scale).to(torch.float16)
    if kv_scale > 1.0:
        q = (q.float() / kv_scale).to(torch.float16)
    sm = 1.0 / math.sqrt(D)
    qd = q.to(DEV).requires_grad_(True)
    kvd = kv.to(DEV).requires_grad_(True)
    kv_quant = qfa.asymmetric_quant_per_token(kvd.detach())
    o = qfa.quant_flash_attn(qd, kvd, kv_quant, sm)
    do = (torch.randn(o.shape, generator=torch.Generator().manual_seed(7)) * do_scale).to(torch.float16)
    o.backward(do.to(DEV))
    codes, scale, zp = (t.cpu() for t in kv_quant)
    dq_ref, dkv_ref = oracle.legacy_bwd(q, codes, scale, zp, do, sm)
    unit = do_scale * kv_scale            # dQ scales with dO and with K = V
    # the gradients leave as float16 (as the reference's do): where they are tiny the reference values are
    # rounded to that format first, subnormals and all, so that the comparison is about the kernels
    r16 = lambda t: t.to(torch.float16).double()
    assert torch.isfinite(qd.grad).all() and torch.isfinite(kvd.grad).all()
    assert_close("dQ", qd.grad.cpu().double() / unit, r16(dq_ref) / unit, scaled=True, rel=REL_TOL[torch.float16])
    assert_close("dKV", kvd.grad.cpu().double() / do_scale, r16(dkv_ref) / do_scale, scaled=True, rel=REL_TOL[torch.float16])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("sdtype", [torch.float16, torch.float32])
@pytest.mark.parametrize("do_scale,kv_scale", [(1.0, 2.0 ** -5), (2.0 ** -14, 2.0 ** -5), (2.0 ** -20, 2.0 ** -11), (300.0, 2.0 ** -5),
                                               (1.0, 40.0), (3.0, 2.0 ** -16), (0.0, 1.0)])
def test_dout_normalisation_through_the_c_abi(qfa, dtype, sdtype, do_scale, kv_scale):
    """qfa_dout_normalise: out = binary16(dO * 2^k) and back = 2^-k, with k the largest integer such that
    max|dO| * 2^k * max|scale| <= 8 and max|dO| * 2^k <= 2^14 (the product of the two maxima taken in fp32) --
    computed here with exact integer arithmetic on the exponents; out and back bit for bit."""
    import numpy as np
    from quant_flash_attn_amd import _lib
    from quant_flash_attn_amd.quant_flash_attn import _normalised_dout
    g = torch.Generator().manual_seed(3)
    do = (torch.randn(3, 5, 17, 64, generator=g) * do_scale).to(dtype)
    do[1, 2, 3, 4] = do_scale * 4.0       # the maximum, an exact power of two when do_scale is one
    sc = (torch.rand(3, 5, 1003, generator=g) * kv_scale).to(sdtype)     # 15 045 scales: a tail after the 16-byte chunks
    if do_scale == 1.0 and kv_scale == 2.0 ** -5:
        sc[0, 0, 0] = 2.0 ** -5           # product of the maxima exactly 2^-3: k = 6, not 5
    amax = np.float32(max(float(do.float().abs().max()), 1e-30))
    smax = np.float32(max(float(sc.float().abs().max()), 1e-30))
    def floor_log2_quot(ce, y):           # floor(log2(2^ce / y)) for a positive float y
        m, e = math.frexp(float(y))       # y = m * 2^e, m in [0.5, 1)
        return ce - e + (1 if m == 0.5 else 0) if y > 0 else 10 ** 6
    k = min(floor_log2_quot(3, np.float32(amax * smax)), floor_log2_quot(14, amax))
    k = max(-100, min(100, k))
    do16, back = _normalised_dout(do.to(DEV), sc.to(DEV))
    pad = torch.cat([sc.flatten()[:1], sc.flatten()]).to(DEV)      # the same scales as a view that is not 16-byte aligned
    do16_b, back_b = _normalised_dout(do.to(DEV), pad[1:])
    assert torch.equal(do16_b, do16) and torch.equal(back_b, back)
    assert do16.dtype == torch.float16 and do16.shape == do.shape and back.dtype == torch.float32
    assert float(back.cpu()) == 2.0 ** -k, (float(back.cpu()), k)
    want = (do.double() * 2.0 ** k).to(torch.float16)
    assert torch.equal(do16.cpu().view(torch.int16), want.view(torch.int16))
    if do_scale > 0:
        top = float(amax) * 2.0 ** k
        assert top <= 2.0 ** 14 and (top * float(smax) > 4.0 * (1 - 1e-6) or top > 2.0 ** 13)


def test_shared_kv_entry_point_long_query_block(qfa):
    """97 queries (a reference test shape, test_accuracy.py:44): the forward splits them over workgroups
    of 16, the backward runs its dQ and dKV kernels."""
    B, H, Nq, Nk, D = 2, 3, 97, 689, 128
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=12)
    sm = 1.0 / math.sqrt(D)
    qd = q.to(DEV).requires_grad_(True)
    kvd = kv.to(DEV).requires_grad_(True)
    kv_quant = qfa.asymmetric_quant_per_token(kvd.detach())
    o = qfa.quant_flash_attn(qd, kvd, kv_quant, sm)
    do = torch.randn(o.shape, generator=torch.Generator().manual_seed(4)).to(torch.float16)
    o.backward(do.to(DEV))
    codes, scale, zp = (t.cpu() for t in kv_quant)
    o_ref, _ = oracle.legacy_fwd(q, codes, scale, zp, sm)
    dq_ref, dkv_ref = oracle.legacy_bwd(q, codes, scale, zp, do, sm)
    assert_close("O", o.detach().cpu(), o_ref, scaled=True)
    assert_close("dQ", qd.grad.cpu(), dq_ref, scaled=True)
    assert_close("dKV", kvd.grad.cpu(), dkv_ref, scaled=True)


@pytest.mark.parametrize("B,H,Nq,Nk,D,seed", [(1, 1, 5, 32, 128, 1158), (1, 3, 5, 33, 256, 1114), (1, 1, 130, 32, 256, 1091),
                                             (2, 2, 17, 1025, 256, 1068)])
def test_nearly_one_hot_softmax_gradient_floor(qfa, B, H, Nq, Nk, D, seed):
    """Scores that grow along the keys make the softmax nearly one-hot; dQ = sm * dS K is then a small
    difference of large terms and the 16-bit rounding of O (which enters delta = rowsum(O o dO), in the
    reference too: quant_flash_attn.py:97-99) alone moves it by a fifth of its size, so the cosine against
    an exact backward says nothing.  The bar here: the error stays within a small multiple of what that
    rounding causes in an otherwise exact fp64 backward, and within the absolute gradient tolerance."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((B, H, Nq, D), generator=g) * 0.2 + 1.0
    kv = torch.randn((B, H, Nk, D), generator=g) * 0.3 + torch.linspace(-1, 3, Nk).view(1, 1, Nk, 1)
    do = torch.randn((B, H, Nq, D), generator=g)
    q, kv, do = q.half(), kv.half(), do.half()
    sm = 1.0 / math.sqrt(D)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV))
    o, lse = qfa.attn_fwd_shared_kv(q.to(DEV), codes, scale, zp, sm)
    dq, dkv = qfa.attn_bwd_shared_kv(q.to(DEV), codes, scale, zp, o, do.to(DEV), lse, sm)
    c, s_, z = codes.cpu(), scale.cpu(), zp.cpu()
    dq_ref, dkv_ref = oracle.legacy_bwd(q, c, s_, z, do, sm)
    kvh = (c.double() - z.double()) * s_.double()
    P = torch.softmax(sm * (q.double() @ kvh.transpose(-1, -2)), -1)
    delta16 = ((P @ kvh).half().double() * do.double()).sum(-1, keepdim=True)     # the only rounding kept
    dq_floor = sm * (P * (do.double() @ kvh.transpose(-1, -2) - delta16)) @ kvh
    floor = max_abs(dq_floor, dq_ref)
    err = max_abs(dq.cpu(), dq_ref)
    assert err <= 3.0 * floor + 2.0 ** -11 * float(dq_ref.abs().max()) + 1e-4, (err, floor)
    assert err <= 2e-2 * max(1.0, float(dq_ref.abs().max()))
    assert_close("dKV", dkv.cpu(), dkv_ref, scaled=True)


def test_entry_point_head_dim_256_beyond_the_query_limit(qfa):
    """600 queries at head_dim 256: longer than the query blocks the shared-KV kernels are normally given, but
    the INT8-score kernels stop at head_dim 128, so the reference's entry point keeps them on this path."""
    B, H, Nq, Nk, D = 1, 2, 600, 700, 256
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=21)
    sm = 1.0 / math.sqrt(D)
    qd = q.to(DEV).requires_grad_(True)
    kvd = kv.to(DEV).requires_grad_(True)
    kv_quant = qfa.asymmetric_quant_per_token(kvd.detach())
    o = qfa.quant_flash_attn(qd, kvd, kv_quant, sm)
    do = torch.randn(o.shape, generator=torch.Generator().manual_seed(4)).to(torch.float16)
    o.backward(do.to(DEV))
    codes, scale, zp = (t.cpu() for t in kv_quant)
    o_ref, _ = oracle.legacy_fwd(q, codes, scale, zp, sm)
    dq_ref, dkv_ref = oracle.legacy_bwd(q, codes, scale, zp, do, sm)
    assert_close("O", o.detach().cpu(), o_ref, scaled=True)
    assert_close("dQ", qd.grad.cpu(), dq_ref, scaled=True)
    assert_close("dKV", kvd.grad.cpu(), dkv_ref, scaled=True)


@pytest.mark.parametrize("B,H,Nq,Nk,D", [(1, 2, 16, 4096, 128), (1, 1, 1, 20000, 64), (2, 3, 40, 3001, 128), (1, 8, 5, 1023, 64)])
def test_shared_kv_forward_split_over_keys(qfa, B, H, Nq, Nk, D):
    """Few (batch, head) pairs: the wrapper hands the library a workspace and the keys of a query block are
    split over several workgroups, merged by a second kernel.  Same oracle, same bars; and the split result
    agrees with the unsplit one (workspace = NULL) to a rounding of the output."""
    from quant_flash_attn_amd import _lib
    assert _lib.lib().qfa_attn_fwd_shared_kv_workspace_bytes(B, H, Nq, Nk, D) > 0
    assert _lib.lib().qfa_attn_fwd_shared_kv_workspace_bytes(512, 16, 16, 3000, 128) == 0
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=Nk)
    sm = 1.0 / math.sqrt(D)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV))
    qd = q.to(DEV)
    o, lse = qfa.attn_fwd_shared_kv(qd, codes, scale, zp, sm)
    o1 = torch.empty_like(o)
    lse1 = torch.empty_like(lse)
    s3 = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    rc = _lib.lib().qfa_attn_fwd_shared_kv(qd.data_ptr(), codes.data_ptr(), scale.data_ptr(), _lib.QFA_F16, zp.data_ptr(),
                                           o1.data_ptr(), lse1.data_ptr(), _lib.QFA_F16, B, H, Nq, Nk, D, *s3(qd), *s3(codes),
                                           *s3(o1), sm, None, 0, _lib.stream_of(qd))
    assert rc == 0
    torch.cuda.synchronize()
    o_ref, lse_ref = oracle.legacy_fwd(q, codes.cpu(), scale.cpu(), zp.cpu(), sm)
    assert_close("O", o.cpu(), o_ref, scaled=True)
    assert max_abs(lse.cpu(), lse_ref) < LSE_TOL
    assert max_abs(o.cpu(), o1.cpu()) <= 2.0 ** -9 * max(1.0, float(o_ref.abs().max()))
    assert max_abs(lse.cpu(), lse1.cpu()) < 1e-4


def test_shared_kv_offsets_cancel(qfa):
    """Every token with the same nonzero codes and extreme zero points: the 1152-offset terms the
    kernel adds to make the codes binary16 operands are orders of magnitude above the result and
    must cancel exactly.  O = the common dequantized row, whatever the softmax weights."""
    B, H, Nq, Nk, D = 1, 2, 16, 96, 128
    g = torch.Generator().manual_seed(5)
    row = torch.randint(-128, 128, (1, 1, 1, D), generator=g, dtype=torch.int32).to(torch.int8)
    codes = row.expand(B, H, Nk, D).contiguous()
    zp = torch.full((B, H, Nk, 1), -128, dtype=torch.int8)
    scale = torch.full((B, H, Nk, 1), 0.03125, dtype=torch.float16)
    q = torch.randn((B, H, Nq, D), generator=g).to(torch.float16)
    o, lse = qfa.attn_fwd_shared_kv(q.to(DEV), codes.to(DEV), scale.to(DEV), zp.to(DEV), 0.1)
    want = ((row.double() + 128.0) * 0.03125).expand(B, H, Nq, D)
    assert max_abs(o.cpu(), want) <= 2.0 ** -9 * float(want.abs().max())   # one fp16 rounding of the output
    o_ref, lse_ref = oracle.legacy_fwd(q, codes, scale, zp, 0.1)
    assert max_abs(lse.cpu(), lse_ref) < LSE_TOL


def test_shared_kv_strided_views(qfa):
    """q and the codes handed over as views of larger buffers (token stride > D)."""
    B, H, Nq, Nk, D = 2, 2, 16, 200, 64
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=9)
    sm = 0.125
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV))
    big_c = torch.zeros((B, H, Nk, 2 * D), dtype=torch.int8, device=DEV)
    big_c[..., :D] = codes
    big_q = torch.zeros((B, H, Nq, 3 * D), dtype=torch.float16, device=DEV)
    big_q[..., D:2 * D] = q.to(DEV)
    o1, l1 = qfa.attn_fwd_shared_kv(q.to(DEV), codes, scale, zp, sm)
    o2, l2 = qfa.attn_fwd_shared_kv(big_q[..., D:2 * D], big_c[..., :D], scale, zp, sm)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)


def test_shared_kv_rejects_bad_arguments(qfa):
    q = torch.zeros((1, 1, 16, 96), dtype=torch.float16, device=DEV)
    codes = torch.zeros((1, 1, 64, 96), dtype=torch.int8, device=DEV)
    scale = torch.ones((1, 1, 64, 1), dtype=torch.float16, device=DEV)
    zp = torch.zeros((1, 1, 64, 1), dtype=torch.int8, device=DEV)
    with pytest.raises(RuntimeError, match="head_dim"):
        qfa.attn_fwd_shared_kv(q, codes, scale, zp, 0.1)
    with pytest.raises(TypeError):
        qfa.attn_fwd_shared_kv(q.float(), codes, scale, zp, 0.1)


@pytest.mark.parametrize("B,H,Nq,Nk", [(2, 3, 16, 700), (1, 2, 40, 2100)])
def test_shared_kv_graph_capture_and_replay(qfa, B, H, Nq, Nk):
    """Quantizer + shared-KV forward + backward captured into a HIP graph (the second shape also takes the
    split over keys with its merge kernel and the two-kernel backward): the library only enqueues kernels,
    so replays with new contents in the static inputs reproduce the eager results bit for bit."""
    D = 128
    sm = 1.0 / math.sqrt(D)
    st_q = torch.zeros(B, H, Nq, D, dtype=torch.float16, device=DEV)
    st_kv = torch.zeros(B, H, Nk, D, dtype=torch.float16, device=DEV)
    st_do = torch.zeros(B, H, Nq, D, dtype=torch.float16, device=DEV)

    def step(q, kv, do):
        codes, scale, zp = qfa.asymmetric_quant_per_token(kv)
        o, lse = qfa.attn_fwd_shared_kv(q, codes, scale, zp, sm)
        dq, dkv = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, do, lse, sm)
        return o, lse, dq, dkv

    def make(seed):
        q, kv = _inputs(("normal", "offset", "outlier")[seed % 3], B, H, Nq, Nk, D, torch.float16, seed=50 + seed)
        do = torch.randn(q.shape, generator=torch.Generator().manual_seed(seed)).to(torch.float16)
        return q.to(DEV), kv.to(DEV), do.to(DEV)

    inputs = [make(i) for i in range(3)]
    for s, t in zip((st_q, st_kv, st_do), inputs[0]):
        s.copy_(t)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(st_q, st_kv, st_do)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(st_q, st_kv, st_do)
    for rep in range(2):
        for inp in inputs:
            eager = step(*inp)
            torch.cuda.synchronize()
            for s, t in zip((st_q, st_kv, st_do), inp):
                s.copy_(t)
            graph.replay()
            torch.cuda.synchronize()
            for name, a_, b_ in zip(("O", "LSE", "dQ", "dKV"), outs, eager):
                assert torch.equal(a_, b_), f"graph replay differs from eager: {name} (round {rep})"


def test_shared_kv_full_reference_test_shape(qfa):
    """The reference's largest accuracy shape at FULL size (test_accuracy.py:44: Z=99, H=53, 97 queries, 689 keys,
    head_dim 128; 5247 (batch, head) pairs): the forward runs 7 workgroups of 16 queries per pair, the backward its dQ
    and dKV kernels with their key-chunk plan at a large pair count.  Sampled pairs against the dense fp64 oracle,
    determinism, and a zero dO giving exactly zero gradients."""
    Z, H, Nq, Nk, D = 99, 53, 97, 689, 128
    g = torch.Generator(device=DEV).manual_seed(20)
    q = torch.randn((Z, H, Nq, D), generator=g, device=DEV, dtype=torch.float16)
    kv = torch.randn((Z, H, Nk, D), generator=g, device=DEV, dtype=torch.float16)
    do = torch.randn((Z, H, Nq, D), generator=g, device=DEV, dtype=torch.float16)
    sm = 1.0 / math.sqrt(D)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv)
    del kv
    o, lse = qfa.attn_fwd_shared_kv(q, codes, scale, zp, sm)
    dq, dkv = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, do, lse, sm)
    dq2, dkv2 = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, do, lse, sm)
    dq0, dkv0 = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, torch.zeros_like(do), lse, sm)
    torch.cuda.synchronize()
    assert torch.equal(dq, dq2) and torch.equal(dkv, dkv2)
    assert float(dq0.abs().max()) == 0.0 and float(dkv0.abs().max()) == 0.0
    assert torch.isfinite(o.float()).all() and torch.isfinite(dq.float()).all() and torch.isfinite(dkv.float()).all()
    for b, h in ((0, 0), (41, 17), (98, 52)):
        sl = lambda t: t[b:b + 1, h:h + 1].cpu()
        o_ref, lse_ref = oracle.legacy_fwd(sl(q), sl(codes), sl(scale), sl(zp), sm)
        (dq_ref, dkv_ref), (nq, nkv) = oracle.legacy_bwd(sl(q), sl(codes), sl(scale), sl(zp), sl(do), sm, o=sl(o), spread=True)
        assert_close(f"O[{b},{h}]", sl(o), o_ref, scaled=True)
        assert max_abs(sl(lse), lse_ref) < LSE_TOL
        assert_close(f"dQ[{b},{h}]", sl(dq), dq_ref, scaled=True, spread=nq)
        assert_close(f"dKV[{b},{h}]", sl(dkv), dkv_ref, scaled=True, spread=nkv)


@pytest.mark.parametrize("D", [128, 64])
def test_shared_kv_full_benchmark_size(qfa, D):
    """The reference's benchmark shape at full size (compute_flops.py:96: Z=512, H=16, 16 queries, 3000 keys):
    sampled (batch, head) slices against the dense fp64 oracle, plus size-independent properties --
    determinism (two runs bit-identical), softmax weights summing to one (a constant channel of kv comes out
    of O as that constant), and a zero dO giving exactly zero gradients."""
    Z, H, Nq, Nk = 512, 16, 16, 3000
    g = torch.Generator(device=DEV).manual_seed(7)
    q = torch.randn((Z, H, Nq, D), generator=g, device=DEV, dtype=torch.float16)
    kv = torch.randn((Z, H, Nk, D), generator=g, device=DEV, dtype=torch.float16)
    kv[..., 0] = 1.0                                   # a constant channel: O[..., 0] must be 1
    do = torch.randn((Z, H, Nq, D), generator=g, device=DEV, dtype=torch.float16)
    sm = 1.0 / math.sqrt(D)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv)
    del kv
    o, lse = qfa.attn_fwd_shared_kv(q, codes, scale, zp, sm)
    dq, dkv = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, do, lse, sm)
    o2, lse2 = qfa.attn_fwd_shared_kv(q, codes, scale, zp, sm)
    dq2, dkv2 = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, do, lse, sm)
    torch.cuda.synchronize()
    assert torch.equal(o, o2) and torch.equal(lse, lse2) and torch.equal(dq, dq2) and torch.equal(dkv, dkv2)
    # the constant channel dequantizes to 1 up to one quantization step; softmax weights sum to one
    kv0 = (codes[..., 0].float() - zp[..., 0].float()) * scale[..., 0].float()
    assert float((o[..., 0].float() - 1.0).abs().max()) <= float((kv0 - 1.0).abs().max()) + 2.0 ** -9
    dq0, dkv0 = qfa.attn_bwd_shared_kv(q, codes, scale, zp, o, torch.zeros_like(do), lse, sm)
    assert float(dq0.abs().max()) == 0.0 and float(dkv0.abs().max()) == 0.0
    for b, h in ((0, 0), (137, 5), (511, 15)):
        sl = lambda t: t[b:b + 1, h:h + 1].cpu()
        o_ref, lse_ref = oracle.legacy_fwd(sl(q), sl(codes), sl(scale), sl(zp), sm)
        dq_ref, dkv_ref = oracle.legacy_bwd(sl(q), sl(codes), sl(scale), sl(zp), sl(do), sm)
        assert_close(f"O[{b},{h}]", sl(o), o_ref, scaled=True)
        assert max_abs(sl(lse), lse_ref) < LSE_TOL
        assert_close(f"dQ[{b},{h}]", sl(dq), dq_ref, scaled=True)
        assert_close(f"dKV[{b},{h}]", sl(dkv), dkv_ref, scaled=True)


@pytest.mark.parametrize("Nq", [16, 48])
def test_shared_kv_backward_strided_views(qfa, Nq):
    """q, o, dO, the codes and the gradient buffers handed over as views of larger buffers (token stride
    > D, [B,N,H,D] storage): same bits as with dense tensors, through the C entry point directly."""
    from quant_flash_attn_amd import _lib
    B, H, Nk, D = 2, 3, 300, 64
    q, kv = _inputs("normal", B, H, Nq, Nk, D, torch.float16, seed=21)
    do = torch.randn(q.shape, generator=torch.Generator().manual_seed(5)).to(torch.float16)
    sm = 0.125
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV))
    qd, dod = q.to(DEV), do.to(DEV)
    o, lse = qfa.attn_fwd_shared_kv(qd, codes, scale, zp, sm)
    dq, dkv = qfa.attn_bwd_shared_kv(qd, codes, scale, zp, o, dod, lse, sm)

    def bnhd(t, pad):   # [B,N,H,D+pad] storage viewed as [B,H,N,D]
        buf = torch.zeros((t.shape[0], t.shape[2], t.shape[1], t.shape[3] + pad), dtype=t.dtype, device=DEV)
        view = buf.permute(0, 2, 1, 3)[..., :t.shape[3]]
        view.copy_(t)
        return view
    q_v, o_v, do_v, c_v = bnhd(qd, 8), bnhd(o, 16), bnhd(dod, 0), bnhd(codes, 64)
    dq_v, dkv_v = bnhd(torch.zeros_like(dq), 24), bnhd(torch.zeros_like(dkv), 8)
    s3 = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    rc = _lib.lib().qfa_attn_bwd_shared_kv(
        q_v.data_ptr(), c_v.data_ptr(), scale.data_ptr(), _lib.QFA_F16, zp.data_ptr(), o_v.data_ptr(), do_v.data_ptr(),
        lse.data_ptr(), dq_v.data_ptr(), dkv_v.data_ptr(), _lib.QFA_F16, _lib.QFA_F16, None, B, H, Nq, Nk, D,
        *s3(q_v), *s3(c_v), *s3(o_v), *s3(do_v), *s3(dq_v), *s3(dkv_v), sm, _lib.stream_of(qd))
    assert rc == 0, _lib.lib().qfa_last_error()
    torch.cuda.synchronize()
    assert torch.equal(dq_v, dq) and torch.equal(dkv_v, dkv)


@pytest.mark.parametrize("Nq", [16, 40])
def test_shared_kv_large_row_sums(qfa, Nq):
    """Row sums of q beyond 2^15, where the rank-1 offset removal switches to its x32 scaling (without it the
    correction operand overflows binary16 and O is NaN).  (c*q, sm_scale/c) is the same attention problem as
    (q, sm_scale): O and dKV must not change and dQ must scale by 1/c, although the first run takes the x32
    path and the second does not; both also match the fp64 oracle."""
    B, H, Nk, D, c = 1, 2, 500, 128, 256.0
    g = torch.Generator().manual_seed(17)
    q = (2.0 + 0.1 * torch.randn((B, H, Nq, D), generator=g)).to(torch.float16)
    kv = torch.randn((B, H, Nk, D), generator=g).to(torch.float16)
    do = torch.randn((B, H, Nq, D), generator=g).to(torch.float16)
    sm = 1.0 / math.sqrt(D)
    qc = (q.float() * c).to(torch.float16)          # exact: a power of two
    assert float(qc.float().sum(-1).abs().min()) > 32768.0 and float(q.float().sum(-1).abs().max()) < 32768.0
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv.to(DEV))
    outs = []
    for qq, s_ in ((q, sm), (qc, sm / c)):
        o, lse = qfa.attn_fwd_shared_kv(qq.to(DEV), codes, scale, zp, s_)
        dq, dkv = qfa.attn_bwd_shared_kv(qq.to(DEV), codes, scale, zp, o, do.to(DEV), lse, s_)
        outs.append((o.cpu(), lse.cpu(), dq.cpu(), dkv.cpu()))
    (o1, l1, dq1, dkv1), (o2, l2, dq2, dkv2) = outs
    assert max_abs(o1, o2) <= 2.0 ** -9 * float(o1.abs().max()) and max_abs(l1, l2) < 1e-3
    assert max_abs(dkv1, dkv2) <= 2e-3 * max(1.0, float(dkv1.abs().max()))
    # dS is held in binary16 with sm_scale folded in: an sm_scale 256 times smaller than usual pushes it into
    # the subnormal range, so dQ of the second run agrees to the gradient tolerance only
    assert max_abs(dq1, dq2.float() * c) <= 2e-2 * max(1.0, float(dq1.abs().max()))
    o_ref, lse_ref = oracle.legacy_fwd(qc, codes.cpu(), scale.cpu(), zp.cpu(), sm / c)
    dq_ref, dkv_ref = oracle.legacy_bwd(qc, codes.cpu(), scale.cpu(), zp.cpu(), do, sm / c)
    assert_close("O", o2, o_ref, scaled=True)
    assert max_abs(l2, lse_ref) < LSE_TOL
    assert_close("dQ", dq2.double() * c, dq_ref * c, scaled=True, rel=REL_TOL[dq2.dtype])
    assert_close("dKV", dkv2, dkv_ref, scaled=True)

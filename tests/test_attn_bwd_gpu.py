"""GPU parity of the HIP backward kernels against the CPU oracle: closed-form / autograd gradients
of fp64 attention on the dequantized Q^, K^ (quant_flash_attn.py:153-164 restated, K and V
separate).  Bar, for every element of dQ, dK, dV:  |got - want| <= 2e-2 + ulp * (|want| + spread)  with ulp the
rounding step of the output type and spread the 2-norm of the summed terms, and cosine >= 0.999
(helpers.py says where the two relative terms come from)."""
import math

import pytest
import torch

from helpers import assert_close, max_abs, rounded_output_floor
from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _fwd_bwd(qfa, q, k, v, do, causal, sm):
    qq = qfa.quantize_for_attention(q.to(DEV))
    kq = qfa.quantize_for_attention(k.to(DEV))
    vg, dog = v.to(DEV), do.to(DEV)
    o, lse = qfa.attn_fwd_quantized(qq, kq, vg, causal, sm)
    dq, dk, dv = qfa.attn_bwd_quantized(qq, kq, vg, o, dog, lse, causal, sm)
    torch.cuda.synchronize()
    return qq, kq, o, lse, dq, dk, dv


def _oracle_bwd(qq, kq, v, do, o, causal, sm, b=None, h=None):
    """((dQ, dK, dV), (their spreads)) from the closed forms in fp64, given what the kernel is given: the codes and
    the saved 16-bit O (the reference's backward takes delta from the saved o too, quant_flash_attn.py:97-99)."""
    sel = (lambda t: t.cpu()) if b is None else (lambda t: t.cpu()[b:b + 1, h:h + 1])
    qh = oracle.dequantize_per_token(sel(qq.codes), sel(qq.scale), sel(qq.zero_point), torch.float64)
    kh = oracle.dequantize_per_token(sel(kq.codes), sel(kq.scale), sel(kq.zero_point), torch.float64)
    return oracle.attn_bwd(qh, kh, sel(v), sel(do), causal, sm, o=sel(o), spread=True)


def _check_grads(tag, got, want, spreads, rel=None):
    for name, g, w, sp in zip(("dQ", "dK", "dV"), got, want, spreads):
        assert_close(name + tag, g, w, scaled=True, spread=sp, rel=rel)


CASES = [
    (1, 2, 128, 128, 128, False, "normal", torch.bfloat16),
    (1, 2, 128, 128, 128, True, "offset", torch.bfloat16),
    (2, 3, 384, 384, 128, True, "offset", torch.bfloat16),
    (1, 4, 256, 256, 64, False, "normal", torch.bfloat16),
    (2, 2, 512, 512, 64, True, "uniform", torch.bfloat16),
    (1, 2, 1024, 1024, 128, False, "outlier", torch.bfloat16),
    (1, 2, 200, 200, 128, False, "offset", torch.bfloat16),     # ragged
    (1, 3, 333, 333, 64, True, "uniform", torch.bfloat16),      # ragged, causal
    (2, 2, 97, 689, 128, False, "normal", torch.bfloat16),      # short Q, long ragged KV
    (1, 2, 640, 640, 128, True, "offset", torch.float16),
    # causal with many heads: the kernels dispatch the blocks of a group of heads together; 12 and 19 heads
    # leave a partial group at the end, 16 fills two groups of eight
    (3, 4, 320, 320, 64, True, "normal", torch.bfloat16),
    (1, 19, 300, 300, 128, True, "offset", torch.bfloat16),
    (2, 8, 512, 512, 64, True, "uniform", torch.float16),
    # head_dim 256: 32-row tiles, one wave per SIMD
    (1, 2, 128, 128, 256, False, "normal", torch.bfloat16),
    (2, 3, 384, 384, 256, True, "offset", torch.bfloat16),
    (1, 2, 512, 512, 256, True, "outlier", torch.float16),
    (1, 2, 333, 333, 256, True, "uniform", torch.bfloat16),     # ragged, causal
    (2, 2, 97, 689, 256, False, "offset", torch.float16),       # short Q, long ragged KV
    (1, 3, 200, 200, 256, False, "uniform", torch.bfloat16),    # ragged
    # causal with fewer queries than keys: the mask is aligned to the last key
    (2, 2, 128, 384, 128, True, "normal", torch.bfloat16),
    (1, 3, 97, 689, 128, True, "offset", torch.float16),        # ragged both ways, offset 592
    (1, 2, 200, 333, 64, True, "uniform", torch.bfloat16),
    (1, 2, 1, 300, 128, True, "normal", torch.bfloat16),        # one query: sees every key
    (2, 2, 160, 200, 256, True, "offset", torch.bfloat16),
]


@pytest.mark.parametrize("B,H,Nq,Nk,D,causal,config,dtype", CASES)
def test_backward_vs_oracle(qfa, B, H, Nq, Nk, D, causal, config, dtype):
    N = max(Nq, Nk)
    q, k, v, do = make_inputs(config, B, H, N, D, seed=Nq + D + 1, dtype=dtype)
    q, do = q[:, :, :Nq].contiguous(), do[:, :, :Nq].contiguous()
    k, v = k[:, :, :Nk].contiguous(), v[:, :, :Nk].contiguous()
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse, dq, dk, dv = _fwd_bwd(qfa, q, k, v, do, causal, sm)
    want, spreads = _oracle_bwd(qq, kq, v, do, o, causal, sm)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape and dq.dtype == dtype
    _check_grads("", (dq.cpu(), dk.cpu(), dv.cpu()), want, spreads)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("sharp", [False, True])
def test_extreme_row_sums_and_zero_points(qfa, D, sharp):
    """Rows that sit entirely at one end of their range: zero point -128 with codes near +127 and zero point +127
    with codes near -128, so that rq - D*zq comes close to +-255*D (65 280 at head_dim 256, where it no longer splits into
    two 7-bit digits) and the code row sums reach +-127*D.  The integer zero-point correction of the score kernels
    has to stay exact for every pairing of such query and key rows, forward and backward.
    With sm_scale = 1/sqrt(D) the scores of these rows lie within +-0.1 and the gradients below the absolute bar
    (a loose check); `sharp` takes sm_scale = 8192 / D, which puts the scores of like-signed rows tens of units above the rest and
    spreads them over a few units among themselves: an error in a high
    digit of the correction (2^16 integer units are 0.2 to 0.8 of a score then) would redistribute the probabilities and
    move dK and dV by many times the bar."""
    B, H, N = 1, 2, 192
    g = torch.Generator().manual_seed(D)
    def rows():
        x = torch.randn((B, H, N, D), generator=g) * 0.05
        hi = 0.08 * (0.97 + 0.03 * torch.rand((B, H, N, D), generator=g))
        hi[..., 0] = 0.0
        x[:, :, 0::3] = hi[:, :, 0::3]          # all positive, minimum 0: zero point -128, codes near +127
        x[:, :, 1::3] = -hi[:, :, 1::3]         # all negative, maximum 0: zero point +127, codes near -128
        return x.to(torch.bfloat16)
    q, k = rows(), rows().flip(2)
    v = torch.randn((B, H, N, D), generator=g).to(torch.bfloat16)
    do = torch.randn((B, H, N, D), generator=g).to(torch.bfloat16)
    sm = 8192.0 / D if sharp else 1.0 / math.sqrt(D)
    for causal in (False, True):
        qq, kq, o, lse, dq, dk, dv = _fwd_bwd(qfa, q, k, v, do, causal, sm)
        c = qq.rowsum.cpu().long().reshape(B, H, N) - D * qq.zero_point.cpu().long().reshape(B, H, N)
        assert c.max() > 240 * D and c.min() < -240 * D, "the inputs do not reach the range they are meant to test"
        assert kq.rowsum.abs().max() > 120 * D
        qh = oracle.dequantize_per_token(qq.codes.cpu(), qq.scale.cpu(), qq.zero_point.cpu(), torch.float64)
        kh = oracle.dequantize_per_token(kq.codes.cpu(), kq.scale.cpu(), kq.zero_point.cpu(), torch.float64)
        o_ref, lse_ref = oracle.attn_fwd(qh, kh, v, causal, sm)
        assert_close(f"O causal={causal}", o.cpu(), o_ref)
        assert max_abs(lse.cpu(), lse_ref) < 2.0 ** -8
        want, spreads = _oracle_bwd(qq, kq, v, do, o, causal, sm)
        if sharp:   # the check has teeth only if the gradients stand clear of the absolute bar
            assert float(want[1].pow(2).mean().sqrt()) > 2e-2 and float(want[2].pow(2).mean().sqrt()) > 2e-2
        # sharp: P, dS and the dequantized operand each enter the matrix pipe rounded to 8 bits, i.e. the error of an
        # element has a standard deviation of 2^-9 of its spread, and the usual relative bar of 2^-7 is four of those:
        # the largest of 10^5 elements of these heavy-tailed sums passes that now and then (measured 2^-6.7).  The errors
        # this case is after are tens of percent.
        _check_grads(f" causal={causal}", (dq.cpu(), dk.cpu(), dv.cpu()), want, spreads, rel=2.0 ** -6 if sharp else None)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_backward_constant_rows_at_the_clamps(qfa, D, causal):
    """The backward twin of the forward test of the same name: constant rows of +-300 (scale 1, codes +127 / -128,
    zero points -128 / +127) between random rows.  These rows drive every term of the zero-point correction of both
    backward kernels to the end of its range (rq - D*zq = +-255 D, row sums +-128 D, integer scores +-255^2 D).
    sm_scale = 1e-3: a constant query then spreads its weight evenly over the constant keys of its sign (scores of
    +-8 000 at head_dim 128), a random query sees scores of a few units, and a correction that is off in a digit
    (128 integer units or more: 0.13 of a score) would move the probabilities, dV = P^T dO and dK = sm dS^T Q^
    by ten percent and more.  (A ONE-unit error cannot be seen from the backward at all: it recomputes P from the
    saved fp32 LSE, whose last bit is worth one integer unit at the end of the range, in the reference too; the
    forward test pins single units through O.)"""
    B, H, N = 1, 2, 96
    g = torch.Generator().manual_seed(5 * D + causal)
    def rows():
        x = torch.randn((B, H, N, D), generator=g)
        x[:, :, 0::3] = 300.0
        x[:, :, 1::3] = -300.0
        return x.to(torch.bfloat16)
    q, k = rows(), rows()
    v = torch.randn((B, H, N, D), generator=g).to(torch.bfloat16)
    do = torch.randn((B, H, N, D), generator=g).to(torch.bfloat16)
    sm = 1e-3
    qq, kq, o, lse, dq, dk, dv = _fwd_bwd(qfa, q, k, v, do, causal, sm)
    assert qq.codes[0, 0, 0].eq(127).all() and qq.zero_point[0, 0, 0].item() == -128
    assert kq.codes[0, 0, 1].eq(-128).all() and kq.zero_point[0, 0, 1].item() == 127
    want, spreads = _oracle_bwd(qq, kq, v, do, o, causal, sm)
    for w in want:   # the check has teeth only if the gradients stand clear of the absolute bar
        assert float(w.pow(2).mean().sqrt()) > 2e-2
    _check_grads(f" causal={causal}", (dq.cpu(), dk.cpu(), dv.cpu()), want, spreads)


@pytest.mark.parametrize("D", [64, 128, 256])
def test_delta_kernel(qfa, D):
    from quant_flash_attn_amd import _lib
    o = torch.randn(2, 3, 130, D, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    do = torch.randn(2, 3, 130, D, generator=torch.Generator().manual_seed(2)).to(torch.bfloat16)
    og, dog = o.to(DEV), do.to(DEV)
    delta = torch.empty(2, 3, 130, dtype=torch.float32, device=DEV)
    s = (og.stride(0), og.stride(1), og.stride(2))
    rc = _lib.lib().qfa_bwd_delta(og.data_ptr(), dog.data_ptr(), delta.data_ptr(), _lib.QFA_BF16, 2, 3, 130, D,
                                  *s, *s, torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "qfa_bwd_delta")
    assert max_abs(delta.cpu(), oracle.bwd_delta(o, do)) < 1e-4


@pytest.mark.parametrize("config,B,H,N,D,causal", [("offset", 4, 32, 4096, 128, True),
                                                   ("uniform", 16, 16, 2048, 64, True),
                                                   ("outlier", 1, 16, 16384, 128, False)])
def test_full_size_sampled_heads_and_properties(qfa, config, B, H, N, D, causal):
    q, k, v, do = make_inputs(config, B, H, N, D, seed=0)
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse, dq, dk, dv = _fwd_bwd(qfa, q, k, v, do, causal, sm)
    for t in (dq, dk, dv):
        assert torch.isfinite(t.float()).all()
    if N <= 4096:   # dense fp64 oracle on two heads
        for (b, h) in [(0, 0), (B - 1, H - 1)]:
            want, spreads = _oracle_bwd(qq, kq, v, do, o, causal, sm, b, h)
            _check_grads(f"[{b},{h}]", tuple(t.cpu()[b:b + 1, h:h + 1] for t in (dq, dk, dv)), want, spreads)
    # gradients are linear in dO: doubling dO doubles them (exactly, except where 16-bit
    # intermediates fall into the subnormal range, hence a tolerance of one part in 2^9)
    dq2, dk2, dv2 = qfa.attn_bwd_quantized(qq, kq, v.to(DEV), o, do.to(DEV) * 2, lse, causal, sm)
    for a2, a1 in ((dq2, dq), (dk2, dk), (dv2, dv)):
        assert (a2.float() - 2 * a1.float()).abs().max() <= 2.0 ** -8 * float(a1.float().abs().max())
    # softmax rows sum to one => each row of dS sums to zero => dQ vanishes when K^ rows are all equal;
    # cheaper size-independent check used here: dV summed over keys equals dO summed over queries
    # weighted by rows of P that sum to one:  sum_j dV[j] = sum_i dO[i]
    lhs = dv.float().sum(2)
    rhs = do.to(DEV).float().sum(2)
    assert (lhs - rhs).abs().max() < 0.02 * math.sqrt(N)


@pytest.mark.parametrize("D", [128, 256])
def test_autograd_entry_points(qfa, D):
    """quant_flash_attn_qkv(q,k,v,causal,sm) and the reference-style quant_flash_attn(q, kv, kv_quant, sm)."""
    B, H, N = 2, 2, 256
    q, k, v, do = make_inputs("offset", B, H, N, D, seed=21)
    sm = 1.0 / math.sqrt(D)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    o = qfa.quant_flash_attn_qkv(qg, kg, vg, True, sm)
    o.backward(do.to(DEV))
    qc, _, zq, sq, _ = oracle.quantize_per_token(q)
    kc, _, zk, sk, _ = oracle.quantize_per_token(k)
    qh, kh = oracle.dequantize_per_token(qc, sq, zq, torch.float64), oracle.dequantize_per_token(kc, sk, zk, torch.float64)
    o_ref, _ = oracle.attn_fwd(qh, kh, v, True, sm)
    want, spreads = oracle.attn_bwd(qh, kh, v, do, True, sm, o=o.detach().cpu(), spread=True)
    assert_close("O", o.detach().cpu(), o_ref)
    _check_grads("", (qg.grad.cpu(), kg.grad.cpu(), vg.grad.cpu()), want, spreads)


@pytest.mark.parametrize("B,H,Nq,Nk,D,causal", [(2, 2, 256, 256, 128, True), (1, 3, 100, 333, 64, False),
                                                (1, 2, 128, 320, 256, True)])
def test_quantized_kv_entry_point(qfa, B, H, Nq, Nk, D, causal):
    """K and V as two INT8 tensors (codes, fp16 scale, zero point, as asymmetric_quant_per_token returns them):
    O and the gradients against the oracle on the dequantized operands, the gradients of K and V landing in the
    16-bit placeholder leaves as in the reference's contract (quant_flash_attn.py:232-237)."""
    N = max(Nq, Nk)
    q, k, v, do = make_inputs("offset", B, H, N, D, seed=77 + D, dtype=torch.float16)
    q, do = q[:, :, :Nq].contiguous(), do[:, :, :Nq].contiguous()
    k, v = k[:, :, :Nk].contiguous(), v[:, :, :Nk].contiguous()
    sm = 1.0 / math.sqrt(D)
    qg, kg, vg = (t.to(DEV).requires_grad_(True) for t in (q, k, v))
    k_quant = qfa.asymmetric_quant_per_token(kg.detach())
    v_quant = qfa.asymmetric_quant_per_token(vg.detach())
    o = qfa.quant_flash_attn_quantized_kv(qg, kg, vg, k_quant, v_quant, causal, sm)
    o.backward(do.to(DEV))
    qc, _, zq, sq, _ = oracle.quantize_per_token(q)
    qh = oracle.dequantize_per_token(qc, sq, zq, torch.float64)
    kh = oracle.dequantize_per_token(*(t.cpu() for t in k_quant), torch.float64)       # fp16 scale, as stored
    vh = oracle.dequantize_per_token(*(t.cpu() for t in v_quant)).to(torch.float16)    # what the P.V product streams
    o_ref, _ = oracle.attn_fwd(qh, kh, vh, causal, sm)
    want, spreads = oracle.attn_bwd(qh, kh, vh, do, causal, sm, o=o.detach().cpu(), spread=True)
    assert_close("O", o.detach().cpu(), o_ref)
    _check_grads("", (qg.grad.cpu(), kg.grad.cpu(), vg.grad.cpu()), want, spreads)


@pytest.mark.parametrize("Z,H,Nq,Nkv,D", [(2, 4, 18, 512, 64), (2, 8, 32, 1024, 128), (4, 16, 16, 2048, 64), (1, 2, 17, 1023, 128),
                                          (3, 5, 97, 689, 128),      # the reference's shapes (test_accuracy.py:35-45, small batch)
                                          (1, 2, 600, 700, 128),     # query block past the shared-KV kernels: INT8-score path
                                          (2, 2, 97, 689, 256),      # compute_flops.py:94 sweeps head_dim 256
                                          (1, 2, 1100, 1200, 256)])  # past the shared-KV kernels at head_dim 256
def test_reference_entry_point_shared_kv(qfa, Z, H, Nq, Nkv, D):
    """The reference's own test (test_accuracy.py:47-133): fp16 q, kv ~ N(0,1), seed 20, quantize kv
    externally, forward + backward, against un-quantized fp16-input attention at its tolerances
    (O atol 1e-1; dQ atol 1e-2 rtol 1e-2; dKV atol 1e-2 rtol 2e-2) and against the shared-KV oracle."""
    torch.manual_seed(20)
    q = torch.randn(Z, H, Nq, D).to(torch.float16)
    kv = torch.randn(Z, H, Nkv, D).to(torch.float16)
    do = torch.randn(Z, H, Nq, D).to(torch.float16)
    sm = 1.0 / math.sqrt(D)
    qg = q.to(DEV).requires_grad_(True)
    kvg = kv.to(DEV).requires_grad_(True)
    kv_quant = qfa.asymmetric_quant_per_token(kvg.detach())
    out = qfa.quant_flash_attn(qg, kvg, kv_quant, sm)
    out.backward(do.to(DEV))
    # un-quantized attention in fp64 (what fp16 SDPA approximates)
    qr, kvr = q.double().requires_grad_(True), kv.double().requires_grad_(True)
    ref = torch.nn.functional.scaled_dot_product_attention(qr, kvr, kvr, is_causal=False, scale=sm)
    ref.backward(do.double())
    assert torch.allclose(out.detach().cpu().double(), ref.detach(), atol=1e-1, rtol=0)
    assert torch.allclose(qg.grad.cpu().double(), qr.grad, atol=1e-2, rtol=1e-2)
    assert torch.allclose(kvg.grad.cpu().double(), kvr.grad, atol=1e-2, rtol=2e-2)
    # shared-KV oracle on the same codes: Q as it is for the shared-KV kernels (the reference's
    # computation), quantized per token where the INT8-score kernels take over
    from quant_flash_attn_amd.quant_flash_attn import shared_kv_max_q
    codes, scale, zp = (t.cpu() for t in kv_quant)
    qh = q
    if Nq > shared_kv_max_q(D):
        qc, _, zq, sq, _ = oracle.quantize_per_token(q)
        qh = oracle.dequantize_per_token(qc, sq, zq, torch.float64)
    o_ref, _ = oracle.legacy_fwd(qh, codes, scale, zp, sm)
    (dq_ref, dkv_ref), (nq, nkv) = oracle.legacy_bwd(qh, codes, scale, zp, do, sm, o=out.detach().cpu(), spread=True)
    assert_close("O", out.detach().cpu(), o_ref, scaled=True)
    assert_close("dQ", qg.grad.cpu(), dq_ref, scaled=True, spread=nq)
    assert_close("dKV", kvg.grad.cpu(), dkv_ref, scaled=True, spread=nkv)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("n", [16, 64 * 1024 - 8, 3 * 1024 * 1024 + 40])
def test_sum_grads_is_the_fp32_sum_rounded_once(qfa, dtype, n):
    """dkv = dK + dV of the reference's entry point (quant_flash_attn.py:161) through the C-ABI: both addends
    widened to fp32, added, rounded once to the 16-bit format -- bit for bit, also in place (out = a), with values
    that cancel, overflow the format and non-finite ones."""
    from quant_flash_attn_amd import _lib
    g = torch.Generator().manual_seed(n)
    a = (torch.randn(n, generator=g) * 8).to(dtype)
    b = (torch.randn(n, generator=g) * 8).to(dtype)
    b[::7] = -a[::7]
    big = torch.finfo(dtype).max
    special = torch.tensor([big, big, -big, float("inf"), float("nan"), 0.0, -0.0, 2.0 ** -20], dtype=dtype)
    a[:8], b[:8] = special, special.flip(0)
    a[8:16], b[8:16] = special, special
    a, b = a.to(DEV), b.to(DEV)
    want = (a.float() + b.float()).to(dtype)
    out = torch.empty_like(a)
    code = _lib.DTYPE_CODE[dtype]
    _lib.check(_lib.lib().qfa_sum_grads(a.data_ptr(), b.data_ptr(), out.data_ptr(), code, n, _lib.stream_of(a)), "sum")
    _lib.check(_lib.lib().qfa_sum_grads(a.data_ptr(), b.data_ptr(), a.data_ptr(), code, n, _lib.stream_of(a)), "sum")
    torch.cuda.synchronize()
    for got in (out, a):
        assert torch.equal(got.view(torch.int16)[~want.isnan()], want.view(torch.int16)[~want.isnan()])
        assert torch.equal(got.isnan(), want.isnan())
    assert _lib.lib().qfa_sum_grads(a.data_ptr(), b.data_ptr(), out.data_ptr(), code, 12, _lib.stream_of(a)) != 0


def test_graph_capture_and_replay(qfa):
    """The whole step (both quantizers, forward, backward) captured into a HIP graph: every entry point
    only enqueues kernels on the caller's stream (no allocation, no memset, no synchronisation inside
    the library), so a replay with new contents in the static input buffers must reproduce the eager
    result bit for bit.  Replayed several times with eager work and synchronisations in between."""
    B, H, N, D = 2, 3, 320, 128
    sm = 1.0 / math.sqrt(D)
    static = [torch.zeros(B, H, N, D, dtype=torch.bfloat16, device=DEV) for _ in range(4)]

    def step(q, k, v, do):
        qq = qfa.quantize_for_attention(q)
        kq = qfa.quantize_for_attention(k)
        o, lse = qfa.attn_fwd_quantized(qq, kq, v, True, sm)
        dq, dk, dv = qfa.attn_bwd_quantized(qq, kq, v, o, do, lse, True, sm)
        return o, lse, dq, dk, dv

    inputs = [tuple(t.to(DEV) for t in make_inputs(cfg, B, H, N, D, seed=40 + i))
              for i, cfg in enumerate(("normal", "offset", "outlier"))]
    for s, t in zip(static, inputs[0]):
        s.copy_(t)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):      # warm-up on the capture stream, as torch asks
        step(*static)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(*static)
    for rep in range(2):
        for inp in inputs:
            eager = step(*inp)
            torch.cuda.synchronize()
            for s, t in zip(static, inp):
                s.copy_(t)
            graph.replay()
            torch.cuda.synchronize()
            for name, a_, b_ in zip(("O", "LSE", "dQ", "dK", "dV"), outs, eager):
                assert torch.equal(a_, b_), f"graph replay differs from eager: {name} (round {rep})"


@pytest.mark.parametrize("B,H,Nq,Nk,D,causal,seed", [(1, 2, 128, 128, 64, True, 3101385), (3, 3, 384, 64, 64, False, 3101466)])
def test_nearly_one_hot_rows_meet_the_rounded_output_floor(qfa, B, H, Nq, Nk, D, causal, seed):
    """A key far above the rest makes the softmax rows nearly one-hot: dS = P o (dP - delta) then cancels to
    the rounding of delta = rowsum(O o dO), and O reaches every backward rounded to 16 bits (the reference
    sums it in fp16 as well, quant_flash_attn.py:97-99).  dK of the dominant key collects that error over all
    queries and leaves the 2e-2 bar (0.10 here).  The kernels must stay within the bar of the SAME exact
    formulas evaluated with delta from the rounded O, i.e. add nothing of their own."""
    dt = torch.bfloat16
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Nq, D, generator=g) * 0.3 + 2.0
    k = torch.randn(B, H, Nk, D, generator=g) * 0.3
    v = torch.randn(B, H, Nk, D, generator=g).to(dt)
    do = torch.randn(B, H, Nq, D, generator=g).to(dt)
    k[:, :, torch.randint(0, Nk, (max(1, Nk // 50),), generator=g)] += 5.0
    q, k = q.to(dt), k.to(dt)
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse, dq, dk, dv = _fwd_bwd(qfa, q, k, v, do, causal, sm)
    qh = oracle.dequantize_per_token(qq.codes.cpu(), qq.scale.cpu(), qq.zero_point.cpu(), torch.float64)
    kh = oracle.dequantize_per_token(kq.codes.cpu(), kq.scale.cpu(), kq.zero_point.cpu(), torch.float64)
    o_ref, lse_ref = oracle.attn_fwd(qh, kh, v, causal, sm)
    dq_floor, dk_floor = rounded_output_floor(qh, kh, v, do, o_ref, lse_ref, dt, causal, sm)
    want, spreads = oracle.attn_bwd(qh, kh, v, do, causal, sm, o=o.cpu(), spread=True)
    _check_grads("", (dq.cpu(), dk.cpu(), dv.cpu()), want, spreads)
    rq, rk, rv = oracle.attn_bwd(qh, kh, v, do, causal, sm)
    # and against the exact gradients they are no further off than that floor is (10 % slack)
    assert max_abs(dk.cpu(), rk) <= 1.1 * max_abs(dk_floor, rk) + 2e-2
    assert max_abs(dq.cpu(), rq) <= 1.1 * max_abs(dq_floor, rq) + 2e-2


def test_rounded_dequantized_operands_cost_no_accuracy(qfa):
    """The dK and dQ products take the dequantized Q^, K^ rounded to the 16-bit type as one operand and dS rounded to
    it as the other.  The alternative keeps the integers (code - zero point) exact in the 16-bit operand and folds the
    scale into dS in fp32 before rounding.  Keys with a large common part make K^ rounding as visible as it gets
    (dQ is a sum of terms that cancel down to the keys' differences).  Both schemes are evaluated in fp64 with
    exactly those roundings: they differ by a percent in RMS error, and the kernel sits on the first one."""
    dt = torch.bfloat16
    B, H, N, D = 1, 2, 256, 128
    g = torch.Generator().manual_seed(7)
    q = torch.randn(B, H, N, D, generator=g).to(dt)
    k = (torch.randn(B, H, N, D, generator=g) * 0.5 + 4.0).to(dt)
    v = torch.randn(B, H, N, D, generator=g).to(dt)
    do = torch.randn(B, H, N, D, generator=g).to(dt)
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse, dq, dk, dv = _fwd_bwd(qfa, q, k, v, do, False, sm)
    qh = oracle.dequantize_per_token(qq.codes.cpu(), qq.scale.cpu(), qq.zero_point.cpu(), torch.float64)
    kh = oracle.dequantize_per_token(kq.codes.cpu(), kq.scale.cpu(), kq.zero_point.cpu(), torch.float64)
    (rq, _, _), _ = oracle.attn_bwd(qh, kh, v, do, False, sm, o=o.cpu(), spread=True)
    r = lambda t: t.to(dt).double()
    s = (qh @ kh.transpose(-1, -2)) * sm
    p = torch.exp(s - torch.logsumexp(s, -1)[..., None])
    ds = p * (do.double() @ v.double().transpose(-1, -2) - (o.cpu().double() * do.double()).sum(-1, keepdim=True))
    k_int = kq.codes.cpu().double() - kq.zero_point.cpu().double().reshape(B, H, N, 1)
    k_scale = kq.scale.cpu().double().reshape(B, H, 1, N)
    dq_rounded_khat = r((r(ds) @ r(kh)) * sm)               # what the kernels do
    dq_exact_integers = r((r(ds * k_scale) @ k_int) * sm)   # the alternative
    rms = lambda t: float(t.pow(2).mean().sqrt())
    e_kernel, e_a, e_b = rms(dq.cpu().double() - rq), rms(dq_rounded_khat - rq), rms(dq_exact_integers - rq)
    assert e_a <= 1.05 * e_b, (e_a, e_b)            # rounding K^ costs at most a few percent of the error dS carries anyway
    assert e_kernel <= 1.15 * e_a, (e_kernel, e_a)  # and the kernel adds nothing of its own

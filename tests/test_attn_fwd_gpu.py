"""GPU parity of the HIP forward kernel against the CPU oracle: fp64 attention on the dequantized
Q^, K^ (quant_flash_attn.py:50-83 restated), tolerance max-abs <= 2e-2 and cosine >= 0.999 on O
(bf16/fp16 outputs), LSE to 1e-3.  Full benchmark sizes are covered by sampled heads and by
size-independent properties."""
import math

import pytest
import torch

from helpers import assert_close, max_abs
from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
LSE_TOL = 2.0 ** -8   # row sums are taken over the 16-bit-rounded probabilities (2^-9 relative each)


def _run(qfa, q, k, v, causal, sm):
    qq = qfa.quantize_for_attention(q.to(DEV))
    kq = qfa.quantize_for_attention(k.to(DEV))
    o, lse = qfa.attn_fwd_quantized(qq, kq, v.to(DEV), causal, sm)
    torch.cuda.synchronize()
    return qq, kq, o, lse


def _oracle_fwd(qq, kq, v, causal, sm, heads=None):
    sel = (lambda t: t.cpu()) if heads is None else (lambda t: t.cpu()[heads[0]:heads[0] + 1, heads[1]:heads[1] + 1])
    qh = oracle.dequantize_per_token(sel(qq.codes), sel(qq.scale), sel(qq.zero_point), torch.float64)
    kh = oracle.dequantize_per_token(sel(kq.codes), sel(kq.scale), sel(kq.zero_point), torch.float64)
    return oracle.attn_fwd(qh, kh, sel(v), causal, sm)


CASES = [
    # B, H, Nq, Nk, D, causal, config, dtype
    (1, 2, 128, 128, 128, False, "normal", torch.bfloat16),
    (1, 2, 128, 128, 128, True, "offset", torch.bfloat16),
    (2, 3, 384, 384, 128, True, "offset", torch.bfloat16),
    (1, 4, 256, 256, 64, False, "normal", torch.bfloat16),      # shape of the plumbing configuration
    (2, 2, 512, 512, 64, True, "uniform", torch.bfloat16),
    (1, 2, 1024, 1024, 128, False, "outlier", torch.bfloat16),
    (1, 2, 200, 200, 128, False, "offset", torch.bfloat16),     # ragged
    (1, 3, 333, 333, 64, True, "uniform", torch.bfloat16),      # ragged, causal
    (2, 2, 97, 689, 128, False, "normal", torch.bfloat16),      # short Q, long ragged KV (reference test shape)
    (1, 2, 17, 1023, 128, False, "normal", torch.float16),
    (1, 2, 640, 640, 128, True, "offset", torch.float16),
    # causal with many heads: query blocks of a group of heads are dispatched together; 12 and 19 heads leave
    # a partial group at the end
    (3, 4, 320, 320, 64, True, "normal", torch.bfloat16),
    (1, 19, 300, 300, 128, True, "offset", torch.bfloat16),
    # head_dim 256 (compute_flops.py:94): one workgroup per CU, three-term zero-point correction
    (1, 2, 256, 256, 256, False, "normal", torch.bfloat16),
    (2, 3, 384, 384, 256, True, "offset", torch.bfloat16),
    (1, 2, 1024, 1024, 256, True, "outlier", torch.float16),
    (1, 2, 333, 333, 256, True, "uniform", torch.bfloat16),     # ragged, causal
    (2, 2, 97, 689, 256, False, "offset", torch.float16),       # short Q, long ragged KV
    (1, 3, 700, 700, 256, False, "uniform", torch.bfloat16),
    # causal with fewer queries than keys: the mask is aligned to the last key
    (2, 2, 128, 384, 128, True, "normal", torch.bfloat16),
    (1, 3, 97, 689, 128, True, "offset", torch.float16),        # ragged both ways, offset 592
    (1, 2, 200, 333, 64, True, "uniform", torch.bfloat16),
    (1, 2, 1, 300, 128, True, "normal", torch.bfloat16),        # one query: sees every key
    (2, 2, 160, 200, 256, True, "offset", torch.bfloat16),
]


@pytest.mark.parametrize("B,H,Nq,Nk,D,causal,config,dtype", CASES)
def test_forward_vs_oracle(qfa, B, H, Nq, Nk, D, causal, config, dtype):
    N = max(Nq, Nk)
    q, k, v, _ = make_inputs(config, B, H, N, D, seed=Nq + D, dtype=dtype)
    q, k, v = q[:, :, :Nq].contiguous(), k[:, :, :Nk].contiguous(), v[:, :, :Nk].contiguous()
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse = _run(qfa, q, k, v, causal, sm)
    o_ref, lse_ref = _oracle_fwd(qq, kq, v, causal, sm)
    assert o.dtype == dtype and o.shape == (B, H, Nq, D) and lse.shape == (B, H, Nq)
    assert_close("O", o.cpu(), o_ref)
    assert max_abs(lse.cpu(), lse_ref) < LSE_TOL
    # the quantized inputs the kernel consumed are the oracle's
    assert torch.equal(qq.codes.cpu(), oracle.quantize_per_token_c(q)[0])


@pytest.mark.parametrize("D,dtype", [(128, torch.bfloat16), (64, torch.float16), (256, torch.bfloat16)])
@pytest.mark.parametrize("jump", [64, 80, 104, 352])
@pytest.mark.parametrize("causal", [False, True])
def test_scores_jump_far_above_the_running_reference(qfa, D, dtype, jump, causal):
    """Keys from index `jump` on score hundreds of nats above the earlier ones.  The pipelined loop keeps no
    running maximum; it must notice (from the sum of 16 probabilities, before they are multiplied with V) that
    its reference is stale and move it -- in the first or the second half of a 32-key block, depending on
    where the jump sits -- and the earlier keys' contribution must vanish cleanly instead of turning into
    inf/NaN."""
    B, H, N = 1, 2, 512
    g = torch.Generator().manual_seed(jump + D)
    q = (3.0 + 0.3 * torch.randn((B, H, N, D), generator=g)).to(dtype)
    k = 0.1 * torch.randn((B, H, N, D), generator=g)
    k[:, :, jump:] += 3.0
    k[:, 1, jump + 200:] += 2.0          # a second jump in one head
    k = k.to(dtype)
    v = torch.randn((B, H, N, D), generator=g).to(dtype)
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse = _run(qfa, q, k, v, causal, sm)
    o_ref, lse_ref = _oracle_fwd(qq, kq, v, causal, sm)
    sc = sm * (q[0, 0].double() @ k[0, 0].double().T)
    assert float(sc[:, jump:].min() - sc[:, :jump].max()) > 60.0 * math.log(2.0)   # more than 2^60 apart
    assert_close("O", o.cpu(), o_ref)
    assert max_abs(lse.cpu(), lse_ref) < LSE_TOL * max(1.0, float(lse_ref.abs().max()) / 64)


@pytest.mark.parametrize("D", [64, 128, 256])
@pytest.mark.parametrize("causal", [False, True])
def test_constant_rows_at_the_clamps_give_exact_integer_scores(qfa, D, causal):
    """Constant rows of +-300 quantize to scale 1, codes +127 / -128 and zero points -128 / +127: the largest integer
    score, code row sums and zero-point terms the kernels can meet (+-255 * 255 * D), all of one sign at once.  With
    sm_scale = 4 every query of such a row gives equal weight to the keys of its own sign and none to the others,
    and an integer score off by one would give one key e^4 times the weight of its peers: O must be the mean of V
    over those keys.  Checks the exactness of the INT8 product plus the zero-point correction at the end of its
    range, in the pipelined loop (first tile) and in the masked one (ragged second tile)."""
    B, H, Nq, Nk = 1, 2, 96, 96
    g = torch.Generator().manual_seed(3 * D + causal)
    def rows(n):
        x = torch.randn((B, H, n, D), generator=g)
        x[:, :, 0::3] = 300.0
        x[:, :, 1::3] = -300.0
        return x.to(torch.bfloat16)
    q, k = rows(Nq), rows(Nk)
    v = torch.randn((B, H, Nk, D), generator=g).to(torch.bfloat16)
    sm = 4.0
    qq, kq, o, lse = _run(qfa, q, k, v, causal, sm)
    assert qq.codes[0, 0, 0].eq(127).all() and qq.zero_point[0, 0, 0].item() == -128 and qq.scale[0, 0, 0].item() == 1.0
    assert kq.codes[0, 0, 1].eq(-128).all() and kq.zero_point[0, 0, 1].item() == 127
    o_ref, lse_ref = _oracle_fwd(qq, kq, v, causal, sm)
    rows_pm = [i for i in range(Nq) if i % 3 != 2 and not (causal and i < 3)]
    assert_close("O of the constant rows", o.cpu()[:, :, rows_pm], o_ref[:, :, rows_pm])
    # and directly: the mean of V over the visible keys of the query's sign
    vd = v.double()
    for i in rows_pm[:8] + rows_pm[-8:]:
        keys = [j for j in range(Nk) if j % 3 == i % 3 and (not causal or j <= i)]
        assert max_abs(o.cpu()[:, :, i], vd[:, :, keys].mean(2)) < 2e-2, (i, len(keys))
    rel = ((lse.cpu().double() - lse_ref).abs() / lse_ref.abs().clamp_min(1.0))[:, :, rows_pm]
    assert float(rel.max()) < 1e-6


def _may_use_biased_accumulators(qq, D):
    """The kernel's per-query test (head_dim <= 128), restated: every term of the zero-point correction and the
    integer score itself must stay below 2^22 against the worst key."""
    codes = qq.codes.cpu().long()
    zq = qq.zero_point.cpu().long().reshape(codes.shape[:-1])
    c = qq.rowsum.cpu().long().reshape(zq.shape) - D * zq
    mq = (codes - zq[..., None]).abs().sum(-1)
    tq = zq.abs() * (128 * D + 127) + 128 * (c.abs() + 2 * 128)
    return (255 * mq < 2 ** 22) & (tq < 2 ** 22)


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("mixed", [False, True])
def test_rows_that_may_not_use_biased_accumulators(qfa, D, causal, mixed):
    """Query rows that sit at one end of their range (all elements in [0.5, 1]: zero point -128, every code +127)
    fail the bound under which the pipelined loop may accumulate the INT8 product onto a biased fp32 bit pattern:
    their waves run the instance of the loop that converts explicitly.  Long enough for the unrolled steady loop;
    `mixed` puts rows of either kind into one workgroup (the choice is per wave of 32 queries)."""
    B, H, N = 1, 2, 704
    g = torch.Generator().manual_seed(11 * D + 2 * causal + mixed)
    q = torch.randn((B, H, N, D), generator=g)
    k = torch.randn((B, H, N, D), generator=g)
    v = torch.randn((B, H, N, D), generator=g).to(torch.bfloat16)
    pinned = 0.5 + 0.5 * torch.rand((B, H, N, D), generator=g)
    if mixed:
        q[:, :, 32:64] = pinned[:, :, 32:64]
        q[:, :, 300:420] = -pinned[:, :, 300:420]
    else:
        q = pinned
    q, k = q.to(torch.bfloat16), k.to(torch.bfloat16)
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse = _run(qfa, q, k, v, causal, sm)
    ok = _may_use_biased_accumulators(qq, D)
    if D == 64:   # no row can leave the window at this width: the kernel does not even look
        assert ok.all()
    else:
        assert not ok[:, :, 32:64].any() and (mixed == bool(ok[:, :, 64:96].all()))
    o_ref, lse_ref = _oracle_fwd(qq, kq, v, causal, sm)
    assert_close("O", o.cpu(), o_ref)
    assert max_abs(lse.cpu(), lse_ref) < 2.0 ** -8


def test_fp32_plumbing_configuration(qfa):
    """B1 H4 N256 D64 fp32 q,k,v, seed 0, non-causal, through the autograd entry point."""
    torch.manual_seed(0)
    q, k, v = torch.randn(1, 4, 256, 64), torch.randn(1, 4, 256, 64), torch.randn(1, 4, 256, 64)
    sm = 1.0 / 8.0
    o = qfa.quant_flash_attn_qkv(q.to(DEV), k.to(DEV), v.to(DEV), False, sm)
    assert o.dtype == torch.float32
    qc, _, zq, sq, _ = oracle.quantize_per_token(q)
    kc, _, zk, sk, _ = oracle.quantize_per_token(k)
    ref, _ = oracle.attn_fwd(oracle.dequantize_per_token(qc, sq, zq), oracle.dequantize_per_token(kc, sk, zk),
                             v.to(torch.bfloat16), False, sm)
    assert_close("O", o.cpu(), ref)


@pytest.mark.parametrize("config,B,H,N,D,causal", [("offset", 4, 32, 4096, 128, True),
                                                   ("outlier", 1, 16, 16384, 128, False),
                                                   ("uniform", 16, 16, 2048, 64, True)])
def test_full_size_sampled_heads_and_properties(qfa, config, B, H, N, D, causal):
    q, k, v, _ = make_inputs(config, B, H, N, D, seed=0)
    sm = 1.0 / math.sqrt(D)
    qq, kq, o, lse = _run(qfa, q, k, v, causal, sm)
    assert torch.isfinite(o.float()).all() and torch.isfinite(lse).all()
    n_check = min(N, 4096)   # oracle rows per sampled head (dense fp64 scores)
    for (b, h) in [(0, 0), (B - 1, H - 1)]:
        sel = lambda t: t.cpu()[b:b + 1, h:h + 1]
        qh = oracle.dequantize_per_token(sel(qq.codes), sel(qq.scale), sel(qq.zero_point), torch.float64)
        kh = oracle.dequantize_per_token(sel(kq.codes), sel(kq.scale), sel(kq.zero_point), torch.float64)
        rows = slice(N - n_check, N)
        s = (qh[..., rows, :] @ kh.transpose(-1, -2)) * sm
        if causal:
            i = torch.arange(N - n_check, N)[:, None]
            s = s.masked_fill(torch.arange(N)[None, :] > i, float("-inf"))
        o_ref = torch.softmax(s, -1) @ sel(v).double()
        assert_close(f"O[{b},{h}]", o.cpu()[b:b + 1, h:h + 1, rows], o_ref)
        assert max_abs(lse.cpu()[b:b + 1, h:h + 1, rows], torch.logsumexp(s, -1)) < LSE_TOL
    if causal:   # row 0 only sees key 0
        assert torch.equal(o[:, :, 0], v.to(DEV)[:, :, 0])
    # rows of P sum to one: with V = 1 the output is 1 (up to the 16-bit rounding of P)
    ones = torch.ones_like(v, device=DEV)
    o1, lse1 = qfa.attn_fwd_quantized(qq, kq, ones, causal, sm)
    assert (o1.float() - 1.0).abs().max() < 1e-2
    assert torch.equal(lse1, lse)
    # linear in V: O(2V) == 2 O(V) exactly (power-of-two scaling commutes with every rounding)
    o2, _ = qfa.attn_fwd_quantized(qq, kq, (v.to(DEV) * 2), causal, sm)
    assert torch.equal(o2, o * 2)


def test_key_permutation_invariance(qfa):
    """Non-causal attention does not depend on the order of the keys."""
    q, k, v, _ = make_inputs("offset", 1, 2, 512, 128, seed=3)
    sm = 1.0 / math.sqrt(128)
    _, _, o, lse = _run(qfa, q, k, v, False, sm)
    perm = torch.randperm(512, generator=torch.Generator().manual_seed(1))
    _, _, o_p, lse_p = _run(qfa, q, k[:, :, perm], v[:, :, perm], False, sm)
    assert max_abs(o, o_p) <= 2e-2 and max_abs(lse, lse_p) < 2 * LSE_TOL   # O within two bf16 ulps of |O| <= 4


@pytest.mark.parametrize("D", [64, 128, 256])
def test_output_fully_written_and_deterministic(qfa, D):
    q, k, v, _ = make_inputs("normal", 2, 2, 300, D, seed=8)
    sm = 0.1
    qq = qfa.quantize_for_attention(q.to(DEV))
    kq = qfa.quantize_for_attention(k.to(DEV))
    o1, l1 = qfa.attn_fwd_quantized(qq, kq, v.to(DEV), True, sm)
    o2, l2 = qfa.attn_fwd_quantized(qq, kq, v.to(DEV), True, sm)
    assert torch.equal(o1, o2) and torch.equal(l1, l2)
    assert not torch.isnan(o1.float()).any()


@pytest.mark.parametrize("D", [64, 256])
def test_strided_qkv_layout(qfa, D):
    """q, k, v stored [B,N,H,D] and passed as permuted views; forward and backward equal the contiguous run."""
    B, H, N = 2, 3, 256
    q, k, v, _ = make_inputs("offset", B, H, N, D, seed=12)
    mk = lambda t: t.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)
    o = qfa.quant_flash_attn_qkv(mk(q), mk(k), mk(v), True, 0.125)
    o_c = qfa.quant_flash_attn_qkv(q.to(DEV), k.to(DEV), v.to(DEV), True, 0.125)
    assert torch.equal(o, o_c)
    ins = [mk(t).requires_grad_(True) for t in (q, k, v)]
    ins_c = [t.to(DEV).requires_grad_(True) for t in (q, k, v)]
    g = torch.randn(B, H, N, D, generator=torch.Generator().manual_seed(5)).to(torch.bfloat16).to(DEV)
    qfa.quant_flash_attn_qkv(*ins, True, 0.125).backward(g)
    qfa.quant_flash_attn_qkv(*ins_c, True, 0.125).backward(g)
    for a, b in zip(ins, ins_c):
        assert torch.equal(a.grad, b.grad)

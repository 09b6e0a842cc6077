"""INT8 per-token quantized flash attention -- drop-in for the reference's quant_flash_attn.py.

Two autograd entry points, both backed by the HIP kernels behind qfa_attn_fwd / qfa_attn_bwd:

  QuantFlashAttnQKV.apply(q, k, v, causal, sm_scale)            (alias quant_flash_attn_qkv)
      Signature of the repository's fused-attention Function (flash_attn_triton.py:441).  Q and K
      are quantized per token inside (asymmetric_quant.py math), QK^T runs on INT8 MFMA, V stays
      in 16-bit.  Gradients flow straight through the quantizer to q and k.

  QuantFlashAttention.apply(q, kv_fp16, kv_quant, sm_scale)     (alias quant_flash_attn)
      The reference's own entry point (quant_flash_attn.py:173-240): one quantized tensor serves as
      K and V, `kv_fp16` only receives the gradient, backward returns (dq, dkv, None, None) with
      dkv = dK + dV (:161).  Query blocks of up to SHARED_KV_MAX_Q (512; 1024 at head_dim 256) tokens run the reference's
      computation itself in the forward (Q in 16-bit, qfa_attn_fwd_shared_kv) and in the backward
      (qfa_attn_bwd_shared_kv, binary16 arithmetic; bf16 tensors are converted around it).  Longer
      query blocks go through the INT8-score kernels, where Q is quantized per token too (stated
      difference from the reference, which keeps Q in fp16).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from .asymmetric_quant import (QuantizedTokens, code_rowsum, dequantize_per_token, quantize_for_attention,
                               quantize_pair_for_attention)

_IO_DTYPES = (torch.bfloat16, torch.float16)


def _flat(t: torch.Tensor, dtype: torch.dtype, n: int, name: str) -> torch.Tensor:
    t = t.reshape(-1)
    if t.dtype != dtype or t.numel() != n:
        raise ValueError(f"{name}: expected {n} values of {dtype}, got {t.numel()} of {t.dtype}")
    return t.contiguous()


def _rows16(t: torch.Tensor) -> torch.Tensor:
    """[B,H,N,D] tensor whose rows are contiguous and whose strides / base are 16-byte multiples."""
    es = t.element_size()
    ok = (t.stride(3) == 1 and t.stride(2) >= t.shape[3] and t.data_ptr() % 16 == 0
          and all(t.stride(i) > 0 and (t.stride(i) * es) % 16 == 0 for i in range(3)))
    return t if ok else t.contiguous()


def _unpack(qt: QuantizedTokens, name: str):
    codes, scale, zp, rowsum = qt
    if codes.dim() != 4 or codes.dtype != torch.int8:
        raise ValueError(f"{name}.codes must be a 4-D int8 tensor")
    n = codes.shape[0] * codes.shape[1] * codes.shape[2]
    return (_rows16(codes), _flat(scale, torch.float32, n, f"{name}.scale"),
            _flat(zp, torch.int8, n, f"{name}.zero_point"), _flat(rowsum, torch.int32, n, f"{name}.rowsum"))


def attn_fwd_quantized(qq: QuantizedTokens, kq: QuantizedTokens, v: torch.Tensor, causal: bool,
                       sm_scale: float, _entry: str = "qfa_attn_fwd") -> Tuple[torch.Tensor, torch.Tensor]:
    """O, LSE = attention(dequant(qq), dequant(kq), v).  v and O are bf16 or fp16 [B,H,N,D];
    LSE is fp32 [B,H,Nq] (natural log, as quant_flash_attn.py:79)."""
    if v.dtype not in _IO_DTYPES:
        raise TypeError(f"v must be bfloat16 or float16, got {v.dtype}")
    qc, sq, zq, rq = _unpack(qq, "q")
    kc, sk, zk, rk = _unpack(kq, "k")
    _lib.require_gpu(qc, sq, zq, rq, kc, sk, zk, rk, v)
    B, H, Nq, D = qc.shape
    Nk = kc.shape[2]
    if kc.shape != (B, H, Nk, D) or v.shape != (B, H, Nk, D):
        raise ValueError(f"shape mismatch: q {tuple(qc.shape)}, k {tuple(kc.shape)}, v {tuple(v.shape)}")
    v = _rows16(v)
    o = torch.empty((B, H, Nq, D), dtype=v.dtype, device=v.device)
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device=v.device)
    with torch.cuda.device(v.device):
        code = getattr(_lib.lib(), _entry)(     # "qfa_bench_qk_stage" is the QK^T-only timing variant
            qc.data_ptr(), sq.data_ptr(), zq.data_ptr(), rq.data_ptr(),
            kc.data_ptr(), sk.data_ptr(), zk.data_ptr(), rk.data_ptr(),
            v.data_ptr(), o.data_ptr(), lse.data_ptr(), _lib.DTYPE_CODE[v.dtype],
            B, H, Nq, Nk, D,
            qc.stride(0), qc.stride(1), qc.stride(2), kc.stride(0), kc.stride(1), kc.stride(2),
            v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1), o.stride(2),
            float(sm_scale), int(bool(causal)), _lib.stream_of(v))
    _lib.check(code, _entry)
    return o, lse


def attn_bwd_quantized(qq: QuantizedTokens, kq: QuantizedTokens, v: torch.Tensor, o: torch.Tensor,
                       do: torch.Tensor, lse: torch.Tensor, causal: bool, sm_scale: float
                       ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """dQ, dK, dV (w.r.t. the dequantized q^, k^ and v) in v's dtype."""
    if v.dtype not in _IO_DTYPES:
        raise TypeError(f"v must be bfloat16 or float16, got {v.dtype}")
    qc, sq, zq, rq = _unpack(qq, "q")
    kc, sk, zk, rk = _unpack(kq, "k")
    B, H, Nq, D = qc.shape
    Nk = kc.shape[2]
    if o.shape != (B, H, Nq, D) or do.shape != (B, H, Nq, D) or v.shape != (B, H, Nk, D):
        raise ValueError("shape mismatch between o / do / v and the quantized tensors")
    if o.dtype != v.dtype:
        raise TypeError("o and v must have the same dtype")
    if do.dtype != v.dtype:
        do = do.to(v.dtype)
    _lib.require_gpu(qc, kc, v, o, do, lse)
    v, o, do = _rows16(v), _rows16(o), _rows16(do)
    lse = _flat(lse, torch.float32, B * H * Nq, "lse")
    ws_bytes = _lib.lib().qfa_attn_bwd_workspace_bytes(B, H, Nq, Nk, D)
    if ws_bytes <= 0:
        raise ValueError(f"unsupported backward shape B={B} H={H} Nq={Nq} Nk={Nk} D={D}")
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=v.device)
    dq = torch.empty((B, H, Nq, D), dtype=v.dtype, device=v.device)
    dk = torch.empty((B, H, Nk, D), dtype=v.dtype, device=v.device)
    dv = torch.empty((B, H, Nk, D), dtype=v.dtype, device=v.device)
    s = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    with torch.cuda.device(v.device):
        code = _lib.lib().qfa_attn_bwd(
            qc.data_ptr(), sq.data_ptr(), zq.data_ptr(), rq.data_ptr(),
            kc.data_ptr(), sk.data_ptr(), zk.data_ptr(), rk.data_ptr(),
            v.data_ptr(), o.data_ptr(), do.data_ptr(), lse.data_ptr(), workspace.data_ptr(), ws_bytes,
            dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), _lib.DTYPE_CODE[v.dtype],
            B, H, Nq, Nk, D, *s(qc), *s(kc), *s(v), *s(o), *s(do), *s(dq), *s(dk), *s(dv),
            float(sm_scale), int(bool(causal)), _lib.stream_of(v))
    _lib.check(code, "qfa_attn_bwd")
    return dq, dk, dv


# Longest query block the shared-KV kernels are used for.  They stream the codes once per 16 queries
# (from L2 after the first block), which wins while Nq is small against Nk -- the reference's test and
# benchmark shapes; measured crossover with the INT8-score kernels at Nk=4096, D=128: between 512 and
# 1024 queries (fwd 1.16 vs 1.51 ms at 512, 1.14 vs 1.01 ms at 1024).
SHARED_KV_MAX_Q = 512
# head_dim 256 (compute_flops.py:94): the INT8-score kernels run one wave per SIMD there and the crossover moves up
# (Nk=4096: fwd+bwd 5.9 vs 4.5 ms at 512 queries, 9.0 vs 8.9 at 1024; Nq=Nk=2048: 3.9 vs 4.9 ms, INT8-score first).
SHARED_KV_MAX_Q_BY_HEAD_DIM = {256: 1024}   # head_dim -> limit, where it differs from SHARED_KV_MAX_Q


def shared_kv_max_q(head_dim: int) -> int:
    """Longest query block that `quant_flash_attn` gives to the shared-KV kernels at this head_dim."""
    return SHARED_KV_MAX_Q_BY_HEAD_DIM.get(head_dim, SHARED_KV_MAX_Q)


def attn_fwd_shared_kv(q: torch.Tensor, codes: torch.Tensor, scale: torch.Tensor, zero_point: torch.Tensor,
                       sm_scale: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """O, LSE = attention(q, kv, kv) with kv = (codes - zero_point) * scale, q in fp16 / bf16 and NOT
    quantized -- the computation of _attn_fwd_kernel_quantized (quant_flash_attn.py:22-83).
    O has q's dtype; LSE is fp32 [B,H,Nq] (natural log, :79)."""
    if q.dtype not in _IO_DTYPES:
        raise TypeError(f"q must be bfloat16 or float16, got {q.dtype}")
    if codes.dim() != 4 or codes.dtype != torch.int8:
        raise ValueError("codes must be a 4-D int8 tensor")
    _lib.require_gpu(q, codes, scale, zero_point)
    B, H, Nq, D = q.shape
    Nk = codes.shape[2]
    if codes.shape != (B, H, Nk, D):
        raise ValueError(f"shape mismatch: q {tuple(q.shape)}, codes {tuple(codes.shape)}")
    n = B * H * Nk
    if scale.dtype != torch.float32 and scale.dtype != q.dtype:
        scale = scale.to(torch.float32)
    scale = _flat(scale, scale.dtype, n, "scale")
    zero_point = _flat(zero_point, torch.int8, n, "zero_point")
    q, codes = _rows16(q), _rows16(codes)
    o = torch.empty((B, H, Nq, D), dtype=q.dtype, device=q.device)
    lse = torch.empty((B, H, Nq), dtype=torch.float32, device=q.device)
    # scratch for the split over keys the library uses when B*H alone cannot fill the GPU (0: no split)
    ws_bytes = _lib.lib().qfa_attn_fwd_shared_kv_workspace_bytes(B, H, Nq, Nk, D)
    workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=q.device) if ws_bytes > 0 else None
    with torch.cuda.device(q.device):
        code = _lib.lib().qfa_attn_fwd_shared_kv(
            q.data_ptr(), codes.data_ptr(), scale.data_ptr(), _lib.DTYPE_CODE[scale.dtype], zero_point.data_ptr(),
            o.data_ptr(), lse.data_ptr(), _lib.DTYPE_CODE[q.dtype], B, H, Nq, Nk, D,
            q.stride(0), q.stride(1), q.stride(2), codes.stride(0), codes.stride(1), codes.stride(2),
            o.stride(0), o.stride(1), o.stride(2), float(sm_scale),
            workspace.data_ptr() if workspace is not None else None, ws_bytes, _lib.stream_of(q))
    _lib.check(code, "qfa_attn_fwd_shared_kv")
    return o, lse


def attn_bwd_shared_kv(q: torch.Tensor, codes: torch.Tensor, scale: torch.Tensor, zero_point: torch.Tensor,
                       o: torch.Tensor, do: torch.Tensor, lse: torch.Tensor, sm_scale: float,
                       grad_dtype: Optional[torch.dtype] = None, grad_scale: Optional[torch.Tensor] = None
                       ) -> Tuple[torch.Tensor, torch.Tensor]:
    """dQ, dKV of attn_fwd_shared_kv: the computation of _attn_bwd_kernel_quantized
    (quant_flash_attn.py:104-166) with dKV = dV + dK as stored there (:161).  q, o, do fp16
    [B,H,Nq,D] (the kernels compute in binary16); lse as returned by the forward.  dQ and dKV come back
    in `grad_dtype` (fp16 by default, or bf16), multiplied by the one-element device tensor `grad_scale`
    if given.  Up to 32 queries (16 at head_dim 256) run in one fused pass over the codes, longer blocks
    in a dQ kernel plus a dKV kernel."""
    if q.dtype != torch.float16 or o.dtype != torch.float16:
        raise TypeError("the shared-KV backward kernel computes in float16: q and o must be float16")
    grad_dtype = grad_dtype or torch.float16
    if grad_dtype not in _IO_DTYPES:
        raise TypeError(f"grad_dtype must be float16 or bfloat16, got {grad_dtype}")
    if codes.dim() != 4 or codes.dtype != torch.int8:
        raise ValueError("codes must be a 4-D int8 tensor")
    B, H, Nq, D = q.shape
    Nk = codes.shape[2]
    if codes.shape != (B, H, Nk, D) or o.shape != q.shape or do.shape != q.shape:
        raise ValueError("shape mismatch between q / o / do and the codes")
    do = do.to(torch.float16)
    _lib.require_gpu(q, codes, scale, zero_point, o, do, lse)
    if grad_scale is not None:
        _lib.require_gpu(q, grad_scale)
        grad_scale = _flat(grad_scale, torch.float32, 1, "grad_scale")
    n = B * H * Nk
    if scale.dtype not in (torch.float32, torch.float16):
        scale = scale.to(torch.float32)
    scale = _flat(scale, scale.dtype, n, "scale")
    zero_point = _flat(zero_point, torch.int8, n, "zero_point")
    lse = _flat(lse, torch.float32, B * H * Nq, "lse")
    q, codes, o, do = _rows16(q), _rows16(codes), _rows16(o), _rows16(do)
    dq = torch.empty((B, H, Nq, D), dtype=grad_dtype, device=q.device)
    dkv = torch.empty((B, H, Nk, D), dtype=grad_dtype, device=q.device)
    s = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    with torch.cuda.device(q.device):
        code = _lib.lib().qfa_attn_bwd_shared_kv(
            q.data_ptr(), codes.data_ptr(), scale.data_ptr(), _lib.DTYPE_CODE[scale.dtype], zero_point.data_ptr(),
            o.data_ptr(), do.data_ptr(), lse.data_ptr(), dq.data_ptr(), dkv.data_ptr(), _lib.QFA_F16,
            _lib.DTYPE_CODE[grad_dtype], grad_scale.data_ptr() if grad_scale is not None else None,
            B, H, Nq, Nk, D, *s(q), *s(codes), *s(o), *s(do), *s(dq), *s(dkv), float(sm_scale), _lib.stream_of(q))
    _lib.check(code, "qfa_attn_bwd_shared_kv")
    return dq, dkv


def _io_dtype(t: torch.Tensor) -> torch.dtype:
    return t.dtype if t.dtype in _IO_DTYPES else torch.bfloat16


class QuantFlashAttnQKV(torch.autograd.Function):
    """forward(ctx, q, k, v, causal, sm_scale) -> o   (argument order of flash_attn_triton.py:441).

    q, k, v: [B,H,N,D] bf16 / fp16 (fp32 is accepted: V and O then pass through bf16).
    causal keeps key j for query i when j <= i (flash_attn_triton.py:50); with fewer queries than keys the mask is
    aligned to the last key (j <= i + Nk - Nq)."""

    @staticmethod
    def forward(ctx, q, k, v, causal, sm_scale):
        _lib.require_gpu(q, k, v)
        if q.dim() != 4 or k.dim() != 4 or v.dim() != 4:
            raise ValueError("q, k, v must be 4-D (Batch, Heads, Seq, Head_Dim)")
        if q.shape[-1] != k.shape[-1] or k.shape != v.shape or q.shape[:2] != k.shape[:2]:
            raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k {tuple(k.shape)}, v {tuple(v.shape)}")
        qq, kq = quantize_pair_for_attention(q, k)   # one launch for both
        v16 = v.to(_io_dtype(v))
        o, lse = attn_fwd_quantized(qq, kq, v16, causal, sm_scale)
        ctx.save_for_backward(*qq, *kq, v16, o, lse)
        ctx.causal, ctx.sm_scale = bool(causal), float(sm_scale)
        ctx.in_dtypes = (q.dtype, k.dtype, v.dtype)
        return o.to(q.dtype)

    @staticmethod
    def backward(ctx, do):
        t = ctx.saved_tensors
        qq, kq = QuantizedTokens(*t[0:4]), QuantizedTokens(*t[4:8])
        v16, o, lse = t[8], t[9], t[10]
        dq, dk, dv = attn_bwd_quantized(qq, kq, v16, o, do.to(v16.dtype), lse, ctx.causal, ctx.sm_scale)
        dq_t, dk_t, dv_t = ctx.in_dtypes
        return dq.to(dq_t), dk.to(dk_t), dv.to(dv_t), None, None


quant_flash_attn_qkv = QuantFlashAttnQKV.apply


class QuantFlashAttnQuantizedKV(torch.autograd.Function):
    """forward(ctx, q, k_fp16, v_fp16, k_quant, v_quant, causal, sm_scale) -> o; backward -> (dq, dk, dv, None...).

    The reference's contract (quant_flash_attn.py:178-237: the keys and values arrive as INT8 codes with per-token
    scale and zero point, a 16-bit placeholder leaf receives the gradient) with K and V as two separately quantized
    tensors instead of one shared tensor, and a causal flag.  k_quant and v_quant are (codes, scale, zero_point)
    tuples as asymmetric_quant_per_token returns them; k_fp16 and v_fp16 are only placeholders.
    The K codes are used as they are (INT8 scores); V is dequantized once per call by the HIP dequantizer into a
    16-bit tensor that the P.V product streams: converting int8 V inside the attention kernel would add about 110
    vector instructions per 32x32 block to a loop that is bound by its vector instructions, the separate pass adds
    a read of the codes and one 16-bit write and read (8 % of the forward at B4 H32 N4096 D128)."""

    @staticmethod
    def forward(ctx, q, k_fp16, v_fp16, k_quant, v_quant, causal, sm_scale):
        kc, ks, kz = k_quant
        vc, vs, vz = v_quant
        _lib.require_gpu(q, kc, ks, kz, vc, vs, vz)
        if q.dim() != 4 or kc.dim() != 4 or kc.shape != vc.shape or q.shape[-1] != kc.shape[-1] or q.shape[:2] != kc.shape[:2]:
            raise ValueError(f"shape mismatch: q {tuple(q.shape)}, k codes {tuple(kc.shape)}, v codes {tuple(vc.shape)}")
        io = _io_dtype(q)
        qq = quantize_for_attention(q)
        kq = QuantizedTokens(kc, ks.to(torch.float32), kz, code_rowsum(kc))
        v16 = dequantize_per_token(vc, vs, vz, io)
        o, lse = attn_fwd_quantized(qq, kq, v16, causal, sm_scale)
        ctx.save_for_backward(*qq, *kq, v16, o, lse)
        ctx.causal, ctx.sm_scale = bool(causal), float(sm_scale)
        ctx.in_dtypes = (q.dtype, k_fp16.dtype, v_fp16.dtype)
        return o.to(q.dtype)

    @staticmethod
    def backward(ctx, do):
        t = ctx.saved_tensors
        qq, kq = QuantizedTokens(*t[0:4]), QuantizedTokens(*t[4:8])
        v16, o, lse = t[8], t[9], t[10]
        dq, dk, dv = attn_bwd_quantized(qq, kq, v16, o, do.to(v16.dtype), lse, ctx.causal, ctx.sm_scale)
        dq_t, dk_t, dv_t = ctx.in_dtypes
        return dq.to(dq_t), dk.to(dk_t), dv.to(dv_t), None, None, None, None


quant_flash_attn_quantized_kv = QuantFlashAttnQuantizedKV.apply


class QuantFlashAttention(torch.autograd.Function):
    """forward(ctx, q, kv_fp16, kv_quant, sm_scale) -> o; backward -> (dq, dkv, None, None).

    Positional contract of the reference (quant_flash_attn.py:178-237): kv_quant is the
    (codes, scale, zero_point) tuple returned by asymmetric_quant_per_token, kv_fp16 is only a
    placeholder leaf that receives dkv, attention is non-causal, K == V == dequant(kv_quant)."""

    @staticmethod
    def forward(ctx, q, kv_fp16, kv_quant, sm_scale):
        codes, scale, zp = kv_quant
        _lib.require_gpu(q, codes, scale, zp)
        if q.dim() != 4 or codes.shape != kv_fp16.shape or q.shape[-1] != codes.shape[-1]:
            raise ValueError(f"shape mismatch: q {tuple(q.shape)}, kv {tuple(kv_fp16.shape)}, codes {tuple(codes.shape)}")
        ctx.sm_scale = float(sm_scale)
        ctx.q_dtype, ctx.kv_dtype = q.dtype, kv_fp16.dtype
        ctx.shared_kv = q.shape[2] <= shared_kv_max_q(q.shape[3]) and q.dtype in _IO_DTYPES
        if ctx.shared_kv:
            # the reference's computation itself: Q unquantized, the codes streamed once (:50-69)
            o, lse = attn_fwd_shared_kv(q, codes, scale, zp, sm_scale)
            ctx.save_for_backward(q, codes, scale, zp, o, lse)
            return o
        io = _io_dtype(q)
        qq, kq, v16 = _legacy_operands(q, codes, scale, zp, io)
        o, lse = attn_fwd_quantized(qq, kq, v16, False, sm_scale)
        ctx.save_for_backward(*qq, *kq, v16, o, lse)
        return o.to(q.dtype)

    @staticmethod
    def backward(ctx, grad_output):
        t = ctx.saved_tensors
        if ctx.shared_kv:
            q, codes, scale, zp, o, lse = t
            # The backward kernels compute in binary16, and what they feed the matrix pipe is not dO but
            # sm_scale * p * (dP - delta) and that times the key's scale: with dO as it comes, ordinary small
            # gradients land in binary16's subnormals (or flush to zero) there.  dQ and dKV are linear in dO,
            # so dO is handed over scaled by a power of two chosen on the device (no synchronisation) from
            # its largest magnitude and from the largest key scale, and the kernels scale dQ and dKV back
            # while they round them.  q and o convert exactly from bf16 (more mantissa, values of order one).
            do16, back = _normalised_dout(grad_output, scale)
            dq, dkv = attn_bwd_shared_kv(q.to(torch.float16), codes, scale, zp, o.to(torch.float16), do16, lse,
                                         ctx.sm_scale, grad_dtype=q.dtype, grad_scale=back)
            return dq.to(ctx.q_dtype), dkv.to(ctx.kv_dtype), None, None
        else:
            qq, kq = QuantizedTokens(*t[0:4]), QuantizedTokens(*t[4:8])
            v16, o, lse = t[8], t[9], t[10]
        dq, dk, dv = attn_bwd_quantized(qq, kq, v16, o, grad_output.to(v16.dtype), lse, False, ctx.sm_scale)
        # :161 (dk already carries sm_scale): one pass, added in fp32 and rounded once
        dk, dv = dk.contiguous(), dv.contiguous()
        with torch.cuda.device(dk.device):
            _lib.check(_lib.lib().qfa_sum_grads(dk.data_ptr(), dv.data_ptr(), dk.data_ptr(), _lib.DTYPE_CODE[dk.dtype],
                                                dk.numel(), _lib.stream_of(dk)), "qfa_sum_grads")
        dkv = dk.to(ctx.kv_dtype)
        return dq.to(ctx.q_dtype), dkv, None, None


def _normalised_dout(grad_output: torch.Tensor, kv_scale: torch.Tensor):
    """(dO * 2^k as float16, 2^-k as a one-element float32 tensor) for the binary16 backward kernels
    (qfa_dout_normalise: two launches, nothing synchronises).

    k puts the largest |dO| * 2^k * (largest key scale) into (4, 8]: 2^8 for |dO| when the key scales are of the usual
    size (2^-5 for values of order one), higher when they are smaller and lower when they are larger, since the operands
    the kernels form carry the key scale as a factor (ds * scale_j must neither sink into binary16's subnormals nor
    leave its range); dO * 2^k itself stays at or below 2^14."""
    _lib.require_gpu(grad_output, kv_scale)
    if grad_output.dtype not in _IO_DTYPES:   # not what autograd hands over for a 16-bit output; bf16 keeps the range
        grad_output = grad_output.to(torch.bfloat16)
    grad_output = grad_output.contiguous()
    if kv_scale.dtype not in (torch.float32, torch.float16):
        kv_scale = kv_scale.to(torch.float32)
    kv_scale = kv_scale.contiguous()
    if kv_scale.data_ptr() % 16:   # a view that starts inside an allocation
        kv_scale = kv_scale.clone()
    dev = grad_output.device
    do16 = torch.empty(grad_output.shape, dtype=torch.float16, device=dev)
    back = torch.empty(1, dtype=torch.float32, device=dev)
    workspace = torch.empty(_lib.lib().qfa_dout_normalise_workspace_bytes(), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().qfa_dout_normalise(
            grad_output.data_ptr(), _lib.DTYPE_CODE[grad_output.dtype], grad_output.numel(), kv_scale.data_ptr(),
            _lib.DTYPE_CODE[kv_scale.dtype], kv_scale.numel(), workspace.data_ptr(), do16.data_ptr(), back.data_ptr(),
            _lib.stream_of(grad_output)), "qfa_dout_normalise")
    return do16, back


def _legacy_operands(q, codes, scale, zp, io):
    """Operands of the INT8-score kernels for the reference's entry point: Q quantized per token,
    K = the caller's codes with the scale exactly as stored, V = dequant(kv) (quant_flash_attn.py:65)."""
    qq = quantize_for_attention(q)
    kq = QuantizedTokens(codes, scale.to(torch.float32), zp, code_rowsum(codes))
    return qq, kq, dequantize_per_token(codes, scale, zp, io)


quant_flash_attn = QuantFlashAttention.apply

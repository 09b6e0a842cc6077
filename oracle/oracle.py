"""TEST INFRASTRUCTURE ONLY -- CPU oracle for the quantized flash-attention path.

Only tests, the smoke check and the CPU-baseline leg of the benchmark may import
this module.  The shipped package never does: it calls the HIP kernels or raises.

Every function restates, on the CPU, one piece of the reference's algorithm and
cites the lines it follows (paths relative to /root/reference):

  quantize_per_token      asymmetric_quant.py:66-106  (kernel body, order of ops)
  dequantize_per_token    asymmetric_quant.py:158-160
  int_scores              algebraic identity used by the INT8 kernels; checked
                          against dequantize-then-dot (quant_flash_attn.py:65-68)
  attn_fwd                quant_flash_attn.py:50-83 (scale, softmax, LSE = m + ln l),
                          causal rule flash_attn_triton.py:50 (row >= col kept)
  bwd_delta               quant_flash_attn.py:97-99
  attn_bwd                quant_flash_attn.py:153-164 generalised to separate K and V
  legacy_fwd / legacy_bwd quant_flash_attn.py:22-166 literally: K == V == dequant(kv),
                          Q not quantized, dkv = dv + sm_scale * dk (:161)
  reference_cpu_path      test_accuracy.py:76-81,88-103 (eager quantize + dequantized
                          SDPA + backward): the CPU baseline that gets timed

Parity pins (tests/test_oracle_*.py): exact rational brute force on small rows,
hand-computed known answers, constructed rounding ties, agreement of the two
independent quantizer restatements (this numpy one and oracle/quant_oracle.c),
torch.autograd / gradcheck for the backward formulas, torch.softmax / logsumexp /
scaled_dot_product_attention for the forward.  The reference ships no golden
vectors or fixtures for this path, so those are the whole pin.
"""
from __future__ import annotations

import ctypes
import math
import os
from typing import Optional, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_CLIB = None

Q_MIN = np.float32(-128.0)
Q_MAX = np.float32(127.0)


# --------------------------------------------------------------------------- quantizer
def roundf_half_away(y: np.ndarray) -> np.ndarray:
    """C roundf on float32 arrays: nearest, ties away from zero.

    libdevice.round (asymmetric_quant.py:90,103) is roundf.  numpy's round is
    half-to-even, and floor(|y|+0.5) mis-rounds 0.49999997, hence trunc+compare:
    y - trunc(y) is exact in binary32, so the comparison with 0.5 is exact.
    """
    y = np.asarray(y, dtype=np.float32)
    with np.errstate(invalid="ignore"):
        t = np.trunc(y)
        frac = np.abs(y - t)                     # exact, in [0, 1); nan for +-inf
        step = np.where(frac >= np.float32(0.5), np.copysign(np.float32(1.0), y), np.float32(0.0))
    return (t + step.astype(np.float32)).astype(np.float32)


def _to_f32_numpy(x) -> np.ndarray:
    if isinstance(x, torch.Tensor):
        return x.detach().to(torch.float32).cpu().numpy()     # fp16/bf16 -> fp32 is exact
    return np.asarray(x, dtype=np.float32)


def quantize_per_token(x, scale_dtype: torch.dtype = torch.float16):
    """Per-token asymmetric INT8 quantization over the last axis.

    Returns (codes int8 [..., D], scale [..., 1] in scale_dtype, zp int8 [..., 1],
             scale32 float32 [..., 1], rowsum int32 [..., 1]).
    The first three are what asymmetric_quant_per_token returns
    (asymmetric_quant.py:127-129,149); scale32 is the unrounded scale the codes
    were computed with (:86,103); rowsum = sum of the codes of the token.
    """
    xf = _to_f32_numpy(x)
    with np.errstate(over="ignore", invalid="ignore", divide="ignore"):
        mn = xf.min(axis=-1, keepdims=True).astype(np.float32)           # :80
        mx = xf.max(axis=-1, keepdims=True).astype(np.float32)           # :81
        scale = ((mx - mn).astype(np.float32) / np.float32(255.0)).astype(np.float32)   # :84-86
        scale = np.where(scale == 0, np.float32(1.0), scale).astype(np.float32)          # :87
        zpf = (Q_MIN - (mn / scale).astype(np.float32)).astype(np.float32)               # :89
        zp = np.maximum(Q_MIN, np.minimum(Q_MAX, roundf_half_away(zpf)))                 # :90-91
        y = ((xf / scale).astype(np.float32) + zp).astype(np.float32)                    # :103
        codes = np.maximum(Q_MIN, np.minimum(Q_MAX, roundf_half_away(y)))                # :103-104
    codes_i8 = codes.astype(np.int8)
    rowsum = codes_i8.astype(np.int32).sum(axis=-1, keepdims=True, dtype=np.int32)
    scale32 = torch.from_numpy(scale.copy())
    return (torch.from_numpy(codes_i8), scale32.to(scale_dtype),                       # :93 (RNE cast)
            torch.from_numpy(zp.astype(np.int8)), scale32, torch.from_numpy(rowsum))


def _clib():
    global _CLIB
    if _CLIB is None:
        path = os.path.join(_HERE, "libqfa_oracle.so")
        if not os.path.exists(path):
            raise FileNotFoundError(f"{path} not built: run `make -C oracle`")
        lib = ctypes.CDLL(path)
        lib.qfa_oracle_quant_rows_f32.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64,
                                                  ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                  ctypes.c_void_p]
        lib.qfa_oracle_quant_rows_f32.restype = None
        lib.qfa_oracle_dequant_rows_f32.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
                                                    ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p]
        lib.qfa_oracle_dequant_rows_f32.restype = None
        _CLIB = lib
    return _CLIB


def quantize_per_token_c(x):
    """Same contract as quantize_per_token, computed by oracle/quant_oracle.c.

    Returns (codes, scale32, zp, rowsum) with the per-token outputs shaped [..., 1].
    """
    xf = np.ascontiguousarray(_to_f32_numpy(x))
    D = xf.shape[-1]
    rows = xf.size // D
    codes = np.empty(xf.shape, dtype=np.int8)
    scale = np.empty(xf.shape[:-1] + (1,), dtype=np.float32)
    zp = np.empty(xf.shape[:-1] + (1,), dtype=np.int8)
    rowsum = np.empty(xf.shape[:-1] + (1,), dtype=np.int32)
    _clib().qfa_oracle_quant_rows_f32(xf.ctypes.data, rows, D, codes.ctypes.data, scale.ctypes.data,
                                      zp.ctypes.data, rowsum.ctypes.data)
    return (torch.from_numpy(codes), torch.from_numpy(scale), torch.from_numpy(zp),
            torch.from_numpy(rowsum))


def dequantize_per_token(codes: torch.Tensor, scale: torch.Tensor, zp: torch.Tensor,
                         dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """asymmetric_quant.py:160 -- (codes - zp) * scale, in fp32 (or fp64 if asked)."""
    return (codes.to(dtype) - zp.to(dtype)) * scale.to(dtype)


# --------------------------------------------------------------------------- integer scores
def int_scores(qc: torch.Tensor, zq: torch.Tensor, kc: torch.Tensor, zk: torch.Tensor) -> torch.Tensor:
    """sum_d (qc[i,d]-zq[i]) (kc[j,d]-zk[j]) via the expansion the INT8 kernels use:

        A[i,j] - zk[j]*rq[i] - zq[i]*rk[j] + D*zq[i]*zk[j],   A = qc @ kc^T (int), r* = row sums.

    All in int64, so exact.  qc [..., Nq, D], kc [..., Nk, D], zq [..., Nq, 1], zk [..., Nk, 1].
    """
    q = qc.to(torch.int64)
    k = kc.to(torch.int64)
    D = q.shape[-1]
    # integer matmul is not implemented for all torch CPU builds: go through float64 (exact, < 2^53)
    A = (q.to(torch.float64) @ k.to(torch.float64).transpose(-1, -2)).to(torch.int64)
    rq = q.sum(-1, keepdim=True)
    rk = k.sum(-1, keepdim=True)
    zq64 = zq.to(torch.int64)
    zk64 = zk.to(torch.int64)
    return A - rq * zk64.transpose(-1, -2) - zq64 * rk.transpose(-1, -2) + D * zq64 * zk64.transpose(-1, -2)


# --------------------------------------------------------------------------- attention
def _causal_mask(nq: int, nk: int, device=None) -> torch.Tensor:
    """True where the score is kept: row >= col (flash_attn_triton.py:50).  The reference only has nq == nk; for
    nq < nk the mask is aligned to the last key (row + nk - nq >= col), so that the rows are the last nq rows of the
    square case -- what a chunk of queries at the end of a longer key sequence needs."""
    i = torch.arange(nq, device=device)[:, None]
    j = torch.arange(nk, device=device)[None, :]
    return i + (nk - nq) >= j


def attn_fwd(qh: torch.Tensor, kh: torch.Tensor, v: torch.Tensor, causal: bool, sm_scale: float,
             dtype: torch.dtype = torch.float64) -> Tuple[torch.Tensor, torch.Tensor]:
    """O = softmax(sm_scale * qh kh^T [+ causal mask]) v ;  LSE = logsumexp (natural log).

    quant_flash_attn.py:68-79 with separate K and V.  qh, kh are the DEQUANTIZED
    tensors.  Computed densely in `dtype`; returns (O, LSE) in that dtype.
    """
    q, k, vv = qh.to(dtype), kh.to(dtype), v.to(dtype)
    s = (q @ k.transpose(-1, -2)) * sm_scale
    if causal:
        s = s.masked_fill(~_causal_mask(q.shape[-2], k.shape[-2], s.device), float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    p = torch.exp(s - lse[..., None])
    return p @ vv, lse


def bwd_delta(o: torch.Tensor, do: torch.Tensor, dtype: torch.dtype = torch.float64) -> torch.Tensor:
    """delta = rowsum(O * dO)  (quant_flash_attn.py:97-99; accumulated in `dtype`, not fp16)."""
    return (o.to(dtype) * do.to(dtype)).sum(-1)


def attn_bwd(qh, kh, v, do, causal: bool, sm_scale: float, dtype: torch.dtype = torch.float64,
             o: Optional[torch.Tensor] = None, spread: bool = False):
    """Closed-form backward of attn_fwd (quant_flash_attn.py:153-164, K and V separate).

        P = exp(S - LSE);  dV = P^T dO;  dP = dO V^T;  dS = P o (dP - delta)
        dQ = sm_scale dS K^;  dK = sm_scale dS^T Q^
    Gradients are with respect to the dequantized q^, k^ (straight-through to q, k).

    `o`: the output tensor the forward SAVED, as the reference's backward receives it (quant_flash_attn.py:207-223:
    delta = rowsum(o * do) is taken from the saved 16-bit o, :97-99).  None: the exact O of these inputs, which makes
    the result the exact gradient of attn_fwd (what autograd gives).
    `spread`: also return, per gradient element, the 2-norm of the terms of the sum that forms it
    (sqrt(sum_j (a_ij b_jd)^2)): the scale of the rounding error any evaluation with 16-bit operands carries.
    """
    q, k, vv, g = qh.to(dtype), kh.to(dtype), v.to(dtype), do.to(dtype)
    o_exact, lse = attn_fwd(q, k, vv, causal, sm_scale, dtype)
    s = (q @ k.transpose(-1, -2)) * sm_scale
    if causal:
        s = s.masked_fill(~_causal_mask(q.shape[-2], k.shape[-2], s.device), float("-inf"))
    p = torch.exp(s - lse[..., None])
    dv = p.transpose(-1, -2) @ g
    dp = g @ vv.transpose(-1, -2)
    delta = bwd_delta(o_exact if o is None else o, g, dtype)
    ds = p * (dp - delta[..., None])
    dq = (ds @ k) * sm_scale
    dk = (ds.transpose(-1, -2) @ q) * sm_scale
    if not spread:
        return dq, dk, dv
    ds2, p2 = ds * ds, p * p
    nq = torch.sqrt(ds2 @ (k * k)) * sm_scale
    nk = torch.sqrt(ds2.transpose(-1, -2) @ (q * q)) * sm_scale
    nv = torch.sqrt(p2.transpose(-1, -2) @ (g * g))
    return (dq, dk, dv), (nq, nk, nv)


def attn_bwd_autograd(qh, kh, v, do, causal: bool, sm_scale: float, dtype: torch.dtype = torch.float64):
    """The same gradients from torch.autograd (a library routine) -- used to pin attn_bwd."""
    q = qh.detach().to(dtype).requires_grad_(True)
    k = kh.detach().to(dtype).requires_grad_(True)
    vv = v.detach().to(dtype).requires_grad_(True)
    o, _ = attn_fwd(q, k, vv, causal, sm_scale, dtype)
    o.backward(do.to(dtype))
    return q.grad, k.grad, vv.grad


# --------------------------------------------------------------------------- legacy (shared K == V)
def legacy_fwd(q, kv_codes, kv_scale, kv_zp, sm_scale: float, dtype: torch.dtype = torch.float64):
    """quant_flash_attn.py:22-83: K == V == dequant(kv) (scale as stored), Q unquantized, no mask."""
    kvh = dequantize_per_token(kv_codes, kv_scale, kv_zp, dtype)
    return attn_fwd(q.to(dtype), kvh, kvh, False, sm_scale, dtype)


def legacy_bwd(q, kv_codes, kv_scale, kv_zp, do, sm_scale: float, dtype: torch.dtype = torch.float64,
               o: Optional[torch.Tensor] = None, spread: bool = False):
    """quant_flash_attn.py:104-166: returns (dq, dkv) with dkv = dv + sm_scale*dk (:161); `o` and `spread` as in
    attn_bwd (the spread of dkv is that of the two sums together)."""
    kvh = dequantize_per_token(kv_codes, kv_scale, kv_zp, dtype)
    if not spread:
        dq, dk, dv = attn_bwd(q.to(dtype), kvh, kvh, do, False, sm_scale, dtype, o=o)
        return dq, dk + dv
    (dq, dk, dv), (nq, nk, nv) = attn_bwd(q.to(dtype), kvh, kvh, do, False, sm_scale, dtype, o=o, spread=True)
    return (dq, dk + dv), (nq, torch.sqrt(nk * nk + nv * nv))


# --------------------------------------------------------------------------- CPU baseline path
def _quantize_torch_eager(x: torch.Tensor):
    """Torch-eager restatement of asymmetric_quant.py:66-106 (used only for timing the CPU path;
    its results are checked against quantize_per_token in the tests)."""
    xf = x.to(torch.float32)
    mn = xf.amin(-1, keepdim=True)
    mx = xf.amax(-1, keepdim=True)
    scale = (mx - mn) / 255.0
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    zpf = -128.0 - mn / scale

    def roundf(y):
        t = torch.trunc(y)
        return t + torch.where((y - t).abs() >= 0.5, torch.sign(y), torch.zeros_like(y))

    zp = roundf(zpf).clamp_(-128.0, 127.0)
    codes = roundf(xf / scale + zp).clamp_(-128.0, 127.0)
    return codes.to(torch.int8), scale, zp.to(torch.int8)


def reference_cpu_path(q, k, v, causal: bool, sm_scale: float, do: Optional[torch.Tensor] = None):
    """The reference's CPU-runnable path: eager per-token quantize of q and k, dequantize
    (asymmetric_quant.py:160), then F.scaled_dot_product_attention as in test_accuracy.py:76-78,
    plus .backward(dO) (test_accuracy.py:79) when dO is given.  fp32 throughout."""
    qc, sq, zq = _quantize_torch_eager(q)
    kc, sk, zk = _quantize_torch_eager(k)
    qh = dequantize_per_token(qc, sq, zq).requires_grad_(do is not None)
    kh = dequantize_per_token(kc, sk, zk).requires_grad_(do is not None)
    vf = v.to(torch.float32).requires_grad_(do is not None)
    o = torch.nn.functional.scaled_dot_product_attention(qh, kh, vf, is_causal=causal, scale=sm_scale)
    if do is None:
        return o
    o.backward(do.to(torch.float32))
    return o, qh.grad, kh.grad, vf.grad

"""Per-token asymmetric INT8 quantization -- drop-in for the reference's asymmetric_quant.py.

`asymmetric_quant_per_token(x)` keeps the reference's name, argument and return structure
(asymmetric_quant.py:109-149): codes int8 [B,H,N,D], scale [B,H,N,1] (fp16 by default, as the
reference stores it, :128), zero point int8 [B,H,N,1].  The work is done by the HIP kernel
behind qfa_quant_per_token; `quantize_for_attention` additionally returns the fp32 scale and
the per-token code sums that the INT8 attention kernels consume.
"""
from __future__ import annotations

from typing import NamedTuple, Tuple

import torch

from . import _lib


class QuantizedTokens(NamedTuple):
    codes: torch.Tensor      # int8  [B,H,N,D]
    scale: torch.Tensor      # fp32  [B,H,N,1]  (the scale the codes were computed with)
    zero_point: torch.Tensor  # int8  [B,H,N,1]
    rowsum: torch.Tensor     # int32 [B,H,N,1]  sum of the token's codes


def _check_input(x: torch.Tensor) -> torch.Tensor:
    if x.dim() != 4:
        raise ValueError(f"expected a 4-D (Batch, Heads, Seq, Head_Dim) tensor, got shape {tuple(x.shape)}")
    if x.dtype not in _lib.DTYPE_CODE:
        raise TypeError(f"unsupported dtype {x.dtype}: expected float16, bfloat16 or float32")
    _lib.require_gpu(x)
    es = x.element_size()
    ok = (x.stride(3) == 1 and all((x.stride(i) * es) % 16 == 0 and x.stride(i) > 0 for i in range(3))
          and x.stride(2) >= x.shape[3] and x.data_ptr() % 16 == 0)
    return x if ok else x.contiguous()


def _run(x: torch.Tensor, scale_lp_dtype, want_rowsum: bool):
    x = _check_input(x)
    B, H, N, D = x.shape
    codes = torch.empty((B, H, N, D), dtype=torch.int8, device=x.device)
    scale32 = torch.empty((B, H, N, 1), dtype=torch.float32, device=x.device)
    zp = torch.empty((B, H, N, 1), dtype=torch.int8, device=x.device)
    rowsum = torch.empty((B, H, N, 1), dtype=torch.int32, device=x.device) if want_rowsum else None
    scale_lp = None
    if scale_lp_dtype is not None and scale_lp_dtype != torch.float32:
        scale_lp = torch.empty((B, H, N, 1), dtype=scale_lp_dtype, device=x.device)
    with torch.cuda.device(x.device):
        code = _lib.lib().qfa_quant_per_token(
            x.data_ptr(), _lib.DTYPE_CODE[x.dtype], codes.data_ptr(), scale32.data_ptr(),
            scale_lp.data_ptr() if scale_lp is not None else None,
            _lib.DTYPE_CODE[scale_lp_dtype] if scale_lp is not None else 0,
            zp.data_ptr(), rowsum.data_ptr() if rowsum is not None else None,
            B, H, N, D, x.stride(0), x.stride(1), x.stride(2),
            codes.stride(0), codes.stride(1), codes.stride(2), _lib.stream_of(x))
    _lib.check(code, "qfa_quant_per_token")
    return codes, scale32, scale_lp, zp, rowsum


def asymmetric_quant_per_token(input_tensor: torch.Tensor, scale_dtype: torch.dtype = torch.float16
                               ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Quantizes a (Batch, Heads, Seq, Head_Dim) tensor to INT8, one scale / zero point per token.

    Same contract as the reference's function of this name (asymmetric_quant.py:109-149).
    Returns (codes int8 [B,H,N,D], scale [B,H,N,1] of `scale_dtype`, zero_point int8 [B,H,N,1]).
    The codes are computed with the unrounded fp32 scale; the returned scale is its
    round-to-nearest cast (fp16 by default like the reference; pass torch.float32 to keep it).
    """
    if scale_dtype not in (torch.float16, torch.bfloat16, torch.float32):
        raise TypeError(f"scale_dtype must be float16, bfloat16 or float32, got {scale_dtype}")
    codes, scale32, scale_lp, zp, _ = _run(input_tensor, scale_dtype, want_rowsum=False)
    return codes, (scale32 if scale_lp is None else scale_lp), zp


def quantize_for_attention(x: torch.Tensor) -> QuantizedTokens:
    """Quantizes like asymmetric_quant_per_token and also returns what the INT8 attention kernels
    need beside the codes: the fp32 scale and the per-token sum of the codes."""
    codes, scale32, _, zp, rowsum = _run(x, None, want_rowsum=True)
    return QuantizedTokens(codes, scale32, zp, rowsum)


def quantize_pair_for_attention(x0: torch.Tensor, x1: torch.Tensor) -> Tuple[QuantizedTokens, QuantizedTokens]:
    """quantize_for_attention of two tensors (the queries and the keys of an attention call: same batch, heads,
    head dimension and element type, any two lengths) in ONE launch; bit-identical to two separate calls."""
    x0, x1 = _check_input(x0), _check_input(x1)
    if x0.shape[:2] != x1.shape[:2] or x0.shape[3] != x1.shape[3] or x0.dtype != x1.dtype or x0.device != x1.device:
        return quantize_for_attention(x0), quantize_for_attention(x1)
    B, H, _, D = x0.shape
    out = []
    for x in (x0, x1):
        N = x.shape[2]
        out.append((torch.empty((B, H, N, D), dtype=torch.int8, device=x.device),
                    torch.empty((B, H, N, 1), dtype=torch.float32, device=x.device),
                    torch.empty((B, H, N, 1), dtype=torch.int8, device=x.device),
                    torch.empty((B, H, N, 1), dtype=torch.int32, device=x.device)))
    (c0, s0, z0, r0), (c1, s1, z1, r1) = out
    with torch.cuda.device(x0.device):
        code = _lib.lib().qfa_quant_per_token_pair(
            x0.data_ptr(), x1.data_ptr(), _lib.DTYPE_CODE[x0.dtype], c0.data_ptr(), c1.data_ptr(), s0.data_ptr(),
            s1.data_ptr(), z0.data_ptr(), z1.data_ptr(), r0.data_ptr(), r1.data_ptr(), B, H, x0.shape[2], x1.shape[2], D,
            x0.stride(0), x0.stride(1), x0.stride(2), x1.stride(0), x1.stride(1), x1.stride(2),
            c0.stride(0), c0.stride(1), c0.stride(2), c1.stride(0), c1.stride(1), c1.stride(2), _lib.stream_of(x0))
    _lib.check(code, "qfa_quant_per_token_pair")
    return QuantizedTokens(c0, s0, z0, r0), QuantizedTokens(c1, s1, z1, r1)


def dequantize_per_token(codes: torch.Tensor, scale: torch.Tensor, zero_point: torch.Tensor,
                         dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """(codes - zero_point) * scale per token (the reference's dequantize_per_token_torch,
    asymmetric_quant.py:158-160), as a HIP kernel writing `dtype`."""
    _lib.require_gpu(codes, scale, zero_point)
    if codes.dim() != 4 or codes.dtype != torch.int8:
        raise ValueError("codes must be a 4-D int8 tensor")
    if dtype not in _lib.DTYPE_CODE or scale.dtype not in _lib.DTYPE_CODE:
        raise TypeError("dtype and scale.dtype must be float16, bfloat16 or float32")
    B, H, N, D = codes.shape
    if codes.stride(3) != 1 or any(codes.stride(i) % 8 for i in range(3)) or codes.data_ptr() % 8:
        codes = codes.contiguous()
    scale = scale.reshape(-1).contiguous()
    zero_point = zero_point.reshape(-1).contiguous()
    if scale.numel() != B * H * N or zero_point.numel() != B * H * N or zero_point.dtype != torch.int8:
        raise ValueError("scale / zero_point must hold one value per token (zero_point int8)")
    out = torch.empty((B, H, N, D), dtype=dtype, device=codes.device)
    with torch.cuda.device(codes.device):
        code = _lib.lib().qfa_dequant_per_token(
            codes.data_ptr(), scale.data_ptr(), _lib.DTYPE_CODE[scale.dtype], zero_point.data_ptr(),
            out.data_ptr(), _lib.DTYPE_CODE[dtype], B, H, N, D,
            codes.stride(0), codes.stride(1), codes.stride(2), out.stride(0), out.stride(1), out.stride(2),
            _lib.stream_of(codes))
    _lib.check(code, "qfa_dequant_per_token")
    return out


def code_rowsum(codes: torch.Tensor) -> torch.Tensor:
    """int32 [B,H,N,1] sum of each token's codes (what quantize_for_attention emits beside the codes), as a HIP
    kernel, for codes that arrive already quantized."""
    _lib.require_gpu(codes)
    if codes.dim() != 4 or codes.dtype != torch.int8:
        raise ValueError("codes must be a 4-D int8 tensor")
    B, H, N, D = codes.shape
    if codes.stride(3) != 1 or any(codes.stride(i) % 8 for i in range(3)) or codes.data_ptr() % 8:
        codes = codes.contiguous()
    out = torch.empty((B, H, N, 1), dtype=torch.int32, device=codes.device)
    with torch.cuda.device(codes.device):
        code = _lib.lib().qfa_code_rowsum(codes.data_ptr(), out.data_ptr(), B, H, N, D, codes.stride(0),
                                          codes.stride(1), codes.stride(2), _lib.stream_of(codes))
    _lib.check(code, "qfa_code_rowsum")
    return out

"""Writes the committed fixtures of tests/golden/ (run from the repository root: python tests/golden/make_golden.py).

The reference ships no golden vectors for this path and cannot run without a GPU, so the fixtures
are derived here, once, from sources independent of the code they check:

  quant_kat.json   known-answer rows of the per-token quantizer (asymmetric_quant.py:80-104).  Expected
                   codes / scale / zero point come from the exact-rational model in tests/exact_model.py
                   (fractions, no floating point), NOT from the oracle or the kernels.  Inputs are stored
                   as binary32 bit patterns.
  attn_small.npz   two small attention problems: inputs as bf16 bit patterns, quantized operands, and
                   O / LSE / dQ / dK / dV evaluated in fp64 by plain torch formulas written out below
                   (softmax(sm * Q^ K^^T + mask) V and torch.autograd), independent of oracle.attn_*.

  shared_kv_small.npz  two small problems of the reference's own operator (quant_flash_attn.py:22-166: one
                   quantized tensor is K and V, Q stays fp16): q / kv / dO as fp16 bit patterns, the exactly
                   quantized kv (codes, fp16 scale as stored by the reference, zero point), and O / LSE /
                   dQ / dKV from plain fp64 torch formulas + autograd on kv^ = (codes - zp) * fp16(scale).

Fixtures are data only; the tests that read them are tests/test_golden.py (CPU: oracle vs fixtures;
GPU: kernels vs fixtures)."""
import json
import math
import os
import struct
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))           # tests/
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))  # repository root (oracle/)
from exact_model import quant_row_exact  # noqa: E402


def f32_bits(v: float) -> int:
    return struct.unpack("<I", struct.pack("<f", v))[0]


def quant_rows():
    g = torch.Generator().manual_seed(1234)
    rows = []
    D = 32
    rows.append(("range 255: scale 1, zp -128", [0.0, 255.0] + [float(i) + 0.5 for i in range(30)]))
    rows.append(("constant row: scale forced to 1", [3.0] * D))
    rows.append(("constant negative row, zp clamps", [-200.0] * D))
    rows.append(("all positive: zp clamps at -128, large values saturate", [100.0 + 8.0 * i for i in range(D)]))
    rows.append(("all negative: zp clamps at 127", [-355.0 + 7.0 * i for i in range(D)]))
    rows.append(("zero-point tie -116.5 -> -117", [-11.5, 243.5] + [0.25 * i for i in range(30)]))
    rows.append(("tiny range around 1", [1.0 + i * 2.0 ** -20 for i in range(D)]))
    rows.append(("huge values", [(-1) ** i * 3.0e30 * (i + 1) / 32 for i in range(D)]))
    rows.append(("denormal scale", [i * 2.0 ** -140 for i in range(D)]))
    for name, gen in (("normal", lambda: torch.randn(D, generator=g)),
                      ("offset", lambda: torch.randn(D, generator=g) + 2.5),
                      ("uniform(-3,5)", lambda: torch.rand(D, generator=g) * 8 - 3),
                      ("outlier", lambda: torch.randn(D, generator=g) * torch.where(torch.arange(D) == 7, 20.0, 1.0))):
        for dt in (torch.float32, torch.bfloat16, torch.float16):
            for _ in range(2):
                rows.append((f"{name} rounded to {str(dt).split('.')[-1]}", gen().to(dt).to(torch.float32).tolist()))
    out = []
    for name, vals in rows:
        vals = [float(np.float32(v)) for v in vals]
        codes, scale, zp = quant_row_exact(vals)
        out.append({"name": name, "x_bits": [f32_bits(v) for v in vals], "codes": codes,
                    "scale_bits": f32_bits(float(scale)), "zp": zp, "rowsum": sum(codes)})
    return out


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)


def attn_case(seed, B, H, Nq, Nk, D, causal, quantize):
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, Nq, D, generator=g) + 0.5 * torch.randn(B, H, Nq, 1, generator=g)).to(torch.bfloat16)
    k = (torch.randn(B, H, Nk, D, generator=g) + 0.5 * torch.randn(B, H, Nk, 1, generator=g)).to(torch.bfloat16)
    v = torch.randn(B, H, Nk, D, generator=g).to(torch.bfloat16)
    do = torch.randn(B, H, Nq, D, generator=g).to(torch.bfloat16)
    sm = 1.0 / math.sqrt(D)
    qc, zq, sq = quantize(q)
    kc, zk, sk = quantize(k)
    qh = ((qc.double() - zq.double()[..., None]) * sq.double()[..., None]).requires_grad_(True)
    kh = ((kc.double() - zk.double()[..., None]) * sk.double()[..., None]).requires_grad_(True)
    vd = v.double().requires_grad_(True)
    s = sm * qh @ kh.transpose(-1, -2)
    if causal:
        s = s.masked_fill(torch.arange(Nk)[None, :] > torch.arange(Nq)[:, None], float("-inf"))
    lse = torch.logsumexp(s, dim=-1)
    o = torch.softmax(s, dim=-1) @ vd
    o.backward(do.double())
    return {"q": bf16_bits(q), "k": bf16_bits(k), "v": bf16_bits(v), "do": bf16_bits(do),
            "qc": qc.numpy(), "zq": zq.numpy(), "sq": sq.numpy(), "kc": kc.numpy(), "zk": zk.numpy(), "sk": sk.numpy(),
            "o": o.detach().float().numpy(), "lse": lse.detach().float().numpy(),
            "dq": qh.grad.float().numpy(), "dk": kh.grad.float().numpy(), "dv": vd.grad.float().numpy(),
            "causal": np.array(int(causal)), "sm_scale": np.array(sm, dtype=np.float64)}


def f16_bits(t: torch.Tensor) -> np.ndarray:
    return t.to(torch.float16).view(torch.int16).numpy().view(np.uint16)


def shared_kv_case(seed, B, H, Nq, Nk, D, quantize):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Nq, D, generator=g).to(torch.float16)
    kv = (torch.randn(B, H, Nk, D, generator=g) + 0.5 * torch.randn(B, H, Nk, 1, generator=g)).to(torch.float16)
    do = torch.randn(B, H, Nq, D, generator=g).to(torch.float16)
    sm = 1.0 / math.sqrt(D)
    codes, zp, scale32 = quantize(kv)
    scale16 = scale32.to(torch.float16)                     # what the reference stores (asymmetric_quant.py:93,128)
    kvh = ((codes.double() - zp.double()[..., None]) * scale16.double()[..., None]).requires_grad_(True)
    qd = q.double().requires_grad_(True)
    s = sm * qd @ kvh.transpose(-1, -2)
    lse = torch.logsumexp(s, dim=-1)
    o = torch.softmax(s, dim=-1) @ kvh
    o.backward(do.double())
    return {"q": f16_bits(q), "kv": f16_bits(kv), "do": f16_bits(do), "codes": codes.numpy(), "zp": zp.numpy(),
            "scale16": f16_bits(scale16), "o": o.detach().float().numpy(), "lse": lse.detach().float().numpy(),
            "dq": qd.grad.float().numpy(), "dkv": kvh.grad.float().numpy(), "sm_scale": np.array(sm, dtype=np.float64)}


def quantize_exact(x: torch.Tensor):
    """Quantize every row with the exact-rational model (slow, small inputs only)."""
    xs = x.to(torch.float32)
    B, H, N, D = xs.shape
    codes = torch.empty(B, H, N, D, dtype=torch.int8)
    zp = torch.empty(B, H, N, dtype=torch.int8)
    scale = torch.empty(B, H, N, dtype=torch.float32)
    for b in range(B):
        for h in range(H):
            for n in range(N):
                c, s, z = quant_row_exact(xs[b, h, n].tolist())
                codes[b, h, n] = torch.tensor(c, dtype=torch.int8)
                zp[b, h, n] = z
                scale[b, h, n] = float(s)
    return codes, zp, scale


if __name__ == "__main__":
    with open(os.path.join(HERE, "quant_kat.json"), "w") as f:
        json.dump({"D": 32, "rows": quant_rows()}, f, indent=0, separators=(",", ":"))
    cases = {"causal_N64_D64": attn_case(7, 1, 1, 64, 64, 64, True, quantize_exact),
             "ragged_Nq24_Nk72_D128": attn_case(8, 1, 1, 24, 72, 128, False, quantize_exact)}
    flat = {f"{name}/{key}": val for name, c in cases.items() for key, val in c.items()}
    np.savez_compressed(os.path.join(HERE, "attn_small.npz"), **flat)
    skv = {"Nq16_Nk100_D128": shared_kv_case(9, 1, 2, 16, 100, 128, quantize_exact),
           "Nq5_Nk70_D64": shared_kv_case(10, 1, 1, 5, 70, 64, quantize_exact)}
    np.savez_compressed(os.path.join(HERE, "shared_kv_small.npz"),
                        **{f"{name}/{key}": val for name, c in skv.items() for key, val in c.items()})
    print("wrote", os.listdir(HERE))

"""Throughput report in the reference's own terms.

Mirrors the two benchmark scripts of the reference on this build's entry points:
  * compute_flops.py:89-168   Z=512, H=16, N_CTX_Q=16, N_CTX_KV=3000, HEAD_DIM in {64, 128, 256}, fp16:
                              forward and (fwd+bwd - fwd) backward time, TFLOP/s from
                              4*Z*H*Nq*Nkv*D (backward 2.5x, :103-104) and GB/s from the theoretical
                              traffic of calculate_theoretical_io (:39-83, 'quantized' provider);
  * test_speed.py:37-60       Z=256, H=16, N_CTX_Q=16, HEAD_DIM=128, N_CTX_KV in {512..4096}.
The comparison line is torch's scaled_dot_product_attention on the same fp16 tensors (the reference
compares with the flash_attn package, which is not installed here).

    python -m quant_flash_attn_amd.compute_flops [--sweep] [--small]
"""
from __future__ import annotations

import argparse
import json
import sys

import torch

from . import asymmetric_quant_per_token, quant_flash_attn


def theoretical_io(Z, H, Nq, Nkv, D, provider, mode):
    """Bytes read + written, formula of compute_flops.py:39-83."""
    f16, f32, i8 = 2, 4, 1
    io_fwd = Z * H * Nq * D * f16 * 2 + Z * H * Nq * f32
    if provider == "fp16":
        io_fwd += 2 * Z * H * Nkv * D * f16
    else:
        io_fwd += Z * H * Nkv * (D * i8 + f16 + i8)
    if mode == "fwd":
        return io_fwd
    common = 3 * Z * H * Nq * D * f16 + 2 * Z * H * Nq * f32
    if provider == "fp16":
        return common + Z * H * Nq * D * f16 + 4 * Z * H * Nkv * D * f16
    return common + Z * H * Nq * D * f16 + Z * H * Nkv * (D * i8 + f16 + i8) + Z * H * Nkv * D * f16


def _time(fn, warmup, rep):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(rep):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / rep


def measure(Z, H, Nq, Nkv, D, provider, warmup=5, rep=20, dtype=torch.float16):
    dev = "cuda"
    q = torch.randn((Z, H, Nq, D), dtype=dtype, device=dev, requires_grad=True)
    kv = torch.randn((Z, H, Nkv, D), dtype=dtype, device=dev, requires_grad=True)
    sm = 1.0 / D ** 0.5
    if provider == "quantized":
        kv_quant = asymmetric_quant_per_token(kv.detach())
        fwd = lambda: quant_flash_attn(q, kv, kv_quant, sm)                                      # noqa: E731
    else:
        fwd = lambda: torch.nn.functional.scaled_dot_product_attention(q, kv, kv, scale=sm)    # noqa: E731
    flops = 4.0 * Z * H * Nq * Nkv * D
    ms_fwd = _time(lambda: fwd(), warmup, rep)
    go = torch.randn((Z, H, Nq, D), dtype=dtype, device=dev)

    def fwd_bwd():
        q.grad = None
        kv.grad = None
        fwd().backward(go)

    ms_bwd = max(_time(fwd_bwd, warmup, rep) - ms_fwd, 1e-6)
    return {"Time Fwd (ms)": ms_fwd, "TFLOP/s Fwd": flops / (ms_fwd * 1e-3) / 1e12,
            "BW Fwd (GB/s)": theoretical_io(Z, H, Nq, Nkv, D, provider, "fwd") / (ms_fwd * 1e-3) / 1e9,
            "Time Bwd (ms)": ms_bwd, "TFLOP/s Bwd": 2.5 * flops / (ms_bwd * 1e-3) / 1e12,
            "BW Bwd (GB/s)": theoretical_io(Z, H, Nq, Nkv, D, provider, "bwd") / (ms_bwd * 1e-3) / 1e9}


def _table(title, rows):
    cols = ["Time Fwd (ms)", "TFLOP/s Fwd", "BW Fwd (GB/s)", "Time Bwd (ms)", "TFLOP/s Bwd", "BW Bwd (GB/s)"]
    print("-" * 132)
    print(title)
    print("-" * 132)
    print(f"{'implementation':<34} | " + " | ".join(f"{c:>14}" for c in cols))
    for name, r in rows:
        print(f"{name:<34} | " + " | ".join(f"{r[c]:>14.3f}" for c in cols))


def main(argv=None):
    ap = argparse.ArgumentParser()
    ap.add_argument("--sweep", action="store_true", help="also run the N_CTX_KV sweep of test_speed.py")
    ap.add_argument("--small", action="store_true", help="Z=64 instead of 512/256 (quick look)")
    ap.add_argument("--json", action="store_true", help="print one JSON object with all rows at the end")
    args = ap.parse_args(argv)
    if not torch.cuda.is_available():
        sys.exit("compute_flops: needs a GPU")
    out = {}
    names = {"quantized": "this build (INT8 KV, libqfa)", "fp16": "torch SDPA (FP16)"}
    for D in (64, 128, 256):
        Z, H, Nq, Nkv = (64 if args.small else 512), 16, 16, 3000
        rows = [(names[p], measure(Z, H, Nq, Nkv, D, p)) for p in ("quantized", "fp16")]
        _table(f"Z={Z} H={H} N_CTX_Q={Nq} N_CTX_KV={Nkv} HEAD_DIM={D} fp16", rows)
        out[f"Z{Z}_H{H}_Nq{Nq}_Nkv{Nkv}_D{D}"] = dict(rows)
    if args.sweep:
        for Nkv in (512, 1024, 2048, 4096):
            Z, H, Nq, D = (64 if args.small else 256), 16, 16, 128
            rows = [(names[p], measure(Z, H, Nq, Nkv, D, p)) for p in ("quantized", "fp16")]
            _table(f"Z={Z} H={H} N_CTX_Q={Nq} N_CTX_KV={Nkv} HEAD_DIM={D} fp16", rows)
            out[f"Z{Z}_H{H}_Nq{Nq}_Nkv{Nkv}_D{D}"] = dict(rows)
    if args.json:
        print(json.dumps(out))


if __name__ == "__main__":
    main()

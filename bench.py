#!/usr/bin/env python3
"""Benchmark of the INT8 quantized flash-attention hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--quick]

Workload (the configuration the headline metric is quoted on): B=4, H=32, N=4096, D=128, causal,
bf16 q/k/v drawn N(0,1) plus a per-token mean offset N(0, 0.5), already resident in HBM.
One step = per-token INT8 quantization of Q and of K (codes, scale, zero point, row sum) followed
by the attention forward: the whole forward hot path from bf16 q, k, v to bf16 O.

FLOPs follow the reference's convention (compute_flops.py:103-104: forward = 4*B*H*Nq*Nk*D,
backward = 2.5x forward) with the causal half removed; the un-halved figure is printed too.

The single JSON line printed last carries
  value        forward TFLOP/s of the whole step (quantize Q, quantize K, attention forward)
  roofline     the attention forward kernel alone: algorithmic FLOPs per launch / mean launch
               duration from HIP events recorded around every launch of the timed region
  cpu_baseline the reference's CPU-runnable path (torch eager quantize + dequantized SDPA,
               oracle.reference_cpu_path) timed on this machine's host cores on a bounded sample
plus, under "extra": backward and fwd+bwd figures, the quantizer, the QK^T stage alone, the other two GPU
configurations (long context, small head dimension with its stand-alone quantizer rate), torch SDPA bf16 on the
same GPU as the stated stand-in for the reference's Triton kernels (which cannot run these shapes), and the
reference's own benchmark shape.  Before the warm-up steps the same step runs untimed for --settle-ms
milliseconds (reported as settle_ms) so that a short run is not measured on a clock that is still ramping.
"""
from __future__ import annotations

import argparse
import json
import math
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# MI355X published dense peaks
PEAK_INT8_TOPS = 5000.0
PEAK_BF16_TFLOPS = 2500.0
PEAK_HBM_GBS = 8000.0
# HBM bytes per forward launch at the headline configuration, measured with rocprofv3 --pmc:
# FETCH_SIZE 204 131 KiB x 2.000 (calibration: 256 MiB copy reads 131 086) + WRITE_SIZE 133 120 KiB x 1.000
# (profiles/kernels_B4_H32_N4096_D128_causal_bf16.md); algorithmic bytes are 395 MiB -- the causal dispatch
# order keeps four heads in flight per XCD, more than its L2 holds, and the re-reads show up here
FWD_TRAFFIC_BYTES = (204131 * 2 + 133120) * 1024


def flops_fwd(B, H, Nq, Nk, D, causal):
    f = 4.0 * B * H * Nq * Nk * D           # compute_flops.py:103
    return f * 0.5 if causal else f


def time_events(fn, steps, warmup):
    """Mean milliseconds per call from HIP events on torch's current stream (where fn launches)."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(cfg, budget_s=10.0):
    """Reference CPU path (torch eager quantize + dequantize + SDPA, oracle.reference_cpu_path) on head-chunks of
    the same workload until ~budget_s of CPU time per leg: forward (the headline metric's step) and forward +
    backward."""
    from oracle import oracle   # the CPU baseline is the only leg of this file that touches the oracle
    from quant_flash_attn_amd.synthetic import make_inputs
    B, H, N, D, causal = cfg["B"], cfg["H"], cfg["N"], cfg["D"], cfg["causal"]
    sm = 1.0 / math.sqrt(D)
    threads = torch.get_num_threads()
    chunk = 4
    q, k, v, do = (t.float() for t in make_inputs(cfg["dist"], 1, chunk, N, D, seed=1))

    def leg(with_bwd):
        run = (lambda a, b, c, d: oracle.reference_cpu_path(a, b, c, causal, sm, d)) if with_bwd else \
              (lambda a, b, c, d: oracle.reference_cpu_path(a, b, c, causal, sm))
        with torch.set_grad_enabled(with_bwd):
            run(q[:, :1], k[:, :1], v[:, :1], do[:, :1])      # warm-up
            done, t0 = 0, time.perf_counter()
            while True:
                run(q, k, v, do)
                done += chunk
                el = time.perf_counter() - t0
                if el >= budget_s or done >= B * H:
                    return done, el

    done, el = leg(False)
    done_b, el_b = leg(True)
    fl = flops_fwd(1, done, N, N, D, causal)
    fl_b = 3.5 * flops_fwd(1, done_b, N, N, D, causal)
    return {"value": round(fl / el / 1e12, 4), "unit": "TFLOP/s", "cores": threads, "kind": "port",
            "cpu_model": cpu_model(),
            "sample": f"{done} of {B * H} (batch,head) slices of the same workload, N={N} D={D} "
                      f"causal={causal}, fp32 torch eager quantize+dequantize+SDPA forward, {el:.1f} s",
            "fwd_bwd_value": round(fl_b / el_b / 1e12, 4),
            "fwd_bwd_sample": f"{done_b} of {B * H} slices, the same plus .backward(dO), {el_b:.1f} s"}


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--quick", action="store_true",
                    help="skip the other configurations, the torch SDPA stand-in and the D=64 reference shape")
    ap.add_argument("--settle-ms", type=float, default=300.0,
                    help="untimed milliseconds of the same step before the warm-up steps (clock settling)")
    ap.add_argument("--all-configs", action="store_true", help=argparse.SUPPRESS)   # now the default
    ap.add_argument("--sdpa", action="store_true", help=argparse.SUPPRESS)          # now the default
    ap.add_argument("--calib-copy", action="store_true",
                    help="also run a plain 256 MiB device-to-device copy (calibrates rocprofv3 FETCH_SIZE/WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build is single-GPU by design (every (batch, head) is independent; "
              "nothing here uses a second GPU). Run with --gpus 1.", file=sys.stderr)
        sys.exit(2)
    if not torch.cuda.is_available():
        print("bench.py: needs a GPU", file=sys.stderr)
        sys.exit(1)

    import quant_flash_attn_amd as qfa
    from quant_flash_attn_amd.synthetic import make_inputs

    dev = "cuda:0"
    torch.cuda.set_device(0)
    cfg = {"B": 4, "H": 32, "N": 4096, "D": 128, "causal": True, "dist": "offset"}
    B, H, N, D, causal = cfg["B"], cfg["H"], cfg["N"], cfg["D"], cfg["causal"]
    sm = 1.0 / math.sqrt(D)
    q, k, v, do = (t.to(dev) for t in make_inputs(cfg["dist"], B, H, N, D, seed=0))
    F_fwd = flops_fwd(B, H, N, N, D, causal)
    F_bwd = 2.5 * F_fwd                       # compute_flops.py:104

    # ---- the timed region: K steps of (quantize Q, quantize K, forward), wall clock, with HIP
    # events around every attention launch for the kernel's own duration
    def step(evs=None):
        qq, kq = qfa.quantize_pair_for_attention(q, k)   # both tensors in one launch, as quant_flash_attn_qkv does
        if evs is not None:
            evs[0].record()
        o, lse = qfa.attn_fwd_quantized(qq, kq, v, causal, sm)
        if evs is not None:
            evs[1].record()
        return qq, kq, o, lse

    # untimed settling: the same step until settle_ms have passed, so that the clock the timed steps see is the
    # one a long run sees (a 20-step run is 15 ms long; the shader clock takes longer than that to ramp)
    settle_t0 = time.perf_counter()
    while (time.perf_counter() - settle_t0) * 1e3 < args.settle_ms:
        step()
        torch.cuda.synchronize()
    settle_ms = (time.perf_counter() - settle_t0) * 1e3
    for _ in range(args.warmup):
        step()
    events = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        qq, kq, o, lse = step(events[i])
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_step = (t1 - t0) * 1e3 / args.steps
    launch_ms = sorted(a.elapsed_time(b) for a, b in events)
    ms_fwd_kernel = sum(launch_ms) / args.steps
    value = F_fwd / (ms_step * 1e-3) / 1e12

    # ---- extras (outside the timed region)
    extra = {}
    if args.calib_copy:
        src = torch.empty(256 << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    ms_quant = time_events(lambda: qfa.quantize_for_attention(q), 50, 10)
    tok = B * H * N
    quant_bytes = tok * (D * 2 + D + 4 + 1 + 4)          # bf16 in; codes, fp32 scale, zp, rowsum out
    extra["quant_ms_per_tensor"] = round(ms_quant, 4)
    extra["quant_GBps"] = round(quant_bytes / (ms_quant * 1e-3) / 1e9, 1)
    extra["quant_frac_hbm_peak"] = round(quant_bytes / (ms_quant * 1e-3) / 1e9 / PEAK_HBM_GBS, 4)
    # the step's form: queries and keys in one launch (twice the bytes)
    ms_pair = time_events(lambda: qfa.quantize_pair_for_attention(q, k), 50, 10)
    extra["quant_pair_ms"] = round(ms_pair, 4)
    extra["quant_pair_GBps"] = round(2 * quant_bytes / (ms_pair * 1e-3) / 1e9, 1)
    ms_fwd_only = time_events(lambda: qfa.attn_fwd_quantized(qq, kq, v, causal, sm), args.steps, 5)
    extra["fwd_kernel_ms"] = round(ms_fwd_only, 4)
    extra["fwd_kernel_tflops"] = round(F_fwd / (ms_fwd_only * 1e-3) / 1e12, 2)
    extra["fwd_kernel_tflops_unhalved_formula"] = round(2 * F_fwd / (ms_fwd_only * 1e-3) / 1e12, 2)
    ms_bwd = time_events(lambda: qfa.attn_bwd_quantized(qq, kq, v, o, do, lse, causal, sm), max(5, args.steps // 2), 3)
    extra["bwd_ms"] = round(ms_bwd, 4)
    extra["bwd_tflops"] = round(F_bwd / (ms_bwd * 1e-3) / 1e12, 2)
    extra["fwd_bwd_ms_incl_quant"] = round(ms_step + ms_bwd, 4)
    extra["fwd_bwd_tflops_incl_quant"] = round((F_fwd + F_bwd) / ((ms_step + ms_bwd) * 1e-3) / 1e12, 2)
    extra["fwd_bwd_tflops_kernels_only"] = round((F_fwd + F_bwd) / ((ms_fwd_only + ms_bwd) * 1e-3) / 1e12, 2)
    # the QK^T product is half of the forward FLOPs and runs on INT8 MFMA: over the whole kernel, and over
    # the QK^T stage alone (same kernel with the exponentials and P.V compiled out)
    extra["qk_int8_tops_over_whole_fwd_kernel"] = round(0.5 * F_fwd / (ms_fwd_only * 1e-3) / 1e12, 2)
    extra["qk_frac_int8_peak_over_whole_fwd_kernel"] = round(0.5 * F_fwd / (ms_fwd_only * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)
    ms_qk = time_events(lambda: qfa.attn_fwd_quantized(qq, kq, v, causal, sm, _entry="qfa_bench_qk_stage"), args.steps, 5)
    extra["qk_stage_ms"] = round(ms_qk, 4)
    extra["qk_stage_int8_tops"] = round(0.5 * F_fwd / (ms_qk * 1e-3) / 1e12, 2)
    extra["qk_stage_frac_int8_peak"] = round(0.5 * F_fwd / (ms_qk * 1e-3) / 1e12 / PEAK_INT8_TOPS, 4)

    # ---- the reference's own benchmark shape (compute_flops.py:96): shared K = V codes, fp16 Q, 16 queries
    # against 3000 keys.  HBM-bound: bytes = calculate_theoretical_io of compute_flops.py:39-83.
    def shared_kv_leg(D2):
        Z2, H2, Nq2, Nk2 = 512, 16, 16, 3000
        g2 = torch.Generator(device=dev).manual_seed(1)
        kv2 = torch.randn((Z2, H2, Nk2, D2), generator=g2, device=dev, dtype=torch.float16)
        codes2, scale2, zp2 = qfa.asymmetric_quant_per_token(kv2)
        del kv2
        q2 = torch.randn((Z2, H2, Nq2, D2), generator=g2, device=dev, dtype=torch.float16)
        do2 = torch.randn((Z2, H2, Nq2, D2), generator=g2, device=dev, dtype=torch.float16)
        sm2 = 1.0 / math.sqrt(D2)
        o2, lse2 = qfa.attn_fwd_shared_kv(q2, codes2, scale2, zp2, sm2)
        mf = time_events(lambda: qfa.attn_fwd_shared_kv(q2, codes2, scale2, zp2, sm2), 20, 5)
        mb = time_events(lambda: qfa.attn_bwd_shared_kv(q2, codes2, scale2, zp2, o2, do2, lse2, sm2), 10, 3)
        io_f = Z2 * H2 * (Nq2 * D2 * 2 * 2 + Nq2 * 4 + Nk2 * (D2 + 3))
        io_b = Z2 * H2 * (4 * Nq2 * D2 * 2 + 2 * Nq2 * 4 + Nk2 * (D2 + 3) + Nk2 * D2 * 2)
        fl = 4.0 * Z2 * H2 * Nq2 * Nk2 * D2
        return {"fwd_ms": round(mf, 4), "fwd_GBps": round(io_f / mf / 1e6, 1),
                "fwd_frac_hbm_peak": round(io_f / mf / 1e6 / PEAK_HBM_GBS, 4), "fwd_tflops": round(fl / mf / 1e9, 2),
                "bwd_ms": round(mb, 4), "bwd_GBps": round(io_b / mb / 1e6, 1),
                "bwd_frac_hbm_peak": round(io_b / mb / 1e6 / PEAK_HBM_GBS, 4), "bwd_tflops": round(2.5 * fl / mb / 1e9, 2)}
    extra["shared_kv_Z512_H16_Nq16_Nkv3000_D128_fp16"] = shared_kv_leg(128)
    if not args.quick:
        extra["shared_kv_Z512_H16_Nq16_Nkv3000_D64_fp16"] = shared_kv_leg(64)

    if not args.quick:
        import torch.nn.functional as Fn
        qs, ks, vs = (t.clone().requires_grad_(True) for t in (q, k, v))
        ms_s = time_events(lambda: Fn.scaled_dot_product_attention(qs.detach(), ks.detach(), vs.detach(), is_causal=causal, scale=sm), 20, 5)
        extra["torch_sdpa_bf16_fwd_ms"] = round(ms_s, 4)
        extra["torch_sdpa_bf16_fwd_tflops"] = round(F_fwd / (ms_s * 1e-3) / 1e12, 2)

        def fb():
            out = Fn.scaled_dot_product_attention(qs, ks, vs, is_causal=causal, scale=sm)
            out.backward(do)
            qs.grad = ks.grad = vs.grad = None
        ms_sb = time_events(fb, 10, 3)
        extra["torch_sdpa_bf16_fwd_bwd_ms"] = round(ms_sb, 4)
        extra["torch_sdpa_bf16_fwd_bwd_tflops"] = round((F_fwd + F_bwd) / (ms_sb * 1e-3) / 1e12, 2)

    if not args.quick:
        others = {"long_context_B1_H16_N16384_D128_noncausal": (1, 16, 16384, 128, False, "outlier"),
                  "small_head_B16_H16_N2048_D64_causal": (16, 16, 2048, 64, True, "uniform"),
                  # the widest head compute_flops.py:94 sweeps, at the headline's token count and model width
                  "wide_head_B4_H16_N4096_D256_causal": (4, 16, 4096, 256, True, "offset")}
        del q, k, v, do, qq, kq, o, lse
        for name, (b2, h2, n2, d2, c2, dist) in others.items():
            q2, k2, v2, do2 = (t.to(dev) for t in make_inputs(dist, b2, h2, n2, d2, seed=0))
            sm2 = 1.0 / math.sqrt(d2)
            f2 = flops_fwd(b2, h2, n2, n2, d2, c2)
            qq2, kq2 = qfa.quantize_for_attention(q2), qfa.quantize_for_attention(k2)
            o2, lse2 = qfa.attn_fwd_quantized(qq2, kq2, v2, c2, sm2)
            mq = time_events(lambda: qfa.quantize_for_attention(q2), 30, 5)
            mf = time_events(lambda: qfa.attn_fwd_quantized(qq2, kq2, v2, c2, sm2), 20, 3)
            mb = time_events(lambda: qfa.attn_bwd_quantized(qq2, kq2, v2, o2, do2, lse2, c2, sm2), 10, 2)
            qb = b2 * h2 * n2 * (d2 * 2 + d2 + 9)
            extra[name] = {"fwd_ms": round(mf, 4), "fwd_tflops": round(f2 / mf / 1e9, 2), "bwd_ms": round(mb, 4),
                           "bwd_tflops": round(2.5 * f2 / mb / 1e9, 2),
                           "fwd_bwd_tflops": round(3.5 * f2 / (mf + mb) / 1e9, 2),
                           "quant_ms_per_tensor": round(mq, 4), "quant_GBps": round(qb / mq / 1e6, 1),
                           "quant_frac_hbm_peak": round(qb / mq / 1e6 / PEAK_HBM_GBS, 4)}
            del q2, k2, v2, do2, qq2, kq2, o2, lse2

    # ---- roofline of the dominant kernel (attention forward): half its FLOPs are INT8 (QK^T), half
    # bf16 (P.V), so the MFMA time floor is F/2/P_int8 + F/2/P_bf16 and the peak it is priced
    # against is the harmonic blend of the two published peaks
    peak_blend = 2.0 / (1.0 / PEAK_INT8_TOPS + 1.0 / PEAK_BF16_TFLOPS)
    achieved = F_fwd / (ms_fwd_kernel * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": "fwd_kernel<bf16,128,causal>", "achieved": round(achieved, 2),
                "peak": round(peak_blend, 1), "unit": "TFLOP/s", "frac": round(achieved / peak_blend, 4),
                "traffic": FWD_TRAFFIC_BYTES, "algorithmic_flops_per_launch": F_fwd,
                "mean_launch_ms": round(ms_fwd_kernel, 4), "min_launch_ms": round(launch_ms[0], 4),
                "median_launch_ms": round(launch_ms[len(launch_ms) // 2], 4),
                "frac_of_bf16_peak": round(achieved / PEAK_BF16_TFLOPS, 4),
                "peak_note": "harmonic blend of published dense INT8 (5.0 POP/s, QK^T half) and bf16 (2.5 PFLOP/s, PV half)"}

    result = {
        "metric": "attn TFLOPS fwd & fwd+bwd @B4 H32 N4096 D128 causal; % of INT8 MFMA peak",
        "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_step, 4), "settle_ms": round(settle_ms, 1), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 (QK^T, int32 accumulate) + bf16 (P.V) + fp32 softmax", "data": "synthetic",
        "config": {"workload": "forward causal B=4 H=32 N=4096 D=128 bf16: quantize Q, quantize K, attention forward",
                   "flops_convention": "4*B*H*N*N*D/2 (compute_flops.py:103, causal-halved)"},
        "roofline": roofline,
        "cpu_baseline": None if args.no_cpu else cpu_baseline(cfg),
        "extra": extra,
    }
    print(json.dumps(result))


if __name__ == "__main__":
    main()

"""Committed known answers (tests/golden/, written by tests/golden/make_golden.py from the exact-rational
model of the quantizer and from plain fp64 torch formulas): the CPU oracle must reproduce them exactly
(quantizer) or to fp32 round-off (attention), and the HIP kernels must meet them at the same bars as
against the oracle -- bit-exact codes / zero points / scales, O and gradients within 2e-2 (scaled) and
cosine >= 0.999."""
import json
import os
import struct

import numpy as np
import pytest
import torch

from helpers import assert_close
from oracle import oracle

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DEV = "cuda:0"


def _kat():
    with open(os.path.join(GOLDEN, "quant_kat.json")) as f:
        d = json.load(f)
    rows = d["rows"]
    x = torch.tensor([[struct.unpack("<f", struct.pack("<I", b))[0] for b in r["x_bits"]] for r in rows],
                     dtype=torch.float32)
    codes = torch.tensor([r["codes"] for r in rows], dtype=torch.int8)
    scale = torch.tensor([struct.unpack("<f", struct.pack("<I", r["scale_bits"]))[0] for r in rows], dtype=torch.float32)
    zp = torch.tensor([r["zp"] for r in rows], dtype=torch.int8)
    rowsum = torch.tensor([r["rowsum"] for r in rows], dtype=torch.int32)
    return [r["name"] for r in rows], x, codes, scale, zp, rowsum


def _attn_cases():
    z = np.load(os.path.join(GOLDEN, "attn_small.npz"), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in z.files})
    return {n: {k.split("/")[1]: z[k] for k in z.files if k.startswith(n + "/")} for n in names}


def _bf16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.bfloat16)


def test_fixture_files_are_complete():
    names, x, codes, scale, zp, rowsum = _kat()
    assert len(names) >= 30 and x.shape == codes.shape and x.shape[1] == 32
    cases = _attn_cases()
    assert set(cases) == {"causal_N64_D64", "ragged_Nq24_Nk72_D128"}
    for c in cases.values():
        assert {"q", "k", "v", "do", "qc", "zq", "sq", "kc", "zk", "sk", "o", "lse", "dq", "dk", "dv"} <= set(c)


def test_oracle_quantizer_reproduces_known_answers():
    names, x, codes, scale, zp, rowsum = _kat()
    for impl in ("numpy", "c"):
        if impl == "numpy":
            c, _, z, s32, rs = oracle.quantize_per_token(x[None, None], torch.float32)
        else:
            c, s32, z, rs = oracle.quantize_per_token_c(x[None, None])
        c, z, s32, rs = c[0, 0], z.reshape(-1), s32.reshape(-1), rs.reshape(-1)
        for i, n in enumerate(names):
            assert torch.equal(c[i], codes[i]), f"{impl}: codes of row {i} ({n})"
            assert int(z[i]) == int(zp[i]) and float(s32[i]) == float(scale[i]) and int(rs[i]) == int(rowsum[i]), \
                f"{impl}: scale / zero point / row sum of row {i} ({n})"


def test_oracle_attention_reproduces_known_answers():
    for name, c in _attn_cases().items():
        q, k, v, do = (_bf16(c[t]) for t in ("q", "k", "v", "do"))
        qc, _, zq, sq, _ = oracle.quantize_per_token(q, torch.float32)
        kc, _, zk, sk, _ = oracle.quantize_per_token(k, torch.float32)
        assert np.array_equal(qc.numpy(), c["qc"]) and np.array_equal(kc.numpy(), c["kc"]), name
        assert np.array_equal(zq.reshape(c["zq"].shape).numpy(), c["zq"]) and np.array_equal(sk.reshape(c["sk"].shape).numpy(), c["sk"])
        qh = oracle.dequantize_per_token(qc, sq, zq, torch.float64)
        kh = oracle.dequantize_per_token(kc, sk, zk, torch.float64)
        causal, sm = bool(c["causal"]), float(c["sm_scale"])
        o, lse = oracle.attn_fwd(qh, kh, v, causal, sm)
        dq, dk, dv = oracle.attn_bwd(qh, kh, v, do, causal, sm)
        for got, key in ((o, "o"), (lse, "lse"), (dq, "dq"), (dk, "dk"), (dv, "dv")):
            ref = torch.from_numpy(c[key]).double()
            assert (got.double().reshape(ref.shape) - ref).abs().max() <= 2e-6 * max(1.0, ref.abs().max().item()), (name, key)


@pytest.mark.gpu
def test_kernels_meet_quantizer_known_answers(qfa):
    names, x, codes, scale, zp, rowsum = _kat()
    for dtype in (torch.float32,):
        qt = qfa.quantize_for_attention(x[None, None].to(DEV).to(dtype))
        assert torch.equal(qt.codes.cpu()[0, 0], codes)
        assert torch.equal(qt.zero_point.cpu().reshape(-1), zp)
        assert torch.equal(qt.scale.cpu().reshape(-1), scale)
        assert torch.equal(qt.rowsum.cpu().reshape(-1), rowsum)


@pytest.mark.gpu
def test_kernels_meet_attention_known_answers(qfa):
    for name, c in _attn_cases().items():
        q, k, v, do = (_bf16(c[t]).to(DEV) for t in ("q", "k", "v", "do"))
        causal, sm = bool(c["causal"]), float(c["sm_scale"])
        qq, kq = qfa.quantize_for_attention(q), qfa.quantize_for_attention(k)
        assert np.array_equal(qq.codes.cpu().numpy(), c["qc"]) and np.array_equal(kq.codes.cpu().numpy(), c["kc"]), name
        o, lse = qfa.attn_fwd_quantized(qq, kq, v, causal, sm)
        dq, dk, dv = qfa.attn_bwd_quantized(qq, kq, v, o, do, lse, causal, sm)
        torch.cuda.synchronize()
        assert_close(f"{name} O", o.cpu(), torch.from_numpy(c["o"]).double())
        assert (lse.cpu().double().reshape(c["lse"].shape) - torch.from_numpy(c["lse"]).double()).abs().max() < 2.0 ** -8
        assert_close(f"{name} dQ", dq.cpu(), torch.from_numpy(c["dq"]).double(), scaled=True)
        assert_close(f"{name} dK", dk.cpu(), torch.from_numpy(c["dk"]).double(), scaled=True)
        assert_close(f"{name} dV", dv.cpu(), torch.from_numpy(c["dv"]).double(), scaled=True)


def _shared_kv_cases():
    z = np.load(os.path.join(GOLDEN, "shared_kv_small.npz"), allow_pickle=False)
    names = sorted({k.split("/")[0] for k in z.files})
    return {n: {k.split("/")[1]: z[k] for k in z.files if k.startswith(n + "/")} for n in names}


def _f16(bits: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(bits.view(np.int16).copy()).view(torch.float16)


def test_oracle_shared_kv_reproduces_known_answers():
    """oracle.legacy_fwd / legacy_bwd (quant_flash_attn.py:22-166 restated) against the fixture's plain
    fp64 formulas, and the oracle quantizer against the fixture's exactly quantized kv."""
    cases = _shared_kv_cases()
    assert set(cases) == {"Nq16_Nk100_D128", "Nq5_Nk70_D64"}
    for name, c in cases.items():
        q, kv, do = _f16(c["q"]), _f16(c["kv"]), _f16(c["do"])
        codes, scale16, zp, _, _ = oracle.quantize_per_token(kv, torch.float16)
        assert np.array_equal(codes.numpy(), c["codes"]), name
        assert np.array_equal(zp.reshape(c["zp"].shape).numpy(), c["zp"]), name
        assert torch.equal(scale16.reshape(c["scale16"].shape), _f16(c["scale16"])), name
        sm = float(c["sm_scale"])
        o, lse = oracle.legacy_fwd(q, codes, scale16, zp, sm)
        dq, dkv = oracle.legacy_bwd(q, codes, scale16, zp, do, sm)
        for got, key in ((o, "o"), (lse, "lse"), (dq, "dq"), (dkv, "dkv")):
            ref = torch.from_numpy(c[key]).double()
            assert (got.double().reshape(ref.shape) - ref).abs().max() <= 2e-6 * max(1.0, ref.abs().max().item()), (name, key)


@pytest.mark.gpu
def test_kernels_meet_shared_kv_known_answers(qfa):
    """The reference's entry point end to end (quantizer + shared-KV forward + backward kernels)."""
    for name, c in _shared_kv_cases().items():
        q = _f16(c["q"]).to(DEV).requires_grad_(True)
        kv = _f16(c["kv"]).to(DEV).requires_grad_(True)
        sm = float(c["sm_scale"])
        kv_quant = qfa.asymmetric_quant_per_token(kv.detach())
        assert np.array_equal(kv_quant[0].cpu().numpy(), c["codes"]), name
        assert np.array_equal(kv_quant[2].cpu().reshape(c["zp"].shape).numpy(), c["zp"]), name
        assert torch.equal(kv_quant[1].cpu().reshape(c["scale16"].shape), _f16(c["scale16"])), name
        o = qfa.quant_flash_attn(q, kv, kv_quant, sm)
        o.backward(_f16(c["do"]).to(DEV))
        _, lse = qfa.attn_fwd_shared_kv(q.detach(), *kv_quant, sm)
        torch.cuda.synchronize()
        assert_close(f"{name} O", o.detach().cpu(), torch.from_numpy(c["o"]).double(), scaled=True)
        assert (lse.cpu().double().reshape(c["lse"].shape) - torch.from_numpy(c["lse"]).double()).abs().max() < 2.0 ** -8
        assert_close(f"{name} dQ", q.grad.cpu(), torch.from_numpy(c["dq"]).double(), scaled=True)
        assert_close(f"{name} dKV", kv.grad.cpu(), torch.from_numpy(c["dkv"]).double(), scaled=True)

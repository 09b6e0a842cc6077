"""Pins the CPU oracle of the per-token quantizer (oracle/oracle.py, oracle/quant_oracle.c).

The reference ships no golden vectors for this path (its only test compares with fp16 SDPA at
atol 1e-1), so the oracle is pinned by: an exact-rational evaluation of every binary32 operation
of asymmetric_quant.py:84-104, hand-computed known answers, constructed rounding ties (half away
from zero, where half-to-even would differ), invariants, and agreement of the two independent
restatements (numpy and C).
"""
import math
from fractions import Fraction

import numpy as np
import pytest
import torch

from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs


from exact_model import quant_row_exact, rn32, roundf_exact  # noqa: F401  (exact model of binary32 arithmetic)


def test_rn32_matches_numpy_casts():
    rng = np.random.default_rng(0)
    for v in rng.standard_normal(200) * 10.0 ** rng.integers(-6, 6, 200):
        assert float(rn32(Fraction(float(v)))) == float(np.float32(v))
    # a tie between two binary32 neighbours goes to the even one
    lo = Fraction(1) + Fraction(2) ** -23
    assert rn32(lo + Fraction(2) ** -24) == Fraction(1) + Fraction(2) ** -22


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("dist", ["normal", "offset", "uniform", "positive", "tiny_range"])
def test_oracle_matches_exact_rational_model(dtype, dist):
    g = torch.Generator().manual_seed(hash((str(dtype), dist)) % 2**31)
    D, rows = 16, 24
    if dist == "normal":
        x = torch.randn(rows, D, generator=g)
    elif dist == "offset":
        x = torch.randn(rows, D, generator=g) + 3 * torch.randn(rows, 1, generator=g)
    elif dist == "uniform":
        x = torch.rand(rows, D, generator=g) * 8 - 3
    elif dist == "positive":
        x = torch.rand(rows, D, generator=g) * 2 + 5          # zero point clamps at -128
    else:
        x = 1.0 + torch.rand(rows, D, generator=g) * 1e-3     # scale is tiny
    x = x.to(dtype)
    codes, _, zp, scale32, rowsum = oracle.quantize_per_token(x, torch.float32)
    c_codes, c_scale, c_zp, c_rowsum = oracle.quantize_per_token_c(x)
    for r in range(rows):
        e_codes, e_scale, e_zp = quant_row_exact(x[r].to(torch.float32).tolist())
        assert codes[r].tolist() == e_codes
        assert int(zp[r]) == e_zp
        assert Fraction(float(scale32[r])) == e_scale
        assert int(rowsum[r]) == sum(e_codes)
    assert torch.equal(codes, c_codes) and torch.equal(zp, c_zp)
    assert torch.equal(scale32, c_scale) and torch.equal(rowsum, c_rowsum)


# ---------------------------------------------------------------- hand-computed known answers
def test_known_answers():
    # range 255 -> scale exactly 1, zp = -128: codes are x - 128
    x = torch.tensor([[0.0, 255.0, 1.0, 100.0]])
    codes, scale, zp, scale32, rowsum = oracle.quantize_per_token(x)
    assert scale32.item() == 1.0 and zp.item() == -128
    assert codes.tolist() == [[-128, 127, -127, -28]] and rowsum.item() == -128 + 127 - 127 - 28
    assert scale.dtype == torch.float16 and scale.item() == 1.0
    # [-1, 0, 1, 2]: scale = 3/255 = 1/85, zp = round(-128 + 85) = -43, codes = 85 x - 43
    codes, _, zp, scale32, _ = oracle.quantize_per_token(torch.tensor([[-1.0, 0.0, 1.0, 2.0]]))
    assert zp.item() == -43 and codes.tolist() == [[-128, -43, 42, 127]]
    assert scale32.item() == float(np.float32(3.0) / np.float32(255.0))
    # constant row: scale forced to 1 (asymmetric_quant.py:87); zp = clamp(round(-128 - c))
    codes, _, zp, scale32, _ = oracle.quantize_per_token(torch.full((1, 8), 3.0))
    assert scale32.item() == 1.0 and zp.item() == -128 and codes.tolist() == [[-125] * 8]
    codes, _, zp, scale32, _ = oracle.quantize_per_token(torch.full((1, 8), -200.0))
    assert scale32.item() == 1.0 and zp.item() == 72 and codes.tolist() == [[-128] * 8]
    # all-positive row: zero point clamps at -128 and large values saturate at 127
    codes, _, zp, _, _ = oracle.quantize_per_token(torch.tensor([[100.0, 355.0, 228.0]]))
    assert zp.item() == -128 and codes.tolist() == [[-28, 127, 100]]
    # all-negative row: zero point clamps at +127
    codes, _, zp, _, _ = oracle.quantize_per_token(torch.tensor([[-355.0, -100.0]]))
    assert zp.item() == 127 and codes.tolist() == [[-128, 27]]


def test_rounding_is_half_away_from_zero():
    # scale = 1, zp = -128, so y = x - 128 hits exact .5 ties; half-to-even would give
    # [-128, -126, -126, 0, 2, 2] for the six middle entries
    x = torch.tensor([[0.0, 255.0, 0.5, 1.5, 2.5, 128.5, 129.5, 130.5]])
    codes, _, zp, scale32, _ = oracle.quantize_per_token(x)
    assert scale32.item() == 1.0 and zp.item() == -128
    assert codes.tolist() == [[-128, 127, -128, -127, -126, 1, 2, 3]]
    assert oracle.quantize_per_token_c(x)[0].tolist() == codes.tolist()
    # zero-point tie: min = -11.5, max = 243.5 -> zpf = -116.5 -> -117 (half-to-even: -116)
    x = torch.tensor([[-11.5, 243.5, 0.0]])
    for zp in (oracle.quantize_per_token(x)[2], oracle.quantize_per_token_c(x)[2]):
        assert zp.item() == -117
    # roundf helper itself, including the value floor(|y| + 0.5) gets wrong
    y = np.array([0.5, -0.5, 1.5, 2.5, -2.5, 0.49999997, -0.49999997, 8388609.0, -0.0, 3.0], dtype=np.float32)
    assert oracle.roundf_half_away(y).tolist() == [1, -1, 2, 3, -3, 0, -0.0, 8388609.0, -0.0, 3.0]


def test_fp16_scale_is_rne_cast_of_fp32_scale():
    x = torch.randn(64, 128, generator=torch.Generator().manual_seed(3))
    _, scale16, _, scale32, _ = oracle.quantize_per_token(x, torch.float16)
    assert torch.equal(scale16, scale32.to(torch.float16))


# ---------------------------------------------------------------- invariants on realistic rows
@pytest.mark.parametrize("config", ["normal", "offset", "outlier", "uniform"])
def test_invariants(config):
    q, k, _, _ = make_inputs(config, 1, 2, 256, 128, seed=1)
    for x in (q, k):
        codes, _, zp, scale32, rowsum = oracle.quantize_per_token(x)
        xf = x.float()
        assert codes.dtype == torch.int8 and zp.dtype == torch.int8
        assert torch.equal(rowsum, codes.to(torch.int32).sum(-1, keepdim=True))
        # the row minimum maps to -128 and the maximum to +127 (both signs present here, so the
        # zero point is not clamped); +-1 allowed for the fp32 rounding of the add
        cmin = codes.gather(-1, xf.argmin(-1, keepdim=True)).int()
        cmax = codes.gather(-1, xf.argmax(-1, keepdim=True)).int()
        assert (cmin <= -127).all() and (cmax >= 126).all()
        # monotone: sorting x sorts the codes
        order = xf.argsort(-1)
        assert (codes.gather(-1, order).int().diff(dim=-1) >= 0).all()
        # reconstruction error is at most one quantization step
        xh = oracle.dequantize_per_token(codes, scale32, zp)
        assert ((xh - xf).abs() <= scale32 * 1.0001).all()


def test_c_and_numpy_restatements_agree_on_large_input():
    q, k, _, _ = make_inputs("offset", 2, 4, 1024, 128, seed=5)
    for x in (q, k.float() * 3.7):
        n_codes, _, n_zp, n_scale, n_rowsum = oracle.quantize_per_token(x)
        c_codes, c_scale, c_zp, c_rowsum = oracle.quantize_per_token_c(x)
        assert torch.equal(n_codes, c_codes) and torch.equal(n_zp, c_zp)
        assert torch.equal(n_scale, c_scale) and torch.equal(n_rowsum, c_rowsum)


def test_torch_eager_baseline_matches_oracle():
    """The torch-eager quantizer that the CPU baseline times gives the oracle's codes."""
    q, _, _, _ = make_inputs("uniform", 1, 2, 512, 64, seed=2)
    codes, scale, zp = oracle._quantize_torch_eager(q)
    o_codes, _, o_zp, o_scale, _ = oracle.quantize_per_token(q)
    assert torch.equal(codes, o_codes) and torch.equal(zp, o_zp) and torch.equal(scale, o_scale)


def test_dequantize_closed_form():
    codes = torch.tensor([[[-128, 0, 127]]], dtype=torch.int8)
    scale = torch.tensor([[[0.5]]])
    zp = torch.tensor([[[-3]]], dtype=torch.int8)
    assert oracle.dequantize_per_token(codes, scale, zp).tolist() == [[[-62.5, 1.5, 65.0]]]

"""GPU parity of the HIP per-token quantizer: codes, zero points, fp32 scale and row sums must be
bit-identical to the CPU oracle (asymmetric_quant.py:66-106 restated) on the same inputs."""
import pytest
import torch

from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _check(qfa, x_cpu, name=""):
    xg = x_cpu.to(DEV)
    got = qfa.quantize_for_attention(xg)
    codes, scale16, zp = qfa.asymmetric_quant_per_token(xg)
    torch.cuda.synchronize()
    o_codes, o_scale, o_zp, o_rowsum = oracle.quantize_per_token_c(x_cpu)
    assert torch.equal(got.codes.cpu(), o_codes), f"{name}: codes differ in {(got.codes.cpu() != o_codes).sum().item()} places"
    assert torch.equal(got.zero_point.cpu(), o_zp), f"{name}: zero points differ"
    assert torch.equal(got.scale.cpu(), o_scale), f"{name}: fp32 scales differ"
    assert torch.equal(got.rowsum.cpu(), o_rowsum), f"{name}: row sums differ"
    # reference return structure: int8 codes, fp16 scale [B,H,N,1], int8 zero point [B,H,N,1]
    assert codes.dtype == torch.int8 and scale16.dtype == torch.float16 and zp.dtype == torch.int8
    assert scale16.shape == x_cpu.shape[:-1] + (1,) and zp.shape == scale16.shape
    assert torch.equal(codes.cpu(), o_codes) and torch.equal(zp.cpu(), o_zp)
    assert torch.equal(scale16.cpu(), o_scale.to(torch.float16))
    return got


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", [32, 64, 128, 256])
@pytest.mark.parametrize("config", ["normal", "offset", "outlier", "uniform"])
def test_bit_exact_vs_oracle(qfa, dtype, D, config):
    q, k, _, _ = make_inputs(config, 2, 3, 257, D, seed=D, dtype=dtype)   # ragged N
    _check(qfa, q, f"{config}/q")
    _check(qfa, k, f"{config}/k")


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
@pytest.mark.parametrize("D", [8, 40, 96, 136, 200, 248])
def test_any_head_dim_that_is_a_multiple_of_eight(qfa, dtype, D):
    """The reference handles any HEAD_DIM by masking the tail of its power-of-two block (asymmetric_quant.py:72-75,
    97-99); here the lanes past the row hold a copy of its first elements.  Bit-exact codes, zero points, scales and
    row sums, and the dequantizer on the same widths."""
    config = "offset" if D % 16 else "uniform"
    q, _, _, _ = make_inputs(config, 2, 3, 131, D, seed=D, dtype=dtype)
    got = _check(qfa, q, f"D={D}")
    from quant_flash_attn_amd import dequantize_per_token
    back = dequantize_per_token(got.codes, got.scale, got.zero_point, torch.float32).cpu()
    want = oracle.dequantize_per_token(got.codes.cpu(), got.scale.cpu(), got.zero_point.cpu(), torch.float32)
    assert torch.equal(back, want.reshape(back.shape))


def test_ties_saturation_and_constant_rows(qfa):
    rows = torch.zeros(8, 64)
    rows[0, :8] = torch.tensor([0.0, 255.0, 0.5, 1.5, 2.5, 128.5, 129.5, 130.5])   # exact .5 ties, scale 1
    rows[1, :3] = torch.tensor([-11.5, 243.5, 0.0])                                 # zero-point tie
    rows[2] = 3.0                                                                   # constant row
    rows[3] = -200.0
    rows[4] = torch.linspace(100.0, 355.0, 64)                                      # zp clamps at -128
    rows[5] = torch.linspace(-355.0, -100.0, 64)                                    # zp clamps at +127
    rows[6] = 1.0 + torch.arange(64) * 1e-6                                         # tiny range
    rows[7] = torch.arange(64) * 1e-41                                              # subnormal range
    x = rows.reshape(1, 1, 8, 64)
    got = _check(qfa, x, "special rows")
    assert got.codes[0, 0, 0, :8].tolist() == [-128, 127, -128, -127, -126, 1, 2, 3]
    assert got.zero_point[0, 0, 1].item() == -117


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_wide_exponent_range(qfa, dtype):
    """Tokens scaled by 2^k, k in [-75, 75]: exercises both division paths of the kernel (the FMA
    refinement used in the common exponent range and the IEEE division outside it), plus rows whose
    range is far smaller than their offset."""
    g = torch.Generator().manual_seed(11)
    B, H, N, D = 2, 4, 4096, 128
    x = torch.randn(B, H, N, D, generator=g)
    k = torch.randint(-75, 76, (B, H, N, 1), generator=g).float()
    x = x * torch.exp2(k)
    x[0, 0, ::7] = 1.0 + x[0, 0, ::7].sign() * 1e-5          # tiny range on a large offset
    x[0, 1, ::5] += 300.0                                     # all-positive rows, zero point clamps
    _check(qfa, x.to(dtype), "wide exponent range")


def test_strided_input(qfa):
    """[B,N,H,D] storage viewed as [B,H,N,D] (the usual projection layout)."""
    base = torch.randn(2, 300, 4, 128, generator=torch.Generator().manual_seed(9)).to(torch.bfloat16)
    x = base.permute(0, 2, 1, 3)
    assert not x.is_contiguous()
    xg = base.to(DEV).permute(0, 2, 1, 3)
    got = qfa.quantize_for_attention(xg)
    o_codes, o_scale, o_zp, o_rowsum = oracle.quantize_per_token_c(x.contiguous())
    assert torch.equal(got.codes.cpu(), o_codes) and torch.equal(got.zero_point.cpu(), o_zp)
    assert torch.equal(got.scale.cpu(), o_scale) and torch.equal(got.rowsum.cpu(), o_rowsum)


@pytest.mark.parametrize("config,B,H,N,D", [("offset", 4, 32, 4096, 128), ("uniform", 16, 16, 2048, 64)])
def test_full_size_bit_exact(qfa, config, B, H, N, D):
    """Whole benchmark-size tensors (524 288 tokens) against the C oracle."""
    q, _, _, _ = make_inputs(config, B, H, N, D, seed=0)
    _check(qfa, q, f"{config} full size")


def test_dequantize_kernel(qfa):
    q, _, _, _ = make_inputs("offset", 1, 2, 130, 128, seed=4)
    got = qfa.quantize_for_attention(q.to(DEV))
    ref = oracle.dequantize_per_token(got.codes.cpu(), got.scale.cpu(), got.zero_point.cpu())
    out32 = qfa.dequantize_per_token(got.codes, got.scale, got.zero_point, torch.float32)
    assert torch.equal(out32.cpu(), ref)                                    # one fp32 sub and mul: exact match
    out16 = qfa.dequantize_per_token(got.codes, got.scale.to(torch.float16), got.zero_point, torch.bfloat16)
    ref16 = oracle.dequantize_per_token(got.codes.cpu(), got.scale.cpu().to(torch.float16), got.zero_point.cpu())
    assert torch.equal(out16.cpu(), ref16.to(torch.bfloat16))


@pytest.mark.parametrize("D", [8, 64, 96, 128, 200, 256])
def test_code_rowsum_kernel(qfa, D):
    """Row sums of given codes (qfa_code_rowsum): equal to the integer sum, on contiguous and on strided codes."""
    g = torch.Generator().manual_seed(D)
    codes = torch.randint(-128, 128, (2, 3, 133, D), generator=g, dtype=torch.int8)
    codes[0, 0, 0] = 127
    codes[0, 0, 1] = -128
    got = qfa.code_rowsum(codes.to(DEV))
    want = codes.to(torch.int32).sum(-1, keepdim=True)
    assert got.dtype == torch.int32 and got.shape == (2, 3, 133, 1) and torch.equal(got.cpu(), want)
    strided = codes.permute(0, 2, 1, 3).contiguous().to(DEV).permute(0, 2, 1, 3)      # [B,N,H,D] storage
    assert torch.equal(qfa.code_rowsum(strided).cpu(), want)


def test_outputs_fully_written_and_deterministic(qfa):
    q, _, _, _ = make_inputs("normal", 1, 3, 1000, 64, seed=6)
    xg = q.to(DEV)
    a = qfa.quantize_for_attention(xg)
    b = qfa.quantize_for_attention(xg)
    for s, t in zip(a, b):
        assert torch.equal(s, t)


@pytest.mark.parametrize("D,dtype", [(128, torch.bfloat16), (64, torch.float16), (40, torch.float32), (256, torch.bfloat16)])
def test_pair_launch_is_bit_identical_to_two_launches(qfa, D, dtype):
    """quantize_pair_for_attention (queries and keys in one launch, qfa_quant_per_token_pair) against two calls of
    quantize_for_attention: every output tensor bit for bit, with different lengths and a strided second tensor."""
    g = torch.Generator().manual_seed(D)
    q = (torch.randn((2, 3, 333, D), generator=g) * 1.7 + 0.3).to(dtype).to(DEV)
    k_store = (torch.randn((2, 1029, 3, D), generator=g) - 0.5).to(dtype).to(DEV)   # [B,N,H,D] storage
    k = k_store.permute(0, 2, 1, 3)
    a0, a1 = qfa.quantize_pair_for_attention(q, k)
    b0, b1 = qfa.quantize_for_attention(q), qfa.quantize_for_attention(k)
    for got, want in ((a0, b0), (a1, b1)):
        for x, y in zip(got, want):
            assert x.shape == y.shape and x.dtype == y.dtype and torch.equal(x, y)

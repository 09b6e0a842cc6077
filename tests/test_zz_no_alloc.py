"""The entry point that allocates nothing: qfa_attn_fwd_shared_kv_static keeps the partial results of a split
over keys in a static device array inside the library instead of a caller workspace.  It runs the same
kernels with the same plan as qfa_attn_fwd_shared_kv given a workspace, so O and LSE must be bit-identical --
on two calls in a row that share the array, the second on a smaller input (stale partial results of the first
call lie beyond and between the ones the second call writes)."""
import math

import pytest
import torch

from oracle import oracle
from quant_flash_attn_amd.synthetic import make_inputs

DEV = "cuda:0"


def _problem(qfa, B, H, Nq, Nk, D, dtype, seed):
    q, kv, _, _ = make_inputs("offset", B, H, max(Nq, Nk), D, seed=seed, dtype=dtype)
    q, kv = q[:, :, :Nq].contiguous().to(DEV), kv[:, :, :Nk].contiguous().to(DEV)
    codes, scale, zp = qfa.asymmetric_quant_per_token(kv)
    return q, codes, scale.float().reshape(-1).contiguous(), zp.reshape(-1).contiguous()


def _call(L, entry, q, codes, scale, zp, sm, workspace=None):
    from quant_flash_attn_amd import _lib
    B, H, Nq, D = q.shape
    Nk = codes.shape[2]
    o = torch.full((B, H, Nq, D), float("nan"), dtype=q.dtype, device=q.device)
    lse = torch.full((B, H, Nq), float("nan"), dtype=torch.float32, device=q.device)
    s3 = lambda t: (t.stride(0), t.stride(1), t.stride(2))
    args = [q.data_ptr(), codes.data_ptr(), scale.data_ptr(), _lib.QFA_F32, zp.data_ptr(), o.data_ptr(), lse.data_ptr(),
            _lib.DTYPE_CODE[q.dtype], B, H, Nq, Nk, D, *s3(q), *s3(codes), *s3(o), sm]
    if entry == "qfa_attn_fwd_shared_kv":
        args += [workspace.data_ptr() if workspace is not None else None, workspace.numel() if workspace is not None else 0]
    rc = getattr(L, entry)(*args, _lib.stream_of(q))
    assert rc == 0, L.qfa_last_error()
    return o, lse


@pytest.mark.gpu
def test_static_scratch_entry_point_matches_the_workspace_one(qfa):
    from quant_flash_attn_amd import _lib
    L = _lib.lib()
    # (B, H, Nq, Nk, D, dtype): the first splits its keys widely, the second is smaller in every respect and
    # splits differently, the third needs no split at all (the array is not touched)
    shapes = [(1, 8, 40, 16384, 128, torch.float16), (1, 3, 5, 6000, 64, torch.bfloat16), (2, 300, 16, 200, 128, torch.float16)]
    for i, (B, H, Nq, Nk, D, dtype) in enumerate(shapes):
        need = L.qfa_attn_fwd_shared_kv_workspace_bytes(B, H, Nq, Nk, D)
        assert (need > 0) == (i < 2) and need <= (16 << 20)
        q, codes, scale, zp = _problem(qfa, B, H, Nq, Nk, D, dtype, seed=10 + i)
        sm = 1.0 / math.sqrt(D)
        ws = torch.empty(max(need, 16), dtype=torch.uint8, device=DEV)
        o_ws, lse_ws = _call(L, "qfa_attn_fwd_shared_kv", q, codes, scale, zp, sm, ws if need else None)
        o_st, lse_st = _call(L, "qfa_attn_fwd_shared_kv_static", q, codes, scale, zp, sm)
        torch.cuda.synchronize()
        assert not torch.isnan(o_st.float()).any() and not torch.isnan(lse_st).any()
        assert torch.equal(o_st, o_ws), f"shape {i}: O differs from the workspace entry point"
        assert torch.equal(lse_st, lse_ws), f"shape {i}: LSE differs from the workspace entry point"
        o_ref, lse_ref = oracle.legacy_fwd(q.cpu(), codes.cpu(), scale.cpu().reshape(B, H, Nk, 1),
                                           zp.cpu().reshape(B, H, Nk, 1), sm)
        assert (o_st.cpu().double() - o_ref.double()).abs().max() <= 2e-2 * max(1.0, float(o_ref.abs().max()))
        assert (lse_st.cpu().double() - lse_ref.double()).abs().max() < 2.0 ** -8


def test_static_scratch_rejects_what_does_not_fit(qfa):
    """Validation needs no GPU: a split whose partial results exceed the built-in array is refused."""
    from quant_flash_attn_amd import _lib
    L = _lib.lib()
    B, H, Nq, Nk, D = 1, 500, 16, 4096, 256
    assert L.qfa_attn_fwd_shared_kv_workspace_bytes(B, H, Nq, Nk, D) > (16 << 20)
    p = 0x1000   # never dereferenced
    sq, sc = (H * Nq * D, Nq * D, D), (H * Nk * D, Nk * D, D)
    rc = L.qfa_attn_fwd_shared_kv_static(p, p, p, 0, p, p, p, 1, B, H, Nq, Nk, D, *sq, *sc, *sq, 0.1, None)
    assert rc == -2 and b"scratch" in L.qfa_last_error()
    rc = L.qfa_attn_fwd_shared_kv_static(None, p, p, 0, p, p, p, 1, B, H, Nq, Nk, D, *sq, *sc, *sq, 0.1, None)
    assert rc == -1 and b"null" in L.qfa_last_error()

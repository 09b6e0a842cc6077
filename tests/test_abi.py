"""The C-ABI library: loads without a GPU, exports every symbol include/qfa.h declares, and
rejects malformed calls with an error code and message before touching the device."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "qfa.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(qfa_[a-z_0-9]+)\s*\(", text)))


def test_header_symbols_are_exported(qfa):
    from quant_flash_attn_amd import _lib
    names = _declared_symbols()
    assert names == sorted(_lib._SIGNATURES), "python binding and include/qfa.h list different entry points"
    handle = ctypes.CDLL(_lib.library_path())
    for n in names:
        assert hasattr(handle, n), f"libqfa.so does not export {n}"
    assert _lib.lib().qfa_version() == 100


def test_argument_errors_need_no_gpu(qfa):
    from quant_flash_attn_amd import _lib
    L = _lib.lib()
    ok_ptr = 0x1000  # never dereferenced: validation fails first
    # null pointer
    rc = L.qfa_quant_per_token(None, 2, ok_ptr, ok_ptr, None, 0, ok_ptr, None, 1, 1, 8, 64, 512, 512, 64, 512, 512, 64, None)
    assert rc == -1 and b"null" in L.qfa_last_error()
    # bad dtype
    rc = L.qfa_quant_per_token(ok_ptr, 7, ok_ptr, ok_ptr, None, 0, ok_ptr, None, 1, 1, 8, 64, 512, 512, 64, 512, 512, 64, None)
    assert rc == -1 and b"x_dtype" in L.qfa_last_error()
    # unsupported head_dim
    rc = L.qfa_quant_per_token(ok_ptr, 2, ok_ptr, ok_ptr, None, 0, ok_ptr, None, 1, 1, 8, 44, 384, 384, 48, 384, 384, 48, None)
    assert rc == -2 and b"head_dim" in L.qfa_last_error()
    rc = L.qfa_quant_per_token(ok_ptr, 2, ok_ptr, ok_ptr, None, 0, ok_ptr, None, 1, 1, 8, 264, 4096, 4096, 264, 4096, 4096, 264, None)
    assert rc == -2 and b"head_dim" in L.qfa_last_error()
    # misaligned pointer, bad stride
    rc = L.qfa_quant_per_token(ok_ptr + 2, 2, ok_ptr, ok_ptr, None, 0, ok_ptr, None, 1, 1, 8, 64, 512, 512, 64, 512, 512, 64, None)
    assert rc == -1 and b"aligned" in L.qfa_last_error()
    rc = L.qfa_quant_per_token(ok_ptr, 2, ok_ptr, ok_ptr, None, 0, ok_ptr, None, 1, 1, 8, 64, 512, 512, 60, 512, 512, 64, None)
    assert rc == -1 and b"strides" in L.qfa_last_error()
    # attention: causal with Nq != Nk, bad sm_scale, bad head_dim
    def fwd(Nq=128, Nk=128, D=64, sm=0.125, causal=0, io=2):
        s = (Nq * D * 2, Nq * D, D)
        return L.qfa_attn_fwd(*([ok_ptr] * 11), io, 1, 2, Nq, Nk, D, *s, *s, *s, *s, sm, causal, None)
    assert fwd(Nq=192, Nk=128, causal=1) == -2 and b"causal" in L.qfa_last_error()   # more queries than keys
    assert fwd(sm=0.0) == -1 and b"sm_scale" in L.qfa_last_error()
    assert fwd(D=96) == -2 and b"head_dim" in L.qfa_last_error()
    assert fwd(io=0) == -1 and b"io_dtype" in L.qfa_last_error()
    # token strides of 2^23 elements or more: tile-relative offsets would not fit 31 bits
    big = (1 << 23)
    sb = (2 * 128 * big, 128 * big, big)
    s0 = (128 * 64 * 2, 128 * 64, 64)
    rc = L.qfa_attn_fwd(*([ok_ptr] * 11), 2, 1, 2, 128, 128, 64, *s0, *sb, *s0, *s0, 0.125, 0, None)
    assert rc == -2 and b"token strides" in L.qfa_last_error()
    # sequences beyond 2^28 tokens: byte offsets into the per-token vectors would not fit 31 bits
    long_n = (1 << 28) + 64
    sl = (long_n * 64, long_n * 64, 64)
    rc = L.qfa_attn_fwd(*([ok_ptr] * 11), 2, 1, 1, 128, long_n, 64, *s0, *sl, *sl, *s0, 0.125, 0, None)
    assert rc == -2 and b"2^28" in L.qfa_last_error()
    rc = L.qfa_bwd_delta(None, ok_ptr, ok_ptr, 2, 1, 1, 8, 64, 512, 512, 64, 512, 512, 64, None)
    assert rc == -1
    assert L.qfa_code_rowsum(None, ok_ptr, 1, 1, 8, 64, 512, 512, 64, None) == -1
    assert L.qfa_code_rowsum(ok_ptr, ok_ptr, 1, 1, 8, 44, 512, 512, 64, None) == -2 and b"head_dim" in L.qfa_last_error()
    assert L.qfa_code_rowsum(ok_ptr, ok_ptr, 1, 1, 8, 64, 512, 512, 60, None) == -1 and b"strides" in L.qfa_last_error()
    # backward scratch: one blob per 64-row tile (32-row at head_dim 256) and side; nothing for other widths
    ws = L.qfa_attn_bwd_workspace_bytes
    assert ws(1, 1, 64, 64, 64) == 2 * 64 * 64 * 2 + (5 + 3) * 64 * 4
    assert ws(2, 3, 65, 64, 128) == 6 * (3 * 128 * 64 * 2 + (2 * 5 + 3) * 64 * 4)
    assert ws(1, 1, 64, 32, 256) == 3 * 256 * 32 * 2 + (2 * 5 + 3) * 32 * 4
    assert ws(1, 1, 64, 64, 96) == 0 and ws(1, 1, 0, 64, 64) == 0
    # shared-KV entry points
    def skv_fwd(Nq=16, Nk=100, D=128, io=1, sdt=1, sm=0.1, q=ok_ptr):
        sq, sc = (Nq * D, Nq * D, D), (Nk * D, Nk * D, D)
        return L.qfa_attn_fwd_shared_kv(q, ok_ptr, ok_ptr, sdt, ok_ptr, ok_ptr, ok_ptr, io, 1, 1, Nq, Nk, D,
                                        *sq, *sc, *sq, sm, None, 0, None)
    assert skv_fwd(q=None) == -1 and b"null" in L.qfa_last_error()
    assert skv_fwd(D=96) == -2 and b"head_dim" in L.qfa_last_error()
    assert skv_fwd(io=0) == -1 and b"io_dtype" in L.qfa_last_error()
    assert skv_fwd(io=1, sdt=2) == -1 and b"scale_dtype" in L.qfa_last_error()
    assert skv_fwd(sm=float("nan")) == -1 and b"sm_scale" in L.qfa_last_error()
    def skv_bwd(Nq=16, Nk=100, D=128, io=1, dkv=ok_ptr, gd=1):
        sq, sc = (Nq * D, Nq * D, D), (Nk * D, Nk * D, D)
        return L.qfa_attn_bwd_shared_kv(ok_ptr, ok_ptr, ok_ptr, 0, ok_ptr, ok_ptr, ok_ptr, ok_ptr, ok_ptr, dkv, io,
                                        gd, None, 1, 1, Nq, Nk, D, *sq, *sc, *sq, *sq, *sq, *sc, 0.1, None)
    assert skv_bwd(D=96) == -2 and b"head_dim" in L.qfa_last_error()
    assert skv_bwd(io=2) == -2 and b"QFA_F16" in L.qfa_last_error()
    assert skv_bwd(dkv=None) == -1 and b"null" in L.qfa_last_error()
    assert skv_bwd(gd=0) == -1 and b"grad_dtype" in L.qfa_last_error()
    # queries and keys in one launch: the same checks per tensor
    def pair(x1=ok_ptr, dt=2, N1=8, D=64, sx1=(512, 512, 64)):
        return L.qfa_quant_per_token_pair(ok_ptr, x1, dt, *([ok_ptr] * 8), 1, 1, 8, N1, D, 512, 512, 64, *sx1,
                                          512, 512, 64, 512, 512, 64, None)
    assert pair(x1=None) == -1 and b"null" in L.qfa_last_error()
    assert pair(dt=9) == -1 and b"x_dtype" in L.qfa_last_error()
    assert pair(N1=0) == -1 and b"positive" in L.qfa_last_error()
    assert pair(D=44) == -2 and b"head_dim" in L.qfa_last_error()
    assert pair(x1=ok_ptr + 2) == -1 and b"aligned" in L.qfa_last_error()
    assert pair(sx1=(512, 512, 60)) == -1 and b"strides" in L.qfa_last_error()
    # the two small passes around the backward kernels
    assert L.qfa_sum_grads(ok_ptr, None, ok_ptr, 2, 64, None) == -1 and b"null" in L.qfa_last_error()
    assert L.qfa_sum_grads(ok_ptr, ok_ptr, ok_ptr, 0, 64, None) == -1 and b"dtype" in L.qfa_last_error()
    assert L.qfa_sum_grads(ok_ptr, ok_ptr, ok_ptr, 2, 12, None) == -1 and b"multiple of 8" in L.qfa_last_error()
    assert L.qfa_sum_grads(ok_ptr, ok_ptr + 2, ok_ptr, 2, 64, None) == -1 and b"aligned" in L.qfa_last_error()
    assert L.qfa_dout_normalise_workspace_bytes() > 0
    def norm(dout=ok_ptr, dt=1, n=64, sdt=0, ns=5, ws=ok_ptr):
        return L.qfa_dout_normalise(dout, dt, n, ok_ptr, sdt, ns, ws, ok_ptr, ok_ptr, None)
    assert norm(ws=None) == -1 and b"null" in L.qfa_last_error()
    assert norm(dt=0) == -1 and b"dout_dtype" in L.qfa_last_error()
    assert norm(sdt=2) == -1 and b"scale_dtype" in L.qfa_last_error()
    assert norm(n=20) == -1 and b"multiple of 8" in L.qfa_last_error()
    assert norm(ns=0) == -1 and b"n_scale" in L.qfa_last_error()
    assert norm(dout=ok_ptr + 4) == -1 and b"aligned" in L.qfa_last_error()
    assert L.qfa_dout_normalise(ok_ptr, 1, 64, ok_ptr + 2, 1, 5, ok_ptr, ok_ptr, ok_ptr, None) == -1 and b"aligned" in L.qfa_last_error()


def test_cpu_tensors_are_refused_not_emulated(qfa):
    x = torch.randn(1, 2, 16, 64)
    with pytest.raises(RuntimeError, match="GPU only"):
        qfa.asymmetric_quant_per_token(x)
    with pytest.raises(RuntimeError, match="GPU only"):
        qfa.quant_flash_attn_qkv(x, x, x, False, 0.125)
    with pytest.raises(ValueError):
        qfa.asymmetric_quant_per_token(torch.randn(16, 64))
    codes = torch.zeros(1, 2, 16, 64, dtype=torch.int8)
    quant = (codes, torch.ones(1, 2, 16, 1, dtype=torch.float16), torch.zeros(1, 2, 16, 1, dtype=torch.int8))
    with pytest.raises(RuntimeError, match="GPU only"):
        qfa.quant_flash_attn(x, x, quant, 0.125)
    with pytest.raises(RuntimeError, match="GPU only"):
        qfa.quant_flash_attn_quantized_kv(x, x, x, quant, quant, True, 0.125)


def test_routing_of_the_reference_entry_point():
    """quant_flash_attn gives query blocks up to the measured crossover to the shared-KV kernels: 512 tokens,
    1024 at head_dim 256 (where the INT8-score kernels run one wave per SIMD)."""
    from quant_flash_attn_amd.quant_flash_attn import SHARED_KV_MAX_Q, shared_kv_max_q
    assert SHARED_KV_MAX_Q == 512
    assert shared_kv_max_q(64) == 512 and shared_kv_max_q(128) == 512 and shared_kv_max_q(256) == 1024


def test_missing_library_fails_loudly(monkeypatch):
    from quant_flash_attn_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setenv("QFA_LIB", "/nonexistent/libqfa.so")
    with pytest.raises(RuntimeError, match="not found"):
        _lib.lib()


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "quant_flash_attn_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f
                assert "libqfa_oracle" not in text, f

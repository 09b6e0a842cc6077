"""ctypes binding of libqfa.so (the C ABI declared in include/qfa.h).

The library is loaded from the package directory (or from $QFA_LIB).  There is no
fallback: if it is missing, or a call returns non-zero, a RuntimeError is raised.
"""
from __future__ import annotations

import ctypes
import os
import threading
from ctypes import c_float, c_int, c_int64, c_void_p

import torch

QFA_F32, QFA_F16, QFA_BF16 = 0, 1, 2
DTYPE_CODE = {torch.float32: QFA_F32, torch.float16: QFA_F16, torch.bfloat16: QFA_BF16}

_HERE = os.path.dirname(os.path.abspath(__file__))
_lock = threading.Lock()
_lib = None

# argument lists mirror include/qfa.h one to one
_P, _I, _L, _F = c_void_p, c_int, c_int64, c_float
_SIGNATURES = {
    "qfa_version": (c_int, []),
    "qfa_last_error": (ctypes.c_char_p, []),
    "qfa_quant_per_token": (c_int, [_P, _I, _P, _P, _P, _I, _P, _P, _L, _L, _L, _I] + [_L] * 6 + [_P]),
    "qfa_quant_per_token_pair": (c_int, [_P, _P, _I] + [_P] * 8 + [_L, _L, _L, _L, _I] + [_L] * 12 + [_P]),
    "qfa_dequant_per_token": (c_int, [_P, _P, _I, _P, _P, _I, _L, _L, _L, _I] + [_L] * 6 + [_P]),
    "qfa_code_rowsum": (c_int, [_P, _P, _L, _L, _L, _I, _L, _L, _L, _P]),
    "qfa_attn_fwd": (c_int, [_P] * 11 + [_I, _L, _L, _L, _L, _I] + [_L] * 12 + [_F, _I, _P]),
    "qfa_attn_fwd_shared_kv_workspace_bytes": (c_int64, [_L, _L, _L, _L, _I]),
    "qfa_attn_fwd_shared_kv": (c_int, [_P, _P, _P, _I, _P, _P, _P, _I, _L, _L, _L, _L, _I] + [_L] * 9 + [_F, _P, _L, _P]),
    "qfa_attn_fwd_shared_kv_static": (c_int, [_P, _P, _P, _I, _P, _P, _P, _I, _L, _L, _L, _L, _I] + [_L] * 9 + [_F, _P]),
    "qfa_attn_bwd_shared_kv": (c_int, [_P, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _P, _L, _L, _L, _L, _I] + [_L] * 18
                               + [_F, _P]),
    "qfa_bench_qk_stage": (c_int, [_P] * 11 + [_I, _L, _L, _L, _L, _I] + [_L] * 12 + [_F, _I, _P]),
    "qfa_sum_grads": (c_int, [_P, _P, _P, _I, _L, _P]),
    "qfa_dout_normalise_workspace_bytes": (c_int64, []),
    "qfa_dout_normalise": (c_int, [_P, _I, _L, _P, _I, _L, _P, _P, _P, _P]),
    "qfa_bwd_delta": (c_int, [_P, _P, _P, _I, _L, _L, _L, _I] + [_L] * 6 + [_P]),
    "qfa_attn_bwd_workspace_bytes": (c_int64, [_L, _L, _L, _L, _I]),
    "qfa_attn_bwd": (c_int, [_P] * 13 + [_L] + [_P] * 3 + [_I, _L, _L, _L, _L, _I] + [_L] * 24 + [_F, _I, _P]),
}


def library_path() -> str:
    return os.environ.get("QFA_LIB") or os.path.join(_HERE, "libqfa.so")


def lib():
    """The loaded library.  Raises if libqfa.so has not been built."""
    global _lib
    if _lib is None:
        with _lock:
            if _lib is None:
                path = library_path()
                if not os.path.exists(path):
                    raise RuntimeError(
                        f"quant_flash_attn_amd: {path} not found. Build it with "
                        "`python -m quant_flash_attn_amd.build` (needs hipcc; there is no fallback path).")
                handle = ctypes.CDLL(path)
                for name, (res, args) in _SIGNATURES.items():
                    fn = getattr(handle, name)
                    fn.restype, fn.argtypes = res, args
                _lib = handle
    return _lib


def check(code: int, what: str) -> None:
    if code != 0:
        msg = lib().qfa_last_error().decode("utf-8", "replace")
        raise RuntimeError(f"{what} failed (code {code}): {msg}")


def stream_of(t: torch.Tensor) -> int:
    """Raw hipStream_t of torch's current stream on the tensor's device."""
    return torch.cuda.current_stream(t.device).cuda_stream


def require_gpu(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if not t.is_cuda:
            raise RuntimeError("quant_flash_attn_amd runs on the GPU only: got a tensor on "
                               f"'{t.device}'. There is no CPU implementation in this package.")
    dev = tensors[0].device
    for t in tensors[1:]:
        if t.device != dev:
            raise RuntimeError(f"all tensors must be on the same device, got {dev} and {t.device}")

"""quant_flash_attn_amd -- INT8 per-token quantized flash attention on AMD MI355X (gfx950).

Same Python entry points as yisunlp/quant_flash_attn, backed by hand-written HIP kernels in
libqfa.so (C ABI in include/qfa.h):

    asymmetric_quant_per_token(x)                      -> (codes, scale, zero_point)
    quant_flash_attn(q, kv_fp16, kv_quant, sm_scale)   -> o      (reference entry point)
    quant_flash_attn_qkv(q, k, v, causal, sm_scale)    -> o      (q/k/v entry point, causal flag)
    quant_flash_attn_quantized_kv(q, k_fp16, v_fp16, k_quant, v_quant, causal, sm_scale) -> o
                                                                 (K and V as two INT8 tensors, as a KV cache holds them)

GPU only: a CPU tensor or a missing libqfa.so raises; there is no fallback implementation.
"""
from .asymmetric_quant import (QuantizedTokens, asymmetric_quant_per_token, code_rowsum, dequantize_per_token,
                               quantize_for_attention, quantize_pair_for_attention)
from .quant_flash_attn import (QuantFlashAttention, QuantFlashAttnQKV, attn_bwd_quantized, attn_fwd_quantized,
                               attn_bwd_shared_kv, attn_fwd_shared_kv,
                               QuantFlashAttnQuantizedKV, quant_flash_attn, quant_flash_attn_qkv,
                               quant_flash_attn_quantized_kv)

__all__ = [
    "QuantizedTokens", "asymmetric_quant_per_token", "code_rowsum", "dequantize_per_token", "quantize_for_attention",
    "quantize_pair_for_attention",
    "QuantFlashAttention", "QuantFlashAttnQKV", "QuantFlashAttnQuantizedKV", "quant_flash_attn", "quant_flash_attn_qkv",
    "quant_flash_attn_quantized_kv",
    "attn_fwd_quantized", "attn_bwd_quantized", "attn_fwd_shared_kv", "attn_bwd_shared_kv",
]
__version__ = "0.1.0"

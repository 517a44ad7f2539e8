"""NVFP4-path operators with the names of the reference's ac4k_kernel.ops
(python/ac4k_kernel/ops/__init__.py:5-26), plus the attention forwards that consume the quantizers (NVFP4, and int8 x
fp8; head dims up to 128); the RoPE and sparse-attention operators of the reference are not part of this library."""
from .attention import attention, mha_int8_x_fp8_fwd, mha_nvfp4_fwd
from .linear import fused_linear, linear, linear_nvfp4, linear_prepacked, prepack_weight
from .quant import quantize, quantize_fp8, quantize_int8, quantize_nvfp4

__all__ = [
    "quantize", "linear", "fused_linear", "prepack_weight", "linear_prepacked",
    "quantize_nvfp4", "quantize_fp8", "quantize_int8", "linear_nvfp4", "attention", "mha_nvfp4_fwd", "mha_int8_x_fp8_fwd",
]

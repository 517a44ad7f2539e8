"""`ac4k_kernel.ops`: the NVFP4-path operators under the reference's module path
(python/ac4k_kernel/ops/__init__.py:5-26), re-exported from `ac4k_kernel_amd.ops`."""
import sys as _sys

from ac4k_kernel_amd.ops import (attention, fused_linear, linear, linear_nvfp4, mha_int8_x_fp8_fwd, mha_nvfp4_fwd, quantize, quantize_fp8,
                                 quantize_int8, quantize_nvfp4)

# submodule paths of the reference: ac4k_kernel.ops.quant / ac4k_kernel.ops.linear (taken from
# sys.modules: as attributes of the package, `linear` is the function, not the module)
for _name in ("quant", "linear", "utils", "attention"):
    _sys.modules[__name__ + "." + _name] = _sys.modules["ac4k_kernel_amd.ops." + _name]

__all__ = ["quantize", "linear", "fused_linear", "quantize_nvfp4", "quantize_fp8", "quantize_int8", "linear_nvfp4",
           "attention", "mha_nvfp4_fwd", "mha_int8_x_fp8_fwd"]

"""Import-name alias: `import ac4k_kernel` resolves to the MI355X library in `ac4k_kernel_amd`.

Callers written against the reference package (`from ac4k_kernel.ops import quantize`,
test/test_quantize_bench.py:7; `from ac4k_kernel.ops import linear, quantize`,
test/test_linear_bench.py:4; `from ac4k_kernel.ops import attention`, test/test_attention_bench.py:4)
keep their import lines.  Only the NVFP4 path exists here: the meta API of
python/ac4k_kernel/__init__.py:58-74, the quantize / linear operators of
python/ac4k_kernel/ops/__init__.py:5-26 and `attention` (both precisions, head dims up to 128).  The RoPE and
sparse-attention names of the reference are absent, and asking for them raises AttributeError / ImportError.
"""
import sys as _sys

import ac4k_kernel_amd as _impl
from ac4k_kernel_amd import (__version__, _rocm_ops, get_arch, get_backend, get_info, linear_nvfp4, quantize_fp8,
                             quantize_int8, quantize_nvfp4)

from . import ops

# `ac4k_kernel._rocm_ops` is the binding module name the reference package imports (:39-48)
_sys.modules[__name__ + "._rocm_ops"] = _rocm_ops

__all__ = list(_impl.__all__)

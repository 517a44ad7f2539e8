"""ac4k_kernel_amd — the NVFP4 quantize + linear path of ac4k_kernel on MI355X (gfx950).

Same meta API as the reference package (python/ac4k_kernel/__init__.py:58-74):
get_backend() == "rocm", get_arch() == "gfx950".  Importing the package loads the HIP
library; it raises if the library cannot be loaded.
"""
from ._rocm_ops import (__arch__, __backend__, linear_nvfp4, quantize_fp8, quantize_int8, quantize_nvfp4)
from . import ops

__version__ = "0.1.0"

_backend = __backend__
_arch = __arch__


def get_backend() -> str:
    """Compiled backend: 'rocm'."""
    return _backend


def get_arch() -> str:
    """Compiled architecture: 'gfx950'."""
    return _arch


def get_info() -> dict:
    return {"version": __version__, "backend": _backend, "arch": _arch}


__all__ = ["__version__", "get_backend", "get_arch", "get_info", "ops",
           "quantize_nvfp4", "quantize_fp8", "quantize_int8", "linear_nvfp4"]

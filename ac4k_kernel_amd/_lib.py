"""ctypes loader of libac4k_nvfp4.so, the C-ABI library declared in include/ac4k_nvfp4.h.

There is no fallback: if the library is missing it is built with hipcc once, and if that
fails (or a symbol is missing) the import raises.  Nothing here computes on the CPU.
"""
from __future__ import annotations

import ctypes
import os

from . import build as _build

_i64, _f32, _int, _vp, _cp = ctypes.c_int64, ctypes.c_float, ctypes.c_int, ctypes.c_void_p, ctypes.c_char_p

# name -> (restype, argtypes); must list every function of include/ac4k_nvfp4.h
SIGNATURES = {
    "ac4k_arch": (_cp, []),
    "ac4k_arch_description": (_cp, []),
    "ac4k_backend": (_cp, []),
    "ac4k_version": (_cp, []),
    "ac4k_last_error": (_cp, []),
    "ac4k_global_scale_bf16": (_int, [_vp, _vp, _i64, _f32, _vp]),
    "ac4k_set_quantize_sync_timeout_us": (None, [_i64]),
    "ac4k_debug_last_quantize_path": (_int, []),
    "ac4k_debug_quantize_timeouts_seen": (_i64, []),
    "ac4k_quantize_nvfp4": (_int, [_vp, _vp, _vp, _vp] + [_i64] * 8 + [_int, _vp]),
    "ac4k_quantize_nvfp4_bf16": (_int, [_vp, _vp, _vp, _vp] + [_i64] * 8 + [_int, _f32, _vp]),
    "ac4k_quantize_fp8": (_int, [_vp, _vp, _vp, _vp] + [_i64] * 8 + [_int, _vp]),
    "ac4k_quantize_int8": (_int, [_vp, _vp, _vp, _vp] + [_i64] * 8 + [_vp]),
    "ac4k_linear_nvfp4": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64, _vp]),
    "ac4k_linear_nvfp4_skinny_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "ac4k_linear_nvfp4_skinny": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64,
                                        _vp, _i64, _vp]),
    "ac4k_linear_nvfp4_skinny_static": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64,
                                               _vp]),
    "ac4k_set_linear_tuning": (_int, [_int, _int, _int, _int, _int]),
    "ac4k_prepack_weight_nvfp4_bytes": (_i64, [_i64, _i64]),
    "ac4k_prepack_weight_nvfp4": (_int, [_vp, _vp, _vp, _i64, _i64, _vp]),
    "ac4k_linear_nvfp4_prepacked_workspace_bytes": (_i64, [_i64, _i64, _i64]),
    "ac4k_linear_nvfp4_prepacked": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _int, _i64, _i64, _i64,
                                           _vp, _i64, _vp]),
    "ac4k_linear_nvfp4_fused_bf16": (_int, [_vp, _int, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _int,
                                            _i64, _i64, _i64, _vp, _i64, _vp]),
    "ac4k_mha_nvfp4_fwd": (_int, [_vp] + [_i64] * 4 + [_vp] * 9 + [_i64] * 6 + [_f32, _vp]),
    "ac4k_mha_int8_x_fp8_fwd": (_int, [_vp] + [_i64] * 4 + [_vp, _vp, _int, _vp, _vp, _int, _vp, _vp] + [_i64] * 6 + [_f32, _vp]),
    "ac4k_quantize_int8_token_block_bf16": (_int, [_vp, _vp, _vp] + [_i64] * 7 + [_int, _vp]),
}

_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        path = os.environ.get("AC4K_NVFP4_LIB")  # a prebuilt library elsewhere (kernel experiments)
        if not path:
            path = _build.LIB_PATH
            if not os.path.exists(path):
                _build.build()
        lib = ctypes.CDLL(path)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc: int) -> None:
    """Non-zero status of a C-ABI call -> RuntimeError, like the reference's TORCH_CHECK."""
    if rc != 0:
        raise RuntimeError(load().ac4k_last_error().decode())

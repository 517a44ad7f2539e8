"""ctypes front-end of oracle/nvfp4_oracle.c (test infrastructure only).

Takes and returns CPU torch tensors so tests can compare the C restatement,
the torch restatement and the HIP kernels on identical inputs.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "_build", "libnvfp4_oracle.so")
_lib = None

_i64, _f32, _i32, _vp = ctypes.c_int64, ctypes.c_float, ctypes.c_int32, ctypes.c_void_p


def build(force: bool = False) -> str:
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE] + (["-B"] if force else []))
    return _SO


def lib():
    global _lib
    if _lib is None:
        L = ctypes.CDLL(build())
        L.oracle_f32_to_e4m3.restype = ctypes.c_uint8
        L.oracle_f32_to_e4m3.argtypes = [_f32]
        L.oracle_e4m3_to_f32.restype = _f32
        L.oracle_e4m3_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_f32_to_e2m1.restype = ctypes.c_uint8
        L.oracle_f32_to_e2m1.argtypes = [_f32]
        L.oracle_e2m1_to_f32.restype = _f32
        L.oracle_e2m1_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_f32_to_s8.restype = ctypes.c_int8
        L.oracle_f32_to_s8.argtypes = [_f32]
        L.oracle_global_scale_bf16.restype = _f32
        L.oracle_global_scale_bf16.argtypes = [_vp, _i64, _f32]
        L.oracle_quantize_nvfp4.restype = None
        L.oracle_quantize_nvfp4.argtypes = [_vp, _vp, _vp, _f32] + [_i64] * 8 + [ctypes.c_int]
        L.oracle_quantize_fp8.restype = None
        L.oracle_quantize_fp8.argtypes = [_vp, _vp, _vp, _f32] + [_i64] * 8 + [ctypes.c_int]
        L.oracle_quantize_int8.restype = None
        L.oracle_quantize_int8.argtypes = [_vp, _vp, _vp, _i32] + [_i64] * 8
        L.oracle_linear_nvfp4.restype = None
        L.oracle_linear_nvfp4.argtypes = [_vp, _vp, _vp, _f32, _vp, _vp, _f32, _vp, _i64, _i64, _i64]
        _lib = L
    return _lib


def _align_up(a, b):
    return (a + b - 1) // b * b


def _geometry(x: torch.Tensor, cross_dim: int, reduce_dim: int):
    """4-D view parameters the kernels take: (d0, d1, R, K, s0, s1, sR, sK, lead_shape)."""
    nd = x.ndim
    cross_dim %= nd
    reduce_dim %= nd
    assert cross_dim != reduce_dim
    shape, stride = list(x.shape), list(x.stride())
    lead = [i for i in range(nd) if i not in (cross_dim, reduce_dim)]
    lead_shape = [shape[i] for i in lead]
    ld = [(shape[i], stride[i]) for i in lead]
    while len(ld) < 2:
        ld.insert(0, (1, 0))
    (d0, s0), (d1, s1) = ld
    return d0, d1, shape[cross_dim], shape[reduce_dim], s0, s1, stride[cross_dim], stride[reduce_dim], lead_shape


def global_scale(x: torch.Tensor, max_scale: float = 2688.0) -> torch.Tensor:
    x = x.contiguous()
    v = lib().oracle_global_scale_bf16(x.data_ptr(), x.numel(), max_scale)
    return torch.tensor(v, dtype=torch.float32)


def quantize_nvfp4(x, cross_dim, reduce_dim, swizzle=False, gs=None, max_scale=2688.0):
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    if gs is None:
        gs = global_scale(x, max_scale)
    d0, d1, R, K, s0, s1, sR, sK, lead = _geometry(x, cross_dim, reduce_dim)
    Kp, Rp = _align_up(K, 64), _align_up(R, 16)
    out = torch.full(lead + [R, Kp // 2], 0xCD, dtype=torch.uint8)
    sf = torch.full(lead + [Kp // 64, Rp, 4], 0xCD, dtype=torch.uint8)
    lib().oracle_quantize_nvfp4(out.data_ptr(), sf.data_ptr(), x.data_ptr(), float(gs), d0, d1, R, K,
                                s0, s1, sR, sK, int(swizzle))
    return out, sf, gs


def quantize_fp8(x, cross_dim, reduce_dim, max_scale=448.0, swizzle=False):
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    d0, d1, R, K, s0, s1, sR, sK, lead = _geometry(x, cross_dim, reduce_dim)
    Kp, Rp = _align_up(K, 16), _align_up(R, 16)
    out = torch.full(lead + [R, Kp], 0xCD, dtype=torch.uint8)
    sf = torch.full(lead + [Rp], -1.0, dtype=torch.float32)
    lib().oracle_quantize_fp8(out.data_ptr(), sf.data_ptr(), x.data_ptr(), float(max_scale), d0, d1, R, K,
                              s0, s1, sR, sK, int(swizzle))
    return out, sf


def quantize_int8(x, cross_dim, reduce_dim, max_scale=127):
    assert x.dtype == torch.bfloat16 and x.is_contiguous()
    d0, d1, R, K, s0, s1, sR, sK, lead = _geometry(x, cross_dim, reduce_dim)
    Kp, Rp = _align_up(K, 16), _align_up(R, 16)
    out = torch.full(lead + [R, Kp], -77, dtype=torch.int8)
    sf = torch.full(lead + [Rp], -1.0, dtype=torch.float32)
    lib().oracle_quantize_int8(out.data_ptr(), sf.data_ptr(), x.data_ptr(), int(max_scale), d0, d1, R, K,
                               s0, s1, sR, sK)
    return out, sf


def linear_nvfp4(a, a_sf, a_gs, b, b_sf, b_gs, bias=None) -> torch.Tensor:
    """fp32 [M,N]; the caller rounds to the output dtype."""
    a, b = a.contiguous(), b.contiguous()
    a_sf = a_sf.contiguous().view(torch.uint8)
    b_sf = b_sf.contiguous().view(torch.uint8)
    M, N, K = a.shape[0], b.shape[0], a.shape[1] * 2
    d = torch.empty((M, N), dtype=torch.float32)
    bias_f = None if bias is None else bias.reshape(-1).to(torch.float32).contiguous()
    lib().oracle_linear_nvfp4(d.data_ptr(), a.data_ptr(), a_sf.data_ptr(), float(a_gs), b.data_ptr(),
                              b_sf.data_ptr(), float(b_gs), None if bias_f is None else bias_f.data_ptr(),
                              M, N, K)
    return d

"""`linear` with the reference's signature (python/ac4k_kernel/ops/linear.py:15-75) on the
gfx950 NVFP4 GEMM, plus `fused_linear`, the decode-sized quantize+linear composition."""
from __future__ import annotations

import torch

from .. import _rocm_ops
from .utils import align_up

linear_nvfp4 = _rocm_ops.linear_nvfp4
prepack_weight = _rocm_ops.prepack_weight_nvfp4


class Ac4kLinearOp(torch.nn.Module):

    def forward(self, x, x_scale, x_global_scale, weight, weight_scale, weight_global_scale, bias, out=None):
        if (bias is not None) and (bias.ndim == 1):
            bias = bias.reshape(1, -1)
        if out is None:
            m, n = x.shape[0], weight.shape[0]
            out = torch.empty((m, n), dtype=torch.bfloat16, device=x.device)
        linear_nvfp4(out, x, x_scale, x_global_scale, weight, weight_scale, weight_global_scale, bias)
        return out


def linear(x, x_scale, x_global_scale, weight, weight_scale, weight_global_scale, bias=None, out=None):
    """y = x @ weight.T + bias on NVFP4 operands.

    x [M, K/2] and weight [N, K/2] are packed e2m1 (uint8), *_scale the e4m3 block scales in the
    [K/64, align_up(rows,16), 4] layout, *_global_scale 0-dim fp32.  bias is [N] or [1, N] in
    bf16/fp16/fp32; out defaults to a new bf16 [M, N] and may be bf16, fp16 or fp32.
    """
    return _LINEAR_OP.forward(x, x_scale, x_global_scale, weight, weight_scale, weight_global_scale, bias, out=out)


# one stateless module instance serves every call of the functional form
_LINEAR_OP = Ac4kLinearOp()


def fused_linear(x, weight, weight_scale, weight_global_scale, bias=None, out=None, return_quantized=False):
    """Decode-sized linear on a bf16 activation x [M, K], 1 <= M <= 32, K % 64 == 0:
    equals linear(*quantize(x, 0, 1), weight, weight_scale, weight_global_scale, bias, out)."""
    m, k = x.shape
    n = weight.shape[0]
    dev = x.device
    if (bias is not None) and (bias.ndim == 1):
        bias = bias.reshape(1, -1)
    if out is None:
        out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    x_q = torch.empty((m, k // 2), dtype=torch.uint8, device=dev)
    x_sf = torch.empty((k // 64, align_up(m, 16), 4), dtype=torch.float8_e4m3fn, device=dev)
    x_gs = torch.empty((), dtype=torch.float32, device=dev)
    _rocm_ops.linear_nvfp4_fused(out, x, x_q, x_sf, x_gs, weight, weight_scale, weight_global_scale, bias)
    if return_quantized:
        return out, (x_q, x_sf, x_gs)
    return out


def linear_prepacked(x, x_scale, x_global_scale, weight_image, weight_global_scale, bias=None, out=None, n=None):
    """`linear` on a weight image from `prepack_weight(weight, weight_scale)`: same result as
    linear(x, x_scale, x_global_scale, weight, weight_scale, weight_global_scale, bias, out).  The image
    does not carry N: pass `out` or `n`."""
    if (bias is not None) and (bias.ndim == 1):
        bias = bias.reshape(1, -1)
    if out is None:
        if n is None:
            if bias is None:
                raise RuntimeError("linear_prepacked needs out, n or bias to know N")
            n = bias.shape[-1]
        out = torch.empty((x.shape[0], n), dtype=torch.bfloat16, device=x.device)
    _rocm_ops.linear_nvfp4_prepacked(out, x, x_scale, x_global_scale, weight_image, weight_global_scale, bias)
    return out

"""`quantize` with the reference's signature, shapes and return tuples
(python/ac4k_kernel/ops/quant.py:68-294), running on the gfx950 HIP kernels.

The global-scale reduction that the reference does in Triton (quant.py:21-59) is a HIP
kernel behind the same C ABI.
"""
from __future__ import annotations

import torch

from .. import _rocm_ops
from .utils import align_up

quantize_nvfp4 = _rocm_ops.quantize_nvfp4
quantize_fp8 = _rocm_ops.quantize_fp8
quantize_int8 = _rocm_ops.quantize_int8


def _global_scale(x: torch.Tensor, max_scale: float) -> torch.Tensor:
    out = torch.empty((), dtype=torch.float32, device=x.device)
    _rocm_ops.global_scale(out, x, max_scale)
    return out


_SCALE_MAX_CACHE = {}


def _scale_max_tensor(value, dtype, device):
    """0-dim device scalar for scale_max.  The reference builds one with torch.full on every call
    (quant.py:130-135,177-182); here it is kept per (value, dtype, device).  The fill runs on the stream of
    the first call; until it has completed, calls order their own stream behind it with an event (no host
    synchronisation anywhere).  While the current stream records into a graph nothing is cached: a tensor
    made there lives in the graph's memory pool and is only filled when the graph replays."""
    key = (value, dtype, device)
    hit = _SCALE_MAX_CACHE.get(key)
    if hit is not None:
        t, ev = hit
        if ev is not None:
            if ev.query():
                _SCALE_MAX_CACHE[key] = (t, None)  # filled: nothing to order against any more
            elif not torch.cuda.is_current_stream_capturing():
                torch.cuda.current_stream(device).wait_event(ev)
            else:  # a capture must not depend on work outside it: a scalar of the graph's own
                return torch.full([], value, dtype=dtype, device=device)
        return t
    t = torch.full([], value, dtype=dtype, device=device)
    if device.type != "cuda":
        _SCALE_MAX_CACHE[key] = (t, None)
    elif not torch.cuda.is_current_stream_capturing():
        ev = torch.cuda.Event()
        ev.record(torch.cuda.current_stream(device))
        _SCALE_MAX_CACHE[key] = (t, ev)
    return t


def _lead_shape(shape, cross_dim, reduce_dim):
    return [shape[i] for i in range(len(shape)) if i != cross_dim and i != reduce_dim]


class Ac4kQuantizeOp(torch.nn.Module):

    def forward(self, input: torch.Tensor, cross_dim, reduce_dim, max_scale=None, precision="nvfp4",
                swizzle=False, output=None, sf=None):
        assert input.ndim >= 2 and input.ndim <= 4, "input tensor must be 2D, 3D or 4D"
        assert precision in ["nvfp4", "fp8e4m3", "int8"]
        if cross_dim < 0:
            cross_dim += input.ndim
        if reduce_dim < 0:
            reduce_dim += input.ndim
        assert cross_dim != reduce_dim, "cross_dim and reduce_dim must be different"

        shape = input.shape
        lead = _lead_shape(shape, cross_dim, reduce_dim)
        R, K = shape[cross_dim], shape[reduce_dim]
        dev = input.device

        if precision in ("fp8e4m3", "int8"):
            fp8 = precision == "fp8e4m3"
            out_dtype = torch.float8_e4m3fn if fp8 else torch.int8
            # out [.., cross, align_up(reduce, 16)], sf [.., align_up(cross, 16)] fp32
            if output is None:
                output = torch.empty(lead + [R, align_up(K, 16)], dtype=out_dtype, device=dev)
            if sf is None:
                sf = torch.empty(lead + [align_up(R, 16)], dtype=torch.float32, device=dev)
            if max_scale is None:
                max_scale = 448 if fp8 else 127
            if fp8:
                smax = _scale_max_tensor(float(max_scale), torch.float32, dev)
                quantize_fp8(output, sf, input, smax, cross_dim, reduce_dim, swizzle)
            else:
                smax = _scale_max_tensor(int(max_scale), torch.int32, dev)
                quantize_int8(output, sf, input, smax, cross_dim, reduce_dim)
            return output, sf

        if max_scale is None:
            max_scale = 448.0 * 6.0  # FLOAT8_E4M3_MAX * FLOAT4_E2M1_MAX
        # out [.., cross, align_up(reduce, 64) / 2] u8, sf [.., align_up(reduce, 64) / 64, align_up(cross, 16), 4]
        Kp = align_up(K, 64)
        if output is None:
            output = torch.empty(lead + [R, Kp // 2], dtype=torch.uint8, device=dev)
        if sf is None:
            sf = torch.empty(lead + [Kp // 64, align_up(R, 16), 4], dtype=torch.float8_e4m3fn, device=dev)
        global_scale = torch.empty((), dtype=torch.float32, device=dev)
        _rocm_ops.quantize_nvfp4_with_global_scale(output, sf, global_scale, input, cross_dim, reduce_dim, swizzle,
                                                   float(max_scale))
        return output, sf, global_scale


def quantize(input, cross_dim, reduce_dim, max_scale=None, precision="nvfp4", swizzle=False, output=None,
             sf=None):
    """Quantize a bf16 tensor to nvfp4, fp8e4m3 or int8.

    cross_dim is the M/N (parallel) dim, reduce_dim the K dim.  max_scale defaults to 6*448 for
    nvfp4, 448 for fp8e4m3, 127 for int8.  swizzle permutes the reduce dim as
    reshape(-1,4,4,2).permute(0,2,1,3) for nvfp4 and reshape(-1,2,4,2).permute(0,2,1,3) for fp8e4m3.

    Returns (output, sf, global_scale) for nvfp4 and (output, sf) otherwise:
      nvfp4   output [.., cross, align_up(reduce,64)/2] u8, sf [.., ceil(reduce/64), align_up(cross,16), 4] e4m3
      fp8e4m3 output [.., cross, align_up(reduce,16)] e4m3, sf [.., align_up(cross,16)] fp32
      int8    output [.., cross, align_up(reduce,16)] int8, sf [.., align_up(cross,16)] fp32
    where `..` are the remaining input dims in their original order.
    """
    return _QUANTIZE_OP.forward(input, cross_dim, reduce_dim, max_scale=max_scale, precision=precision,
                                swizzle=swizzle, output=output, sf=sf)


# one stateless module instance serves every call of the functional form
_QUANTIZE_OP = Ac4kQuantizeOp()

"""CPU oracle (torch, vectorised) for the NVFP4 path of ac4k_kernel.

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this
module: it is the checker that `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py` compare the HIP kernels against.

The spec restated here is the reference kernels' operation order evaluated in
IEEE-754 round-to-nearest fp32 (the reference's own `rcp.approx.ftz`,
`--use_fast_math` divisions and Triton `/` are hardware approximations that are
not reproducible off NVIDIA silicon):

  global scale   python/ac4k_kernel/ops/quant.py:33-59,195-200
  nvfp4 kernel   lib/cuda/sm120/quantize_nvfp4.cu:49-157 (arithmetic :73,113-147,
                 zero padding :94-109, scale address :57-60,150-155, swizzle :86-100)
  e2m1 / e4m3    lib/cuda/common/math.cuh:39-80 (cvt.rn.satfinite semantics,
                 first PTX source operand -> high nibble)
  fp8 kernel     lib/cuda/sm120/quantize_fp8.cu:57-185
  int8 kernel    lib/cuda/sm120/quantize_int8.cu:55-168
  shapes         python/ac4k_kernel/ops/quant.py:93-242
  linear         lib/cuda/sm120/linear_nvfp4.cu:586-633,753-805 and
                 lib/cuda/sm120/mma.cuh:13-56 (block-scale semantics);
                 dequantize + fp32 matmul as in test/test_linear_bench.py:7-107

This restatement follows the *test-side* formulation (permute -> pad ->
optional swizzle -> per-block arithmetic, test/test_quantize_bench.py:18-109);
`oracle/nvfp4_oracle.c` follows the *kernel-side* strided indexing.  The two
are written independently and `tests/test_oracle_*.py` checks one against the
other, against closed forms and against the reference's known-answer sets.

Parity pinning status (see tests/test_oracle_*.py):
  global_scale, quantize_nvfp4, e2m1/e4m3 rounding, layouts, swizzle,
  quantize_fp8, dequantize, linear: pinned.
  quantize_int8: the reference holds no test for it; pinned by source reading,
  by brute force over all bf16 inputs against round-half-even + clamp, and by
  the C restatement — "parity unpinned" against reference-held vectors.
  NaN/Inf inputs and all-zero tensors/rows: follow the IEEE evaluation of the
  kernel order; the reference has no test for them — "parity unpinned".
"""
from __future__ import annotations

import torch

E2M1_VALUES = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]
# value of each 4-bit code, sign in bit 3 (test/test_linear_bench.py:18-35)
E2M1_LUT = torch.tensor(E2M1_VALUES + [-v for v in E2M1_VALUES], dtype=torch.float32)

ONE_SIXTH_F32 = torch.tensor(0.16666666666666666, dtype=torch.float32)  # quantize_nvfp4.cu:126


def ceil_div(a: int, b: int) -> int:
    return (a + b - 1) // b


def align_up(a: int, b: int) -> int:
    return ceil_div(a, b) * b


# --------------------------------------------------------------------------
# scalar formats
# --------------------------------------------------------------------------

def f32_to_e4m3_bits(x: torch.Tensor) -> torch.Tensor:
    """cvt.rn.satfinite.e4m3.f32: RNE, |x| >= 448 (incl. inf) -> +-448, NaN -> 0x7F."""
    assert x.dtype == torch.float32
    nan = torch.isnan(x)
    y = torch.clamp(x, min=-448.0, max=448.0)
    y = torch.where(nan, torch.zeros_like(y), y)
    bits = y.to(torch.float8_e4m3fn).view(torch.uint8)
    return torch.where(nan, torch.full_like(bits, 0x7F), bits)


def e4m3_bits_to_f32(b: torch.Tensor) -> torch.Tensor:
    assert b.dtype == torch.uint8
    return b.view(torch.float8_e4m3fn).to(torch.float32)


def f32_to_e2m1_bits(x: torch.Tensor) -> torch.Tensor:
    """cvt.rn.satfinite.e2m1.f32 on one value: RNE on {0,.5,1,1.5,2,3,4,6},
    ties to the even code, saturate to 6, sign bit kept (also for zero),
    NaN -> 0x7 (positive max)."""
    assert x.dtype == torch.float32
    a = x.abs()
    code = ((a > 0.25).to(torch.uint8) + (a >= 0.75).to(torch.uint8) +
            (a > 1.25).to(torch.uint8) + (a >= 1.75).to(torch.uint8) +
            (a > 2.5).to(torch.uint8) + (a >= 3.5).to(torch.uint8) +
            (a > 5.0).to(torch.uint8))
    sign = (x.view(torch.int32) < 0).to(torch.uint8) << 3
    out = code | sign
    return torch.where(torch.isnan(x), torch.full_like(out, 0x7), out)


def f32_to_s8_sat(x: torch.Tensor) -> torch.Tensor:
    """cvt.rni.sat.s8.f32: round half to even, clamp to [-128,127], NaN -> 0."""
    r = torch.round(x)
    r = torch.where(torch.isnan(r), torch.zeros_like(r), r)
    return torch.clamp(r, -128.0, 127.0).to(torch.int8)


# --------------------------------------------------------------------------
# layout helpers
# --------------------------------------------------------------------------

def _norm_dims(ndim, cross_dim, reduce_dim):
    assert 2 <= ndim <= 4, "input tensor must be 2D, 3D or 4D"
    if cross_dim < 0:
        cross_dim += ndim
    if reduce_dim < 0:
        reduce_dim += ndim
    assert cross_dim != reduce_dim, "cross_dim and reduce_dim must be different"
    return cross_dim, reduce_dim


def _to_rows(x: torch.Tensor, cross_dim: int, reduce_dim: int):
    """-> ([B, R, K] contiguous view of x with the other dims flattened in
    original order, list of the other dims' sizes)."""
    lead = [i for i in range(x.ndim) if i not in (cross_dim, reduce_dim)]
    lead_shape = [x.shape[i] for i in lead]
    xr = x.permute(*lead, cross_dim, reduce_dim).contiguous()
    return xr.reshape(-1, x.shape[cross_dim], x.shape[reduce_dim]), lead_shape


def _pad_last(x: torch.Tensor, to: int) -> torch.Tensor:
    if x.shape[-1] == to:
        return x
    return torch.nn.functional.pad(x, [0, to - x.shape[-1]], value=0.0)


# --------------------------------------------------------------------------
# a1  global scale
# --------------------------------------------------------------------------

def global_scale(x: torch.Tensor, max_scale: float = 448.0 * 6.0) -> torch.Tensor:
    """gs = fp32(max|x|) / fp32(max_scale)   (quant.py:33-59,195-200)."""
    assert x.dtype == torch.bfloat16
    amax = x.abs().max().to(torch.float32) if x.numel() else torch.zeros((), dtype=torch.float32)
    return amax / torch.tensor(float(max_scale), dtype=torch.float32)


# --------------------------------------------------------------------------
# a2-a6  nvfp4 quantize
# --------------------------------------------------------------------------

def quantize_nvfp4(x: torch.Tensor, cross_dim: int, reduce_dim: int, swizzle: bool = False,
                   max_scale: float | None = None, gs: torch.Tensor | None = None):
    """-> (out uint8 [.., R, Kp/2], sf uint8(e4m3 bits) [.., Kp/64, Rp, 4], gs fp32 0-dim)."""
    assert x.dtype == torch.bfloat16
    cross_dim, reduce_dim = _norm_dims(x.ndim, cross_dim, reduce_dim)
    if gs is None:
        gs = global_scale(x, 2688.0 if max_scale is None else max_scale)
    gs = gs.to(torch.float32).reshape(())
    xr, lead_shape = _to_rows(x, cross_dim, reduce_dim)
    B, R, K = xr.shape
    Kp, Rp = align_up(K, 64), align_up(R, 16)
    xf = _pad_last(xr.to(torch.float32), Kp)                       # zero padding :94-109
    if swizzle:                                                    # :86-100
        xf = xf.reshape(B, R, Kp // 32, 4, 4, 2).permute(0, 1, 2, 4, 3, 5).reshape(B, R, Kp)
    blk = xf.reshape(B, R, Kp // 16, 16)
    one = torch.ones((), dtype=torch.float32)
    alpha = one / gs                                               # :73
    m = blk.abs().amax(dim=-1)                                     # :113-123
    s32 = alpha * (m * ONE_SIXTH_F32)                              # :126
    sf_bits = f32_to_e4m3_bits(s32)                                # :127-131
    s = e4m3_bits_to_f32(sf_bits)
    o = torch.where(s != 0, alpha * (one / s), torch.zeros_like(s))  # :133-134
    q = f32_to_e2m1_bits(blk * o.unsqueeze(-1)).reshape(B, R, Kp // 2, 2)  # :136-144
    out = (q[..., 0] | (q[..., 1] << 4)).to(torch.uint8)           # even element -> low nibble
    sf = torch.zeros((B, Kp // 64, Rp, 4), dtype=torch.uint8)      # pad rows are written as 0 (:83,150-155)
    sf[:, :, :R, :] = sf_bits.reshape(B, R, Kp // 64, 4).permute(0, 2, 1, 3)
    return (out.reshape(lead_shape + [R, Kp // 2]),
            sf.reshape(lead_shape + [Kp // 64, Rp, 4]), gs)


def e2m1_unpack(packed: torch.Tensor) -> torch.Tensor:
    """uint8 [.., n] -> fp32 [.., 2n]; low nibble first (test_linear_bench.py:15-50)."""
    assert packed.dtype == torch.uint8
    lo = E2M1_LUT[(packed & 0xF).long()]
    hi = E2M1_LUT[(packed >> 4).long()]
    return torch.stack((lo, hi), dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def sf_to_linear(sf: torch.Tensor, rows: int) -> torch.Tensor:
    """[Kp/64, Rp, 4] e4m3 bits -> fp32 [rows, Kp/16] (test_linear_bench.py:7-12)."""
    assert sf.ndim == 3 and sf.shape[2] == 4
    if sf.dtype != torch.uint8:
        sf = sf.view(torch.uint8)
    return e4m3_bits_to_f32(sf.permute(1, 0, 2).reshape(sf.shape[1], -1)[:rows].contiguous())


def dequantize_nvfp4(packed: torch.Tensor, sf: torch.Tensor, gs, dtype=torch.float32) -> torch.Tensor:
    """2-D packed [R, Kp/2] -> [R, Kp]:  e2m1 * (sf * gs)  (test_linear_bench.py:53-67,
    whose caller passes 1/gs because the helper divides, :140-150)."""
    R = packed.shape[0]
    v = e2m1_unpack(packed).to(dtype).reshape(R, -1, 16)
    s = sf_to_linear(sf, R).to(dtype) * torch.as_tensor(gs).to(dtype)
    return (v * s.unsqueeze(-1)).reshape(R, -1)


# --------------------------------------------------------------------------
# a7 / a8  per-row fp8 and int8 quantize
# --------------------------------------------------------------------------

def _rowwise_prepare(x, cross_dim, reduce_dim):
    cross_dim, reduce_dim = _norm_dims(x.ndim, cross_dim, reduce_dim)
    xr, lead_shape = _to_rows(x, cross_dim, reduce_dim)
    B, R, K = xr.shape
    Kp, Rp = align_up(K, 16), align_up(R, 16)
    xf = _pad_last(xr.to(torch.float32), Kp)
    amax = xf.abs().amax(dim=-1) if K else torch.zeros((B, R))
    return xf, amax, lead_shape, B, R, K, Kp, Rp


def quantize_fp8(x: torch.Tensor, cross_dim: int, reduce_dim: int, max_scale: float | None = None,
                 swizzle: bool = False):
    """-> (out uint8(e4m3 bits) [.., R, align_up(K,16)], sf fp32 [.., Rp])
    (quantize_fp8.cu:91-182; swizzle :141-151)."""
    assert x.dtype == torch.bfloat16
    smax = torch.tensor(448.0 if max_scale is None else float(max_scale), dtype=torch.float32)
    xf, amax, lead_shape, B, R, K, Kp, Rp = _rowwise_prepare(x, cross_dim, reduce_dim)
    if swizzle:
        xf = xf.reshape(B, R, Kp // 16, 2, 4, 2).permute(0, 1, 2, 4, 3, 5).reshape(B, R, Kp)
    sf = torch.zeros((B, Rp), dtype=torch.float32)
    sf[:, :R] = amax / smax                                        # :124-128
    recp = smax / amax                                             # :132 (amax == 0 -> +inf)
    out = f32_to_e4m3_bits(xf * recp.unsqueeze(-1))                # :168-182 (0*inf = NaN -> 0x7F)
    return out.reshape(lead_shape + [R, Kp]), sf.reshape(lead_shape + [Rp])


def quantize_int8(x: torch.Tensor, cross_dim: int, reduce_dim: int, max_scale: int | None = None):
    """-> (out int8 [.., R, align_up(K,16)], sf fp32 [.., Rp])  (quantize_int8.cu:55-165)."""
    assert x.dtype == torch.bfloat16
    smax = torch.tensor(float(127 if max_scale is None else int(max_scale)), dtype=torch.float32)
    xf, amax, lead_shape, B, R, K, Kp, Rp = _rowwise_prepare(x, cross_dim, reduce_dim)
    sf = torch.zeros((B, Rp), dtype=torch.float32)
    sf[:, :R] = amax / smax                                        # :127
    recp = smax / amax                                             # :135
    out = f32_to_s8_sat(xf * recp.unsqueeze(-1))                   # :55-59,161-165
    return out.reshape(lead_shape + [R, Kp]), sf.reshape(lead_shape + [Rp])


# --------------------------------------------------------------------------
# a9-a11  linear
# --------------------------------------------------------------------------

def linear_nvfp4(a, a_sf, a_gs, b, b_sf, b_gs, bias=None, out_dtype=torch.bfloat16,
                 acc_dtype=torch.float32) -> torch.Tensor:
    """fp32 dequantize-then-matmul, the accuracy gate of test/test_linear_bench.py:70-107:
    D = cvt(dequant(A) @ dequant(B).T + bias)."""
    da = dequantize_nvfp4(a, a_sf, a_gs, acc_dtype)
    db = dequantize_nvfp4(b, b_sf, b_gs, acc_dtype)
    d = da @ db.t()
    if bias is not None:
        d = d + bias.reshape(1, -1).to(acc_dtype)
    return d.to(out_dtype)


def linear_nvfp4_contract(a, a_sf, a_gs, b, b_sf, b_gs, bias=None, out_dtype=torch.bfloat16):
    """The kernel's own math contract in fp64 (linear_nvfp4.cu:586-633):
    D = cvt( fp32( sum_j sfA sfB sum_i a b ) * fp32(gsA*gsB) + bias ).  The inner sum is
    exact in fp64 for every K the tests use, so this isolates accumulation-order error."""
    one = torch.ones((), dtype=torch.float64)
    da = dequantize_nvfp4(a, a_sf, one, torch.float64)
    db = dequantize_nvfp4(b, b_sf, one, torch.float64)
    acc = (da @ db.t()).to(torch.float32)
    scale = torch.as_tensor(a_gs).to(torch.float32) * torch.as_tensor(b_gs).to(torch.float32)
    d = acc * scale
    if bias is not None:
        d = d + bias.reshape(1, -1).to(torch.float32)
    return d.to(out_dtype)

"""Tensor-level binding over the C ABI: the module the reference's package would import as
`ac4k_kernel._rocm_ops` (python/ac4k_kernel/__init__.py:39-48), with the function names and
positional arguments of `_cuda_ops` (lib/cuda_bindings.cc:64-85, include/ac4k_kernel/ops.h:27-48).

All functions write into caller-provided tensors, return None, enqueue on the current
torch stream and never synchronise.  Argument checks mirror the reference host launchers'
TORCH_CHECKs and raise RuntimeError.
"""
from __future__ import annotations

import torch

from . import _lib

_L = _lib.load()

__arch__ = _L.ac4k_arch().decode()
__arch_description__ = _L.ac4k_arch_description().decode()
__backend__ = _L.ac4k_backend().decode()
__version__ = _L.ac4k_version().decode()

_DTYPE_TAG = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def _check(cond: bool, msg: str, *args) -> None:
    """RuntimeError(msg.format(*args)) unless cond; the message is only built on failure."""
    if not cond:
        raise RuntimeError(msg.format(*args) if args else msg)


def _check_tensor(t, dtype, name: str, suffix: str = "") -> None:
    # one combined test on the hot path; the individual messages are only built on failure
    if isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == dtype and t.is_contiguous():
        return
    name += suffix
    _check(isinstance(t, torch.Tensor), "{} must be a tensor", name)
    _check(t.is_cuda, "{} must be a CUDA tensor", name)
    _check(t.is_contiguous(), "{} must be contiguous", name)
    _check(t.dtype == dtype, "Inconsistency of Tensor type: {} must be {}", name, dtype)


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """hipStream_t of torch's current stream on the current device."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _align_up(a: int, b: int) -> int:
    return (a + b - 1) // b * b


def _quant_geometry(inp: torch.Tensor, cross_dim: int, reduce_dim: int):
    """Checks shared by the three quantizers (quantize_nvfp4.cu:171-190,226-241)."""
    _check_tensor(inp, torch.bfloat16, "in")
    _check(2 <= inp.dim() <= 4, "in must be 2-4D")
    _check(0 <= cross_dim < inp.dim(), "cross_dim must be less than in.dim()")
    _check(0 <= reduce_dim < inp.dim(), "reduce_dim must be less than in.dim()")
    _check(cross_dim != reduce_dim, "cross_dim and reduce_dim must be different")
    shape, stride = list(inp.shape), list(inp.stride())
    lead = [i for i in range(inp.dim()) if i not in (cross_dim, reduce_dim)]
    lead_shape = [shape[i] for i in lead]
    ld = [(shape[i], stride[i]) for i in lead]
    while len(ld) < 2:
        ld.insert(0, (1, 0))
    (d0, s0), (d1, s1) = ld
    _check(inp.numel() > 0, "in must not be empty")
    return lead_shape, (d0, d1, shape[cross_dim], shape[reduce_dim], s0, s1, stride[cross_dim], stride[reduce_dim])


def global_scale(out: torch.Tensor, inp: torch.Tensor, max_scale: float) -> None:
    """out (0-dim fp32) = amax(|inp|) / max_scale  (python/ac4k_kernel/ops/quant.py:33-59)."""
    _check_tensor(inp, torch.bfloat16, "in")
    _check_tensor(out, torch.float32, "global_scale")
    _check(out.dim() == 0, "global_scale must be a scalar")
    _lib.check(_L.ac4k_global_scale_bf16(out.data_ptr(), inp.data_ptr(), inp.numel(), float(max_scale), _stream()))


def quantize_nvfp4(out, sf, inp, global_scale, cross_dim: int, reduce_dim: int, swizzle: bool) -> None:
    lead_shape, geom = _quant_geometry(inp, cross_dim, reduce_dim)
    R, K = geom[2], geom[3]
    _check_tensor(global_scale, torch.float32, "global_scale")
    _check(global_scale.dim() == 0, "global_scale must be a scalar")
    _check_tensor(out, torch.uint8, "out")
    _check(list(out.shape) == lead_shape + [R, _align_up(K, 64) // 2],
           "out must have shape [.., cross, align_up(reduce, 64) / 2]")
    _check_tensor(sf, torch.float8_e4m3fn, "sf")
    _check(list(sf.shape) == lead_shape + [_align_up(K, 64) // 64, _align_up(R, 16), 4], "meet invalid sf shape")
    _lib.check(_L.ac4k_quantize_nvfp4(out.data_ptr(), sf.data_ptr(), inp.data_ptr(), global_scale.data_ptr(),
                                      *geom, int(bool(swizzle)), _stream()))


def quantize_nvfp4_with_global_scale(out, sf, global_scale, inp, cross_dim: int, reduce_dim: int, swizzle: bool,
                                     max_scale: float) -> None:
    """global_scale (written) = amax(|inp|) / max_scale, then quantize_nvfp4 with it: the nvfp4 branch
    of the reference's Ac4kQuantizeOp.forward (quant.py:187-242) behind one C call."""
    lead_shape, geom = _quant_geometry(inp, cross_dim, reduce_dim)
    R, K = geom[2], geom[3]
    _check_tensor(global_scale, torch.float32, "global_scale")
    _check(global_scale.dim() == 0, "global_scale must be a scalar")
    _check_tensor(out, torch.uint8, "out")
    _check(list(out.shape) == lead_shape + [R, _align_up(K, 64) // 2],
           "out must have shape [.., cross, align_up(reduce, 64) / 2]")
    _check_tensor(sf, torch.float8_e4m3fn, "sf")
    _check(list(sf.shape) == lead_shape + [_align_up(K, 64) // 64, _align_up(R, 16), 4], "meet invalid sf shape")
    _lib.check(_L.ac4k_quantize_nvfp4_bf16(out.data_ptr(), sf.data_ptr(), global_scale.data_ptr(), inp.data_ptr(),
                                           *geom, int(bool(swizzle)), float(max_scale), _stream()))


def _quantize_rowwise(fn, out, out_dtype, sf, inp, scale_max, scale_dtype, cross_dim, reduce_dim, *extra):
    lead_shape, geom = _quant_geometry(inp, cross_dim, reduce_dim)
    R, K = geom[2], geom[3]
    _check_tensor(scale_max, scale_dtype, "scale_max")
    _check(scale_max.dim() == 0, "scale_max must be a scalar")
    _check_tensor(out, out_dtype, "out")
    _check(list(out.shape) == lead_shape + [R, _align_up(K, 16)], "out must have shape [.., cross, align_up(reduce, 16)]")
    _check_tensor(sf, torch.float32, "sf")
    _check(list(sf.shape) == lead_shape + [_align_up(R, 16)], "meet invalid sf shape")
    _lib.check(fn(out.data_ptr(), sf.data_ptr(), inp.data_ptr(), scale_max.data_ptr(), *geom, *extra, _stream()))


def quantize_fp8(out, sf, inp, scale_max, cross_dim: int, reduce_dim: int, swizzle: bool) -> None:
    _quantize_rowwise(_L.ac4k_quantize_fp8, out, torch.float8_e4m3fn, sf, inp, scale_max, torch.float32,
                      cross_dim, reduce_dim, int(bool(swizzle)))


def quantize_int8(out, sf, inp, scale_max, cross_dim: int, reduce_dim: int) -> None:
    _quantize_rowwise(_L.ac4k_quantize_int8, out, torch.int8, sf, inp, scale_max, torch.int32,
                      cross_dim, reduce_dim)


def _check_linear_operand(x, x_sf, x_gs, rows, name):
    _check(x.dim() == 2, "{} must be a 2d matrix", name)
    _check_tensor(x, torch.uint8, name)
    K = x.size(1) * 2
    _check(x_sf.dim() == 3, "scale_{} must be a 3d matrix", name)
    _check_tensor(x_sf, torch.float8_e4m3fn, "scale_", name)
    _check(x_sf.shape == ((K + 63) // 64, _align_up(rows, 16), 4), "scale_{} has an invalid shape", name)
    _check_tensor(x_gs, torch.float32, "global_scale_", name)
    _check(x_gs.dim() == 0, "{}_global_scale must be a scalar", name)
    return K


def _skinny_scratch(device, M, N, K):
    """Workspace tensor for the shapes that split K, or None when the shape needs no scratch."""
    nbytes = _L.ac4k_linear_nvfp4_skinny_workspace_bytes(M, N, K)
    if nbytes <= 0:
        return None
    return torch.empty((nbytes,), dtype=torch.uint8, device=device)


def _bias_args(bias, N):
    if bias is None:
        return None, 0
    _check(bias.dtype in _DTYPE_TAG, "bias must be bfloat16, half or float")
    _check(bias.is_cuda and bias.is_contiguous(), "bias must be contiguous")
    _check(bias.dim() == 2, "bias must be a 2d matrix")
    _check(bias.size(0) == 1, "bias shape[0] must be 1")
    _check(bias.size(1) == N, "bias shape[1] must be {}", N)
    return bias.data_ptr(), _DTYPE_TAG[bias.dtype]


def linear_nvfp4(D, A, A_sf, A_global_scale, B, B_sf, B_global_scale, bias=None) -> None:
    """Checks of linear_nvfp4.cu:759-805.  Shapes for which the library asks for scratch (too few output
    tiles for the GPU, long K) get a workspace tensor and the split-K kernels; everything else goes to
    the reference-shaped entry point, which allocates nothing and picks its kernel by shape."""
    _check(isinstance(D, torch.Tensor) and D.dim() == 2, "d must be a 2d matrix")
    _check(D.dtype in _DTYPE_TAG, "d must be bfloat16, half or float")
    _check(D.is_cuda and D.is_contiguous(), "d must be contiguous")
    M, N = D.shape
    _check(A.dim() == 2 and A.size(0) == M, "A size(0) must be {}", M)
    K = _check_linear_operand(A, A_sf, A_global_scale, M, "a")
    _check(K % 16 == 0, "A size(1)*2 must be multiple of 16 but see {}", K)
    _check(B.dim() == 2 and B.size(1) == A.size(1), "B size(1) must equal A size(1)")
    _check(B.size(0) == N, "B size(0) must be {}", N)
    _check_linear_operand(B, B_sf, B_global_scale, N, "b")
    bias_ptr, bias_tag = _bias_args(bias, N)
    if M == 0 or N == 0:
        return
    scratch = _skinny_scratch(D.device, M, N, K)
    if scratch is not None:
        ws = scratch
        _lib.check(_L.ac4k_linear_nvfp4_skinny(D.data_ptr(), _DTYPE_TAG[D.dtype], A.data_ptr(), A_sf.data_ptr(),
                                               A_global_scale.data_ptr(), B.data_ptr(), B_sf.data_ptr(),
                                               B_global_scale.data_ptr(), bias_ptr, bias_tag, M, N, K,
                                               ws.data_ptr(), ws.numel(), _stream()))
        return
    _lib.check(_L.ac4k_linear_nvfp4(D.data_ptr(), _DTYPE_TAG[D.dtype], A.data_ptr(), A_sf.data_ptr(),
                                    A_global_scale.data_ptr(), B.data_ptr(), B_sf.data_ptr(),
                                    B_global_scale.data_ptr(), bias_ptr, bias_tag, M, N, K, _stream()))


def prepack_weight_nvfp4(B, B_sf) -> torch.Tensor:
    """Weight image of B [N, K/2] / B_sf [K/64, align_up(N,16), 4] for linear_nvfp4_prepacked: a uint8
    tensor of ac4k_prepack_weight_nvfp4_bytes(N, K) bytes.  K must be a multiple of 128."""
    _check(B.dim() == 2, "b must be a 2d matrix")
    _check_tensor(B, torch.uint8, "b")
    N, K = B.size(0), B.size(1) * 2
    _check(B_sf.dim() == 3, "scale_b must be a 3d matrix")
    _check_tensor(B_sf, torch.float8_e4m3fn, "scale_", "b")
    _check(B_sf.shape == ((K + 63) // 64, _align_up(N, 16), 4), "scale_b has an invalid shape")
    nbytes = _L.ac4k_prepack_weight_nvfp4_bytes(N, K)
    _check(nbytes > 0, "no weight image for N = {}, K = {}: K must be a multiple of 128", N, K)
    image = torch.empty((nbytes,), dtype=torch.uint8, device=B.device)
    _lib.check(_L.ac4k_prepack_weight_nvfp4(image.data_ptr(), B.data_ptr(), B_sf.data_ptr(), N, K, _stream()))
    return image


def linear_nvfp4_prepacked(D, A, A_sf, A_global_scale, W_image, B_global_scale, bias=None) -> None:
    """linear_nvfp4 on a weight image made by prepack_weight_nvfp4 (N = D.size(1), K = 2 * A.size(1))."""
    _check(isinstance(D, torch.Tensor) and D.dim() == 2, "d must be a 2d matrix")
    _check(D.dtype in _DTYPE_TAG, "d must be bfloat16, half or float")
    _check(D.is_cuda and D.is_contiguous(), "d must be contiguous")
    M, N = D.shape
    _check(A.dim() == 2 and A.size(0) == M, "A size(0) must be {}", M)
    K = _check_linear_operand(A, A_sf, A_global_scale, M, "a")
    _check_tensor(W_image, torch.uint8, "w_image")
    _check(N > 0 and W_image.numel() == _L.ac4k_prepack_weight_nvfp4_bytes(N, K) and W_image.numel() > 0,
           "w_image is not the weight image of a [{}, {}] weight", N, K)
    _check_tensor(B_global_scale, torch.float32, "global_scale_", "b")
    _check(B_global_scale.dim() == 0, "b_global_scale must be a scalar")
    bias_ptr, bias_tag = _bias_args(bias, N)
    if M == 0:
        return
    nbytes = _L.ac4k_linear_nvfp4_prepacked_workspace_bytes(M, N, K)
    ws = torch.empty((nbytes,), dtype=torch.uint8, device=D.device) if nbytes > 0 else None
    _lib.check(_L.ac4k_linear_nvfp4_prepacked(D.data_ptr(), _DTYPE_TAG[D.dtype], A.data_ptr(), A_sf.data_ptr(),
                                              A_global_scale.data_ptr(), W_image.data_ptr(),
                                              B_global_scale.data_ptr(), bias_ptr, bias_tag, M, N, K,
                                              None if ws is None else ws.data_ptr(), nbytes, _stream()))


def linear_nvfp4_fused(D, X, X_q, X_sf, X_global_scale, B, B_sf, B_global_scale, bias=None) -> None:
    """quantize(X, 0, 1) + linear_nvfp4 for a bf16 activation X [M, K], 1 <= M <= 32;
    X_q / X_sf / X_global_scale receive the quantized activation."""
    _check(isinstance(D, torch.Tensor) and D.dim() == 2, "d must be a 2d matrix")
    _check(D.dtype in _DTYPE_TAG, "d must be bfloat16, half or float")
    _check(D.is_cuda and D.is_contiguous(), "d must be contiguous")
    M, N = D.shape
    _check_tensor(X, torch.bfloat16, "x")
    _check(X.dim() == 2 and X.size(0) == M, "x must be [{}, K]", M)
    _check(1 <= M <= 32, "the fused linear takes 1 <= M <= 32")
    K = X.size(1)
    _check(K % 64 == 0, "K must be a multiple of 64")
    _check_tensor(X_q, torch.uint8, "x_q")
    _check(list(X_q.shape) == [M, K // 2], "x_q must be [M, K/2]")
    _check_linear_operand(X_q, X_sf, X_global_scale, M, "x")
    _check(B.dim() == 2 and B.size(0) == N and B.size(1) == K // 2, "weight must be [N, K/2]")
    _check_linear_operand(B, B_sf, B_global_scale, N, "b")
    bias_ptr, bias_tag = _bias_args(bias, N)
    if K % 256 != 0:  # no weight-streaming kernel: the composition itself
        quantize_nvfp4_with_global_scale(X_q, X_sf, X_global_scale, X, 0, 1, False, 2688.0)
        linear_nvfp4(D, X_q, X_sf, X_global_scale, B, B_sf, B_global_scale, bias)
        return
    ws = _skinny_scratch(D.device, M, N, K)  # None: one K range per tile, no scratch
    _lib.check(_L.ac4k_linear_nvfp4_fused_bf16(D.data_ptr(), _DTYPE_TAG[D.dtype], X.data_ptr(), X_q.data_ptr(),
                                               X_sf.data_ptr(), X_global_scale.data_ptr(), B.data_ptr(),
                                               B_sf.data_ptr(), B_global_scale.data_ptr(), bias_ptr, bias_tag,
                                               M, N, K, None if ws is None else ws.data_ptr(),
                                               0 if ws is None else ws.numel(), _stream()))


def _check_attention_operand(x, x_sf, x_gs, B, H, rows, width, name):
    """One packed operand of mha_nvfp4_fwd: x [B,H,rows,width/2], x_sf [B,H,ceil(width/64),align_up(rows,16),4]
    (mha_nvfp4.cu:917-1003)."""
    _check_tensor(x, torch.uint8, name)
    _check(x.dim() == 4 and list(x.shape) == [B, H, rows, width // 2], "{} must be [{}, {}, {}, {}]", name, B, H, rows, width // 2)
    _check_tensor(x_sf, torch.float8_e4m3fn, name + "_sf")
    _check(x_sf.dim() == 5, "{}_sf must be a 5D tensor", name)
    _check(list(x_sf.shape) == [B, H, (width + 63) // 64, _align_up(rows, 16), 4], "Meet invalid {}_sf size", name)
    _check_tensor(x_gs, torch.float32, name + "_global_scale")
    _check(x_gs.dim() == 0, "{}_global_scale must be a float tensor", name)


def mha_nvfp4_fwd(o, q, q_sf, q_global_scale, k, k_sf, k_global_scale, v, v_sf, v_global_scale, sm_scale: float) -> None:
    """Checks of mha_nvfp4.cu:917-1012.  o may be a permuted view (the reference's caller passes one): only its
    shape [B,H,Nq,Dv], dtype and device are checked."""
    _check(isinstance(q, torch.Tensor) and q.dim() == 4, "Q must be a 4D tensor")
    B, H, Nq = q.size(0), q.size(1), q.size(2)
    Dqk = q.size(3) * 2
    _check(Dqk % 16 == 0, "Dqk must be multiple of 16")
    _check(Dqk <= 128, "Dqk must be less than 128")
    _check(isinstance(k, torch.Tensor) and k.dim() == 4, "K must be a 4D tensor")
    _check(k.size(0) == B, "K must have the same batch size as Q")
    _check(k.size(1) == H, "K must have the same head number as Q")
    _check(k.size(3) == q.size(3), "K must have the same dim as Q")
    Nkv = k.size(2)
    _check(isinstance(v, torch.Tensor) and v.dim() == 4, "V must be a 4D tensor")
    Dv = v.size(2)
    _check(Dv <= 128, "Dv must be less than 128")
    _check(v.size(3) * 2 == _align_up(Nkv, 64), "V must have the same sequence length as K")
    _check_attention_operand(q, q_sf, q_global_scale, B, H, Nq, Dqk, "q")
    _check_attention_operand(k, k_sf, k_global_scale, B, H, Nkv, Dqk, "k")
    _check_attention_operand(v, v_sf, v_global_scale, B, H, Dv, _align_up(Nkv, 64), "v")
    _check(isinstance(o, torch.Tensor) and o.is_cuda, "O must be a CUDA tensor")
    _check(o.dtype == torch.bfloat16, "O must be a bfloat16 tensor")
    _check(o.dim() == 4 and list(o.shape) == [B, H, Nq, Dv], "O must be [{}, {}, {}, {}]", B, H, Nq, Dv)
    if B == 0 or H == 0 or Nq == 0:
        return
    _check(Nkv > 0, "K must not be empty")
    _lib.check(_L.ac4k_mha_nvfp4_fwd(o.data_ptr(), *o.stride(), q.data_ptr(), q_sf.data_ptr(), q_global_scale.data_ptr(),
                                     k.data_ptr(), k_sf.data_ptr(), k_global_scale.data_ptr(), v.data_ptr(), v_sf.data_ptr(),
                                     v_global_scale.data_ptr(), B, H, Nq, Nkv, Dqk, Dv, float(sm_scale), _stream()))


def mha_int8_x_fp8_fwd(o, q, q_sf, q_quantize_block_size: int, k, k_sf, k_quantize_block_size: int, v, v_sf,
                       sm_scale: float) -> None:
    """Checks of mha_int8_x_fp8.cu:982-1044.  o may be a permuted view: only its shape [B,H,Nq,Dv], dtype and
    device are checked."""
    _check_tensor(q, torch.int8, "Q")
    _check(q.dim() == 4, "Q must be a 4D tensor")
    B, H, Nq, Dqk = q.size(0), q.size(1), q.size(2), q.size(3)
    _check(Dqk % 16 == 0, "Dqk must be multiple of 16")
    _check(Dqk <= 128, "Dqk must be less than 128")
    _check_tensor(q_sf, torch.float32, "Q_SF")
    _check(q_sf.dim() == 3, "Q_SF must be a 3D tensor")
    _check(list(q_sf.shape) == [B, H, -(-Nq // q_quantize_block_size)], "Meet invalid Q_SF size")
    _check_tensor(k, torch.int8, "K")
    _check(k.dim() == 4, "K must be a 4D tensor")
    _check(k.size(0) == B, "K must have the same batch size as Q")
    _check(k.size(1) == H, "K must have the same head number as Q")
    _check(k.size(3) == Dqk, "K must have the same dim as Q")
    Nkv = k.size(2)
    _check_tensor(k_sf, torch.float32, "K_SF")
    _check(k_sf.dim() == 3, "K_SF must be a 3D tensor")
    _check(list(k_sf.shape) == [B, H, -(-Nkv // k_quantize_block_size)], "Meet invalid K_SF size")
    _check_tensor(v, torch.float8_e4m3fn, "V")
    _check(v.dim() == 4, "V must be a 4D tensor")
    _check(v.size(0) == B, "V must have the same batch size as Q")
    _check(v.size(1) == H, "V must have the same head number as Q")
    Dv = v.size(2)
    _check(v.size(3) == _align_up(Nkv, 16), "Meet invalid v size(3) with {}=={}", v.size(3), _align_up(Nkv, 16))
    _check(Dv <= 128, "Dv must be less than 128")
    _check_tensor(v_sf, torch.float32, "V_SF")
    _check(v_sf.dim() == 3 and list(v_sf.shape) == [B, H, _align_up(Dv, 16)], "Meet invalid v_sf size")
    _check(isinstance(o, torch.Tensor) and o.is_cuda, "O must be a CUDA tensor")
    _check(o.dtype == torch.bfloat16, "O must be a bfloat16 tensor")
    _check(o.dim() == 4 and list(o.shape) == [B, H, Nq, Dv], "O must be [{}, {}, {}, {}]", B, H, Nq, Dv)
    if B == 0 or H == 0 or Nq == 0:
        return
    _check(Nkv > 0, "K must not be empty")
    _lib.check(_L.ac4k_mha_int8_x_fp8_fwd(o.data_ptr(), *o.stride(), q.data_ptr(), q_sf.data_ptr(), int(q_quantize_block_size),
                                          k.data_ptr(), k_sf.data_ptr(), int(k_quantize_block_size), v.data_ptr(),
                                          v_sf.data_ptr(), B, H, Nq, Nkv, Dqk, Dv, float(sm_scale), _stream()))


def quantize_int8_token_block(y, scale, x_bhnd, block: int) -> None:
    """y int8 [B,H,N,align_up(D,16)], scale fp32 [B,H,ceil(N/block)] <- x bf16 viewed as [B,H,N,D] (any batch, head and
    token strides, head dim contiguous): the per-token-block quantizer of python/ac4k_kernel/ops/attention.py:18-99."""
    _check(isinstance(x_bhnd, torch.Tensor) and x_bhnd.is_cuda and x_bhnd.dtype == torch.bfloat16, "x must be a CUDA bfloat16 tensor")
    _check(x_bhnd.dim() == 4 and x_bhnd.stride(3) == 1, "x must be 4D with a contiguous head dim")
    B, H, N, D = x_bhnd.shape
    _check_tensor(y, torch.int8, "y")
    _check(list(y.shape) == [B, H, N, _align_up(D, 16)], "Meet invalid y size")
    _check_tensor(scale, torch.float32, "scale")
    _check(list(scale.shape) == [B, H, -(-N // block)], "Meet invalid scale size")
    if x_bhnd.numel() == 0:
        return
    _lib.check(_L.ac4k_quantize_int8_token_block_bf16(y.data_ptr(), scale.data_ptr(), x_bhnd.data_ptr(), B, H, N, D,
                                                      x_bhnd.stride(0), x_bhnd.stride(1), x_bhnd.stride(2), int(block), _stream()))

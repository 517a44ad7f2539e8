"""CPU oracle (torch, vectorised) for the attention forwards of ac4k_kernel: NVFP4, and INT8 (QK) x FP8 (PV).

TEST INFRASTRUCTURE ONLY.  Nothing in the shipped package may import this module.

The spec restated here is `mha_nvfp4_fwd` (include/ac4k_kernel/ops.h:12-16,
lib/cuda/sm120/mha_nvfp4.cu:911-1077 host checks, :336-905 kernel), evaluated in IEEE
round-to-nearest fp32 where the reference uses hardware approximations (`rcp.approx.ftz`,
`exp2f` under fast-math):

  operands     Q [B,H,Nq,D/2], K [B,H,Nkv,D/2] packed e2m1 with scales [B,H,D/64,rows^16,4];
               V [B,H,Dv,Nkv^64/2] quantized ALONG the kv dim with the swizzle of
               quantize(v, 3, N_dim, swizzle=True) (python/ac4k_kernel/ops/attention.py:114-116),
               scales [B,H,Nkv^64/64,Dv^16,4]                                   mha_nvfp4.cu:894-909
  S            (Qhat . Khat^T) accumulated in fp32, then * (q_gs * k_gs * sm_scale)       :586-598
  softmax      online over kv tiles of 128: m = max(m_old, rowmax(S_tile)),
               p = exp2(S*log2e - m*log2e), l = exp2((m_old - m) log2e) * l + sum(p)      :600-700
               kv positions past Nkv inside the last tile have S = 0 (zero-filled K): they
               enter the row maximum and p, and their p is taken out of l again as
               npad / exp2(m * log2e)                                                     :676-685
  P -> nvfp4   per 16-block, the blocks being the kv positions {8g + 4h + j} (g, j = 0..3) of
               a 32-group for h = 0, 1 - the sets that the swizzle of V turns into contiguous
               16-blocks; global scale fixed at 1/(448*6): sf = e4m3(2688 * (max * (1/6))),
               o = sf != 0 ? 2688 * (1/sf) : 0, q = e2m1(p * o)                           :248-319
  O            O = O * exp2((m_old - m) log2e) + Phat . Vhat^T (fp32), at the end
               O * ((1/l) * (1/2688) * v_gs) -> bf16                                      :705-830

Parity pinning status (tests/test_oracle_attention.py): the end-to-end result against an fp32
softmax(QK^T)V at the tolerance of the reference's own test (test/test_attention_bench.py:19-66,
nvfp4 cases :178-191: atol 0.2, rtol 0.1, cosine similarity > 0.98); the P block structure and its
scale recipe against closed-form cases in which a contiguous-block reading gives a different
answer; the V de-swizzle against quantize->dequantize round trips; the padding rules against a
direct evaluation on the unpadded problem.  The reference holds no stored vectors for this
operator, and the hardware roundings of exp2 / rcp on sm_120 are not observable here.

The second half of the file restates `mha_int8_x_fp8_fwd` (include/ac4k_kernel/ops.h:18-21,
lib/cuda/sm120/mha_int8_x_fp8.cu:979-1137 host, :346-975 kernel) and the Python side in front of it
(python/ac4k_kernel/ops/attention.py:18-99 per-token-block int8 quantize, :137-192 wrapper); its header
is further down.
"""
from __future__ import annotations

import math

import torch

from . import nvfp4_oracle as T

LOG2E = torch.tensor(1.4426950408889634, dtype=torch.float32)
P_ALPHA = torch.tensor(448.0 * 6.0, dtype=torch.float32)   # 1 / (global scale of P)
KV_TILE = 128


def _dequant_rows(packed: torch.Tensor, sf: torch.Tensor, rows: int) -> torch.Tensor:
    """[.., rows, Kp/2] + [.., Kp/64, rows^16, 4] -> fp32 [.., rows, Kp] = e2m1 * sf (no global scale)."""
    lead = packed.shape[:-2]
    p2 = packed.reshape(-1, packed.shape[-2], packed.shape[-1])
    s2 = sf.reshape(-1, *sf.shape[-3:])
    out = [T.dequantize_nvfp4(p2[i], s2[i], 1.0) for i in range(p2.shape[0])]
    return torch.stack(out).reshape(*lead, rows, -1)


def deswizzle_kv(x: torch.Tensor) -> torch.Tensor:
    """Last dim in the stored (swizzled) order of quantize(.., swizzle=True) -> original order.
    The swizzle swaps the two 4-dims of reshape(-1, 4, 4, 2) (quantize_nvfp4.cu:86-100), so it is
    its own inverse."""
    n = x.shape[-1]
    return x.reshape(*x.shape[:-1], n // 32, 4, 4, 2).transpose(-2, -3).reshape(*x.shape[:-1], n)


def quantize_p_tile(p: torch.Tensor):
    """p fp32 [.., 128] (one kv tile) -> (phat fp32 [.., 128] = e2m1 * sf without the 1/2688, sf bits
    [.., 8]) with the interleaved 16-blocks of mha_nvfp4.cu:248-319."""
    assert p.dtype == torch.float32 and p.shape[-1] % 32 == 0
    g32 = p.shape[-1] // 32
    # position inside a 32-group = 8 g + 4 h + j  -> dims (group, g, h, j); a block = fixed (group, h)
    blk = p.reshape(*p.shape[:-1], g32, 4, 2, 4).transpose(-2, -3)            # (.., group, h, g, j)
    m = blk.amax(dim=(-1, -2))
    sf_f = P_ALPHA * (m * T.ONE_SIXTH_F32)
    sf_bits = T.f32_to_e4m3_bits(sf_f)
    s = T.e4m3_bits_to_f32(sf_bits)
    one = torch.ones((), dtype=torch.float32)
    o = torch.where(s != 0, P_ALPHA * (one / s), torch.zeros_like(s))
    q = T.f32_to_e2m1_bits(blk * o[..., None, None])
    phat = T.E2M1_LUT[q.long()] * s[..., None, None]
    phat = phat.transpose(-2, -3).reshape(p.shape)
    return phat, sf_bits.reshape(*p.shape[:-1], g32 * 2)


def mha_nvfp4_fwd(q, q_sf, q_gs, k, k_sf, k_gs, v, v_sf, v_gs, sm_scale: float) -> torch.Tensor:
    """-> O bf16 [B, H, Nq, Dv]."""
    B, H, Nq, Dh = q.shape
    Dqk = Dh * 2
    Nkv = k.shape[2]
    Dv = v.shape[2]
    assert k.shape[3] == Dh and v.shape[3] * 2 == (Nkv + 63) // 64 * 64
    qf = _dequant_rows(q, q_sf, Nq)                      # [B,H,Nq,Dqk]
    kf = _dequant_rows(k, k_sf, Nkv)                     # [B,H,Nkv,Dqk]
    vf = deswizzle_kv(_dequant_rows(v, v_sf, Dv))        # [B,H,Dv,Nkv^64], original kv order
    nkp = (Nkv + KV_TILE - 1) // KV_TILE * KV_TILE
    kf = torch.nn.functional.pad(kf, (0, 0, 0, nkp - Nkv))            # zero-filled K rows: S = 0 there
    vf = torch.nn.functional.pad(vf, (0, nkp - vf.shape[-1]))         # zero V: no contribution
    f32 = lambda x: torch.as_tensor(x, dtype=torch.float32)           # noqa: E731
    qk_scale = f32(q_gs) * f32(k_gs) * f32(sm_scale)                  # :586
    m = torch.full((B, H, Nq), -math.inf, dtype=torch.float32)
    l = torch.zeros((B, H, Nq), dtype=torch.float32)
    o = torch.zeros((B, H, Nq, Dv), dtype=torch.float32)
    for n0 in range(0, nkp, KV_TILE):
        s = (qf @ kf[:, :, n0:n0 + KV_TILE].transpose(-1, -2)) * qk_scale
        m_new = torch.maximum(m, s.amax(dim=-1))
        p = torch.exp2(s * LOG2E - (m_new * LOG2E)[..., None])
        l_new = p.sum(dim=-1)
        if n0 + KV_TILE > Nkv:                                        # :676-685
            l_new = l_new - f32(nkp - Nkv) / torch.exp2(m_new * LOG2E)
        alpha = torch.exp2(m * LOG2E - m_new * LOG2E)                 # exp2(-inf) = 0 on the first tile
        l = alpha * l + l_new
        phat, _ = quantize_p_tile(p)
        o = o * alpha[..., None] + phat @ vf[:, :, :, n0:n0 + KV_TILE].transpose(-1, -2)
        m = m_new
    one = torch.ones((), dtype=torch.float32)
    scale = (one / l) * (one / P_ALPHA) * f32(v_gs)                   # :812-815
    return (o * scale[..., None]).to(torch.bfloat16)


def quantize_qkv(q, k, v, layout: str = "BNHD"):
    """The three quantize calls of _nvfp4_attention (python/ac4k_kernel/ops/attention.py:113-116) with the
    quantizer oracle: q, k, v bf16 [B,N,H,D] (BNHD) or [B,H,N,D] -> the nine operands of mha_nvfp4_fwd."""
    n_dim = 1 if layout == "BNHD" else 2
    return (*T.quantize_nvfp4(q, n_dim, 3), *T.quantize_nvfp4(k, n_dim, 3), *T.quantize_nvfp4(v, 3, n_dim, True))


def attention_nvfp4(q, k, v, layout: str = "BNHD") -> torch.Tensor:
    """attention(q, k, v, layout=layout, precision="nvfp4") of the reference, on the CPU."""
    ops = quantize_qkv(q, k, v, layout)
    o = mha_nvfp4_fwd(*ops, 1.0 / math.sqrt(q.shape[-1]))             # [B,H,N,Dv]
    return o.permute(0, 2, 1, 3).contiguous() if layout == "BNHD" else o


# --------------------------------------------------------------------------
# INT8 (QK) x FP8 (PV) attention
# --------------------------------------------------------------------------
# Spec restated (lib/cuda/sm120/mha_int8_x_fp8.cu):
#   operands   Q int8 [B,H,Nq,Dp], K int8 [B,H,Nkv,Dp] (Dp = head dim padded to 16, pad columns 0) with one fp32
#              scale per block of q_block (32 or 64) / k_block (128) tokens: [B,H,ceil(N/block)]; V e4m3
#              [B,H,Dv,Nkv^16] quantized per (head, d) row along kv with max_scale 2.25 and the 16-group swizzle
#              of quantize_fp8, scales fp32 [B,H,Dv^16]                                        :966-977,979-1040
#   S          int32 dot products (exact), s = float(S) * ((sm_scale * log2e) * q_sf * k_sf)       :476,657-677
#              kv positions past Nkv in the last tile are -inf                                      :679-700
#   softmax    online over kv tiles of 128 with the maximum held 7.5 below the row maximum:
#              m = max(rowmax(s) - 7.5, m_old); p = exp2(s - m) <= 2^7.5; l = l * exp2(m_old - m) + sum(p)
#                                                                                                   :702-776
#   P -> e4m3  cvt.rn.satfinite per element, no scales                                              :323-345
#   O          O = O * exp2(m_old - m) + Phat . Vhat^T per tile; at the end O * ((1/l) * v_sf[d]) -> bf16
#                                                                                                   :828-905
# The reference accumulates Phat . Vhat^T of a tile in fp16 (mma ... f16 accumulators, :858-866) before it adds
# the tile to the fp32 O; this oracle and the HIP kernel accumulate in fp32.  PARITY UNPINNED for that rounding
# and for the hardware exp2: the reference holds no vectors for this operator, its tests compare with fp32
# attention at atol 0.2 / rtol 1e-2 and cosine similarity > 0.99 (test/test_attention_bench.py:69-177), which
# tests/test_oracle_attention.py applies to this oracle.  The Triton quantizer's float -> int8 cast is taken as
# truncation toward zero (fptosi) and its division as IEEE.

EXP_OFFSET = torch.tensor(7.5, dtype=torch.float32)


def int8_block_token_quantize(x: torch.Tensor, layout: str, block: int):
    """_int8_quantize(x, layout, N_dim, BLOCK_SIZE=block) (python/ac4k_kernel/ops/attention.py:18-99):
    x bf16 [B,N,H,D] (BNHD) or [B,H,N,D] -> (y int8 [B,H,N,D^16], scale fp32 [B,H,ceil(N/block)]); one scale =
    max|x| / 127 per block of `block` tokens of a head, y = int8(trunc(x / scale)), 0 where the scale is 0."""
    assert x.dtype == torch.bfloat16 and layout in ("BNHD", "BHND")
    xf = (x.permute(0, 2, 1, 3) if layout == "BNHD" else x).float()
    B, H, N, D = xf.shape
    nb = (N + block - 1) // block
    xp = torch.nn.functional.pad(xf, (0, 0, 0, nb * block - N)).reshape(B, H, nb, block, D)
    scale = xp.abs().amax(dim=(-1, -2)) / torch.tensor(127.0, dtype=torch.float32)
    yq = torch.trunc(xp / scale[..., None, None])
    yq = torch.where(scale[..., None, None] == 0, torch.zeros_like(yq), yq)
    y = torch.zeros((B, H, N, (D + 15) // 16 * 16), dtype=torch.int8)
    y[..., :D] = yq.reshape(B, H, nb * block, D)[:, :, :N].to(torch.int8)
    return y, scale


def deswizzle_fp8(x: torch.Tensor) -> torch.Tensor:
    """Last dim in the stored order of quantize(.., precision="fp8e4m3", swizzle=True) -> original order: the
    swizzle swaps the 2- and 4-dims of reshape(-1, 2, 4, 2) (quantize_fp8.cu:141-151)."""
    n = x.shape[-1]
    return x.reshape(*x.shape[:-1], n // 16, 4, 2, 2).transpose(-2, -3).reshape(*x.shape[:-1], n)


def mha_int8_x_fp8_fwd(q, q_sf, q_block: int, k, k_sf, k_block: int, v, v_sf, sm_scale: float) -> torch.Tensor:
    """-> O bf16 [B, H, Nq, Dv].  q, k int8; v uint8 (e4m3 bits)."""
    B, H, Nq, Dp = q.shape
    Nkv, Dv = k.shape[2], v.shape[2]
    assert k.shape[3] == Dp and k_block == KV_TILE and q_block in (32, 64)
    assert v.shape[3] == (Nkv + 15) // 16 * 16 and v_sf.shape[2] == (Dv + 15) // 16 * 16
    qf, kf = q.float(), k.float()
    vf = deswizzle_fp8(T.e4m3_bits_to_f32(v))                     # [B,H,Dv,Nkv^16], original kv order
    nkp = (Nkv + KV_TILE - 1) // KV_TILE * KV_TILE
    kf = torch.nn.functional.pad(kf, (0, 0, 0, nkp - Nkv))
    vf = torch.nn.functional.pad(vf, (0, nkp - vf.shape[-1]))
    sm = torch.tensor(sm_scale, dtype=torch.float32) * LOG2E      # :476
    rows = torch.arange(Nq) // q_block
    qs = sm * q_sf[:, :, rows]                                    # [B,H,Nq]
    m = torch.full((B, H, Nq), -math.inf, dtype=torch.float32)
    l = torch.zeros((B, H, Nq), dtype=torch.float32)
    o = torch.zeros((B, H, Nq, Dv), dtype=torch.float32)
    pos = torch.arange(KV_TILE)
    for n0 in range(0, nkp, KV_TILE):
        acc = qf @ kf[:, :, n0:n0 + KV_TILE].transpose(-1, -2)    # exact: |sum| < 2^24
        s = acc * (qs * k_sf[:, :, n0 // KV_TILE, None])[..., None]
        s = torch.where((n0 + pos) >= Nkv, torch.full_like(s, -math.inf), s)
        m_new = torch.maximum(s.amax(dim=-1) - EXP_OFFSET, m)
        p = torch.exp2(s - m_new[..., None])
        alpha = torch.exp2(m - m_new)
        l = l * alpha + p.sum(dim=-1)
        phat = T.e4m3_bits_to_f32(T.f32_to_e4m3_bits(p))
        o = o * alpha[..., None] + phat @ vf[:, :, :, n0:n0 + KV_TILE].transpose(-1, -2)
        m = m_new
    one = torch.ones((), dtype=torch.float32)
    return (o * ((one / l)[..., None] * v_sf[:, :, None, :Dv])).to(torch.bfloat16)


def attention_int8_x_fp8(q, k, v, layout: str = "BNHD", q_block: int = 64, k_block: int = 128) -> torch.Tensor:
    """attention(q, k, v, layout=layout, precision="int8+fp8e4m3") of the reference, on the CPU
    (python/ac4k_kernel/ops/attention.py:137-192): K minus its mean over the tokens (in bf16), the two block
    quantizers, V per (head, d) row in e4m3 with max_scale 2.25 and swizzle, then the kernel."""
    n_dim = 1 if layout == "BNHD" else 2
    k = k - k.mean(dim=n_dim, keepdim=True)
    q8, q_sf = int8_block_token_quantize(q, layout, q_block)
    k8, k_sf = int8_block_token_quantize(k, layout, k_block)
    v8, v_sf = T.quantize_fp8(v, 3, n_dim, 2.25, True)
    o = mha_int8_x_fp8_fwd(q8, q_sf, q_block, k8, k_sf, k_block, v8, v_sf, 1.0 / math.sqrt(q.shape[-1]))
    return o.permute(0, 2, 1, 3).contiguous() if layout == "BNHD" else o

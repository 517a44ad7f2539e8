"""Pins the CPU oracle of the NVFP4 attention forward (oracle/attention_oracle.py) without a GPU."""
import math

import pytest
import torch

from conftest import make_input
from oracle import attention_oracle as A
from oracle import nvfp4_oracle as T


def sdpa_fp32(q, k, v, layout):
    q, k, v = (t.float() for t in (q, k, v))
    if layout == "BNHD":
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
    s = q @ k.transpose(-1, -2) / math.sqrt(q.shape[-1])
    o = torch.softmax(s, dim=-1) @ v
    return o.transpose(1, 2).contiguous() if layout == "BNHD" else o


# the reference's own nvfp4 cases (test/test_attention_bench.py:178-191), then ragged sequence lengths
# (one kv tile partly filled, several tiles with a tail), several heads and batches, both layouts
CASES = [(1, 256, 1, 128, "BNHD"), (1, 64, 1, 128, "BNHD"), (2, 100, 3, 128, "BHND"), (1, 33, 2, 128, "BNHD"),
         (1, 300, 1, 128, "BNHD"), (1, 129, 1, 128, "BHND")]


@pytest.mark.parametrize("B,N,H,D,layout", CASES)
def test_oracle_against_fp32_attention(B, N, H, D, layout):
    """Tolerance of the reference's test: cosine similarity > 0.98, atol 0.2, rtol 0.1."""
    shape = (B, N, H, D) if layout == "BNHD" else (B, H, N, D)
    q, k, v = (make_input(shape, seed=s + N) for s in (1, 2, 3))
    o = A.attention_nvfp4(q, k, v, layout)
    ref = sdpa_fp32(q, k, v, layout)
    assert o.shape == ref.shape and o.dtype == torch.bfloat16
    cos = torch.nn.functional.cosine_similarity(o.float().flatten(), ref.flatten(), dim=0).item()
    assert cos > 0.98, cos
    if (B, N, H, D, layout) in CASES[:2]:   # the reference's own cases, at its own tolerance
        torch.testing.assert_close(o.float(), ref, atol=2e-1, rtol=1e-1)
    else:  # short rows average less quantization noise: a few elements in ten thousand pass 0.2; none reaches 0.4
        err = (o.float() - ref).abs()
        inside = (err <= 2e-1 + 1e-1 * ref.abs()).float().mean().item()
        assert inside > 0.999 and err.max().item() < 0.4, (inside, err.max().item())


def test_p_blocks_are_the_interleaved_sets():
    """Positions {8g + 4h + j} of a 32-group form the block h.  Values 1 on the h = 0 sets and 2^-8 on the
    h = 1 sets: each block has its own scale (448 and 1.75), both come back exactly.  Contiguous 16-blocks
    would put 1 and 2^-8 under one scale and round the small ones to zero."""
    pos = torch.arange(128)
    h = (pos % 8) // 4
    p = torch.where(h == 0, torch.tensor(1.0), torch.tensor(2.0 ** -8)).reshape(1, 128)
    phat, sf = A.quantize_p_tile(p)
    assert torch.equal(phat / A.P_ALPHA, p)
    assert sf.reshape(4, 2).tolist() == [[0x7E, 0x3E]] * 4   # e4m3 codes of 448 and 1.75
    # a block of zeros keeps scale 0 and multiplier 0; an isolated 1 in an h = 1 set is alone in its block
    p = torch.zeros(1, 128)
    p[0, 32 + 13] = 1.0                                      # group 1, g = 1, h = 1, j = 1
    phat, sf = A.quantize_p_tile(p)
    assert torch.equal(phat / A.P_ALPHA, p) and sf.flatten().tolist() == [0, 0, 0, 0x7E, 0, 0, 0, 0]


def test_p_scale_recipe_matches_the_quantizer_with_global_scale_1_over_2688():
    """P's quantization is the nvfp4 recipe with the global scale fixed at 1/2688 (mha_nvfp4.cu:253,276-306):
    on a tile whose 32-groups are permuted into the stored order it must equal the quantizer oracle."""
    g = torch.Generator().manual_seed(5)
    p = torch.rand((7, 128), generator=g).to(torch.bfloat16)           # bf16 so that the quantizer oracle takes it
    phat, sf = A.quantize_p_tile(p.float())
    # the quantizer's swizzle gathers the same sets: its block b of a 32-group holds positions {8g + 4b + j}
    out, qsf, _ = T.quantize_nvfp4(p, 0, 1, True, gs=torch.tensor(1.0 / 2688.0))
    deq = A.deswizzle_kv(T.dequantize_nvfp4(out, qsf, 1.0))
    assert torch.equal(deq, phat)
    assert torch.equal(T.sf_to_linear(qsf, 7), T.e4m3_bits_to_f32(sf))


def test_v_deswizzle_round_trip():
    v = make_input((1, 2, 200, 128), seed=9)                            # [B,H,N,D]
    out, sf, gs = T.quantize_nvfp4(v, 3, 2, True)                       # -> [B,H,D,N^64/2]
    deq = A.deswizzle_kv(A._dequant_rows(out, sf, 128)) * gs            # [B,H,D,256], original kv order
    ref = v.float().transpose(-1, -2)
    got = deq[..., :200]
    cos = torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0).item()
    assert cos > 0.99 and (got - ref).abs().max() < 0.3 * ref.abs().max()
    assert torch.all(deq[..., 200:] == 0)                               # padding positions quantize to zero


def test_output_is_linear_in_v_global_scale_and_invariant_to_row_order():
    q, k, v = (make_input((1, 70, 2, 128), seed=s) for s in (11, 12, 13))
    ops = list(A.quantize_qkv(q, k, v, "BNHD"))
    o1 = A.mha_nvfp4_fwd(*ops, 0.1).float()
    ops2 = list(ops)
    ops2[8] = ops[8] * 4.0
    o2 = A.mha_nvfp4_fwd(*ops2, 0.1).float()
    torch.testing.assert_close(o2, o1 * 4.0, atol=0.0, rtol=2 ** -7)    # both rounded to bf16 once
    # permuting the query rows (packed rows and their scale rows) permutes the output rows, bit for bit
    perm = torch.randperm(70, generator=torch.Generator().manual_seed(1))
    ops3 = list(ops)
    ops3[0] = ops[0][:, :, perm]
    sfq = ops[1].clone()
    sfq[:, :, :, :70] = ops[1][:, :, :, perm]
    ops3[1] = sfq
    o3 = A.mha_nvfp4_fwd(*ops3, 0.1).float()
    assert torch.equal(o3, o1[:, :, perm])


# --------------------------------------------------------------------------- INT8 (QK) x FP8 (PV)
def _sdpa(q, k, v, layout):
    q, k, v = (t.float() for t in (q, k, v))
    if layout == "BNHD":
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
    o = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(q.shape[-1]), dim=-1) @ v
    return o.transpose(1, 2).contiguous() if layout == "BNHD" else o


@pytest.mark.parametrize("B,N,H,layout", [(1, 256, 1, "BNHD"), (1, 100, 1, "BNHD"), (2, 111, 2, "BHND"), (1, 444, 1, "BNHD")])
def test_int8_x_fp8_oracle_within_the_reference_tolerance_of_fp32_attention(B, N, H, layout):
    """The end-to-end pin the reference itself uses for this operator (test/test_attention_bench.py:69-177, its
    D = 128 shapes and ragged lengths): atol 0.2, rtol 1e-2, cosine similarity > 0.99 against fp32 attention."""
    shape = (B, N, H, 128) if layout == "BNHD" else (B, H, N, 128)
    g = torch.Generator().manual_seed(N)
    q, k, v = (torch.randn(shape, generator=g).to(torch.bfloat16) for _ in range(3))
    o = A.attention_int8_x_fp8(q, k, v, layout)
    ref = _sdpa(q, k, v, layout)
    cos = torch.nn.functional.cosine_similarity(o.float().flatten(), ref.flatten(), dim=0).item()
    assert cos > 0.99, cos
    torch.testing.assert_close(o.float(), ref, atol=2e-1, rtol=1e-2)


def test_token_block_quantizer_closed_forms():
    """One scale per block of tokens = max|x| / 127 over all columns; values truncated toward zero; a zero block
    gives scale 0 and zeros; the head dim is padded to 16 with zeros; BNHD and BHND agree."""
    x = torch.zeros((1, 40, 1, 20), dtype=torch.bfloat16)
    x[0, 0, 0, 3] = 127.0      # block 0 (tokens 0-15): scale 1
    x[0, 5, 0, 7] = -2.75      # -> trunc(-2.75) = -2 (rounding to nearest would give -3)
    x[0, 15, 0, 0] = 0.99      # -> 0
    x[0, 32, 0, 1] = -63.5     # block 2 (tokens 32-39, ragged): scale 0.5 -> -127
    x[0, 39, 0, 19] = 0.75     # -> trunc(1.5) = 1
    y, s = A.int8_block_token_quantize(x, "BNHD", 16)
    assert list(y.shape) == [1, 1, 40, 32] and list(s.shape) == [1, 1, 3]
    assert s.tolist() == [[[1.0, 0.0, 0.5]]]
    assert y[0, 0, 0, 3] == 127 and y[0, 0, 5, 7] == -2 and y[0, 0, 15, 0] == 0
    assert y[0, 0, 32, 1] == -127 and y[0, 0, 39, 19] == 1
    assert int(y.abs().sum()) == 127 + 2 + 127 + 1 and (y[..., 20:] == 0).all()
    y2, s2 = A.int8_block_token_quantize(x.permute(0, 2, 1, 3).contiguous(), "BHND", 16)
    assert torch.equal(y, y2) and torch.equal(s, s2)


def test_fp8_deswizzle_inverts_the_quantizer_swizzle():
    v = torch.arange(64, dtype=torch.float32).reshape(1, 1, 2, 32).to(torch.bfloat16) / 64
    plain, _ = T.quantize_fp8(v, 2, 3, 448.0, False)
    swz, _ = T.quantize_fp8(v, 2, 3, 448.0, True)
    assert not torch.equal(plain, swz)
    assert torch.equal(A.deswizzle_fp8(swz), plain)


def test_int8_x_fp8_kernel_oracle_closed_forms():
    """Cases a person can evaluate: (1) one kv position: O is the dequantized V row whatever Q and K are;
    (2) equal scores: O is the mean of the V rows, through the 7.5 offset, p = 2^7.5 -> e4m3(181.02) = 176 for every
    position, so numerator and denominator scale alike only up to e4m3(p) / p, which the result must show;
    (3) kv positions past Nkv are masked: appending garbage rows behind Nkv changes nothing."""
    g = torch.Generator().manual_seed(3)
    v = torch.randn((1, 1, 1, 128), generator=g).to(torch.bfloat16)           # [B,H,Nkv=1,D]
    v8, v_sf = T.quantize_fp8(v, 3, 2, 2.25, True)
    q = torch.randint(-127, 128, (1, 1, 5, 128), generator=g, dtype=torch.int8)
    k = torch.randint(-127, 128, (1, 1, 1, 128), generator=g, dtype=torch.int8)
    one = torch.ones((1, 1, 1))
    o = A.mha_int8_x_fp8_fwd(q, one, 64, k, one, 128, v8, v_sf, 0.01)
    # p = 2^7.5 -> e4m3 176; l = 181.02; O = 176 / 181.02 * dequant(V)
    p = torch.exp2(torch.tensor(7.5))
    vd = T.e4m3_bits_to_f32(v8)[0, 0, :, 0] * v_sf[0, 0]
    expect = ((176.0 * T.e4m3_bits_to_f32(v8)[0, 0, :, 0]) * ((1.0 / p) * v_sf[0, 0])).to(torch.bfloat16)
    assert torch.equal(o[0, 0, 0], expect) and torch.equal(o[0, 0, 4], expect)
    assert torch.allclose(o[0, 0, 0].float(), vd * (176.0 / p), rtol=1e-2)
    # (2) all scores equal (K = 0): mean of V over 48 positions, times 176 / 2^7.5
    v = torch.randn((1, 1, 48, 128), generator=g).to(torch.bfloat16)
    v8, v_sf = T.quantize_fp8(v, 3, 2, 2.25, True)
    k0 = torch.zeros((1, 1, 48, 128), dtype=torch.int8)
    o = A.mha_int8_x_fp8_fwd(q, one, 64, k0, one, 128, v8, v_sf, 0.01)
    vdq = A.deswizzle_fp8(T.e4m3_bits_to_f32(v8))[0, 0, :, :48] * v_sf[0, 0, :, None]     # [D, 48]
    assert torch.allclose(o[0, 0, 2].float(), vdq.mean(dim=1) * (176.0 / p), atol=4e-3, rtol=1e-2)
    # (3) the masked tail: V is stored to a multiple of 16, K rows behind Nkv do not exist; a longer K / V pair that
    # agrees on the first 40 positions gives another result, the same pair cut to 40 the same one
    k = torch.randint(-127, 128, (1, 1, 48, 128), generator=g, dtype=torch.int8)
    sf = torch.full((1, 1, 1), 0.02)
    o48 = A.mha_int8_x_fp8_fwd(q, sf, 64, k, sf, 128, v8, v_sf, 0.05)
    v40 = v[:, :, :40]
    v8c, v_sfc = T.quantize_fp8(v40, 3, 2, 2.25, True)
    o40 = A.mha_int8_x_fp8_fwd(q, sf, 64, k[:, :, :40], sf, 128, v8c, v_sfc, 0.05)
    full = torch.softmax((q.float() @ k[:, :, :40].float().transpose(-1, -2)) * (0.02 * 0.02 * 0.05), -1) @ v40.float()
    assert not torch.allclose(o48.float(), o40.float(), atol=1e-2)
    assert torch.allclose(o40.float(), full, atol=5e-2, rtol=5e-2)

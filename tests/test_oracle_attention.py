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

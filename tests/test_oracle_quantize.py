"""Pins the quantize oracles: the reference's own known-answer sets re-expressed as closed
forms (test/test_quantize_bench.py:150-198 nvfp4, :223-300 fp8), explicit index formulas for
layout and swizzle, and the two independent restatements (torch, C) against each other."""
import random

import pytest
import torch

from conftest import make_input
from oracle import c_oracle as C
from oracle import nvfp4_oracle as T


def value_set_input(shape, vals, seed):
    g = torch.Generator().manual_seed(seed)
    t = torch.tensor(vals, dtype=torch.bfloat16)
    return t[torch.randint(0, len(vals), shape, generator=g)]


def to_rows(x, cross, red):
    lead = [i for i in range(x.ndim) if i not in (cross % x.ndim, red % x.ndim)]
    return x.permute(*lead, cross, red).contiguous().reshape(-1, x.shape[cross], x.shape[red])


# ---------------------------------------------------------------------------
# nvfp4 known answers: inputs from {+-1,+-2,+-4,+-6}
# ---------------------------------------------------------------------------
NVFP4_CASES = [((1024, 1024), 1, 0, False), ((128, 512), 0, 1, False), ((128, 512), 0, 1, True),
               ((77, 200), 0, 1, False), ((77, 200), 1, 0, True), ((3, 50, 70), 1, 2, False),
               ((2, 3, 33, 40), 3, 1, True), ((5, 16), 0, 1, False)]


@pytest.mark.parametrize("impl", ["torch", "c"])
@pytest.mark.parametrize("shape,cross,red,swz", NVFP4_CASES)
def test_nvfp4_value_set_closed_form(impl, shape, cross, red, swz):
    x = value_set_input(shape, [1, 2, 4, 6, -1, -2, -4, -6], seed=hash((shape, cross)) % 1000)
    q = T.quantize_nvfp4 if impl == "torch" else C.quantize_nvfp4
    out, sf, gs = q(x, cross, red, swz)
    # closed forms on this value set (every quotient is an exact e2m1 grid point):
    rows = to_rows(x, cross, red).float()
    B, R, K = rows.shape
    Kp, Rp = (K + 63) // 64 * 64, (R + 15) // 16 * 16
    rows = torch.nn.functional.pad(rows, [0, Kp - K])
    if swz:
        rows = rows.reshape(-1, 4, 4, 2).permute(0, 2, 1, 3).reshape(B, R, Kp)
    blk = rows.reshape(B, R, Kp // 16, 16)
    bmax = blk.abs().amax(-1, keepdim=True)
    gs_ref = x.float().abs().max() / 2688.0
    assert gs.item() == gs_ref.item()
    expect = torch.where(bmax > 0, blk * 6.0 / bmax.clamp(min=1), torch.zeros_like(blk))  # x / gs / (bmax/gs/6)
    dec = T.e2m1_unpack(out.reshape(B, R, Kp // 2)).reshape(B, R, Kp // 16, 16)
    torch.testing.assert_close(dec, expect, atol=1e-3, rtol=1e-6)
    sf_ref = (bmax.squeeze(-1) / gs_ref / 6.0).to(torch.float8_e4m3fn).float()
    sf_lin = T.e4m3_bits_to_f32(sf.reshape(B, Kp // 64, Rp, 4)).permute(0, 2, 1, 3).reshape(B, Rp, Kp // 16)
    torch.testing.assert_close(sf_lin[:, :R], sf_ref, atol=1e-3, rtol=1e-6)
    assert torch.all(sf_lin[:, R:] == 0)
    assert list(out.shape)[-2:] == [R, Kp // 2] and list(sf.shape)[-3:] == [Kp // 64, Rp, 4]


def test_nvfp4_scale_address_formula():
    # sf byte of (row r, 16-block j) sits at [j // 4, r, j % 4]; out byte j holds elements 2j (low), 2j+1 (high)
    x = make_input((19, 130), seed=3)
    out, sf, gs = T.quantize_nvfp4(x, 0, 1)
    xf = torch.nn.functional.pad(x.float(), [0, 192 - 130])
    alpha = 1.0 / gs
    for r in [0, 7, 18]:
        for j in [0, 3, 4, 8, 11]:
            blk = xf[r, 16 * j:16 * j + 16]
            s32 = alpha * (blk.abs().max() * T.ONE_SIXTH_F32)
            code = T.f32_to_e4m3_bits(s32.reshape(1))[0]
            assert sf[j // 4, r, j % 4] == code
            s = T.e4m3_bits_to_f32(code.reshape(1))[0]
            o = alpha * (1.0 / s) if s != 0 else torch.zeros(())
            q = T.f32_to_e2m1_bits(blk * o)
            for i in range(8):
                assert out[r, 8 * j + i] == (q[2 * i] | (q[2 * i + 1] << 4))
    assert torch.all(sf[:, 19:, :] == 0) and sf.shape == (3, 32, 4) and out.shape == (19, 96)
    assert torch.all(out[:, 65:] == 0) and torch.all(sf[2, :, 1:] == 0)  # zero padding of the reduce dim


def test_nvfp4_swizzle_index_formula():
    # out position t*8+q*2+r of every 32-group reads input position q*8+t*2+r (quantize_nvfp4.cu:89-93)
    x = make_input((4, 128), seed=5)
    perm = torch.empty(128, dtype=torch.long)
    for g in range(4):
        for t in range(4):
            for q in range(4):
                for r in range(2):
                    perm[g * 32 + t * 8 + q * 2 + r] = g * 32 + q * 8 + t * 2 + r
    a = T.quantize_nvfp4(x, 0, 1, swizzle=True)
    b = T.quantize_nvfp4(x[:, perm].contiguous(), 0, 1, swizzle=False)
    assert all(torch.equal(p, q) for p, q in zip(a, b))


def test_nvfp4_dequant_roundtrip_error_bound():
    x = make_input((64, 256), seed=7)
    out, sf, gs = T.quantize_nvfp4(x, 0, 1)
    xd = T.dequantize_nvfp4(out, sf, gs)
    blk = x.float().reshape(64, 16, 16)
    bmax = blk.abs().amax(-1, keepdim=True)
    # e2m1 spacing is at most 2 on a 0..6 grid -> error <= (1/6 + scale rounding 1/16) of the block max
    assert torch.all((xd.reshape(64, 16, 16) - blk).abs() <= bmax * (1.0 / 6.0 + 1.0 / 16.0) + 1e-6)
    requant = T.quantize_nvfp4(xd.to(torch.bfloat16), 0, 1, gs=gs)
    assert requant[0].shape == out.shape


def test_nvfp4_edges():
    # zero block inside a non-zero tensor: scale 0, nibbles keep the sign of zero
    x = torch.zeros((2, 64), dtype=torch.bfloat16)
    x[0, 0] = 3.0
    x[1, 20] = -0.0
    for q in (T.quantize_nvfp4, C.quantize_nvfp4):
        out, sf, gs = q(x, 0, 1)
        assert gs.item() == (torch.tensor(3.0) / torch.tensor(2688.0)).item()
        assert sf[0, 0, 0] == 0x7E and out[0, 0] == 0x07       # block max -> scale 448, value 6
        assert torch.all(sf[0, 1, :] == 0) and out[1, 10] == 0x08 and out[1].sum() == 8
    # scale underflow: block max below 2^-10 * 6 * gs -> sf 0 and all-zero nibbles
    y = torch.full((1, 64), 1.0, dtype=torch.bfloat16)
    y[0, 16:32] = 1e-6
    out, sf, gs = T.quantize_nvfp4(y, 0, 1)
    assert sf[0, 0, 1] == 0 and torch.all(out[0, 8:16] == 0)


def test_global_scale_closed_form_and_max_scale():
    x = make_input((33, 77), seed=9)
    amax = x.float().abs().max()
    assert T.global_scale(x).item() == (amax / 2688.0).item() == C.global_scale(x).item()
    assert T.global_scale(x, 100.0).item() == (amax / 100.0).item() == C.global_scale(x, 100.0).item()
    assert T.global_scale(torch.zeros((4, 4), dtype=torch.bfloat16)).item() == 0.0


# ---------------------------------------------------------------------------
# fp8 known answers: integer set, max_scale 2.25, bit equality (test_quantize_bench.py:223-300)
# ---------------------------------------------------------------------------
FP8_CASES = [((1024, 1024), 0, 1, False), ((1, 300, 40, 128), 3, 1, True), ((1024, 10), 0, 1, False),
             ((16, 16), 0, 1, True), ((777, 879), 0, 1, True), ((50, 70), 1, 0, False)]


@pytest.mark.parametrize("impl", ["torch", "c"])
@pytest.mark.parametrize("shape,cross,red,swz", FP8_CASES)
def test_fp8_value_set_bit_exact(impl, shape, cross, red, swz):
    vals = [-8, -6, -5, -4, 1, 2, 3, 4, 5, 6, 8, 9]
    x = value_set_input(shape, vals, seed=len(shape) * 31 + shape[0])
    rnd = random.Random(9527)
    rows = to_rows(x, cross, red)
    for b in range(rows.shape[0]):           # per-row clipping as in the reference test
        for r in range(0, rows.shape[1], 3):
            mv = abs(rnd.choice(vals))
            rows[b, r] = rows[b, r].clamp(-mv, mv)
    lead = [i for i in range(x.ndim) if i not in (cross, red)]
    inv = [0] * x.ndim
    for pos, d in enumerate(lead + [cross, red]):
        inv[d] = pos
    x = rows.reshape([x.shape[i] for i in lead] + [x.shape[cross], x.shape[red]]).permute(*inv).contiguous()
    q = T.quantize_fp8 if impl == "torch" else C.quantize_fp8
    out, sf = q(x, cross, red, 2.25, swz)
    rows = to_rows(x, cross, red).float()
    B, R, K = rows.shape
    Kp, Rp = (K + 15) // 16 * 16, (R + 15) // 16 * 16
    rows = torch.nn.functional.pad(rows, [0, Kp - K])
    if swz:
        rows = rows.reshape(-1, 2, 4, 2).permute(0, 2, 1, 3).reshape(B, R, Kp)
    amax = rows.abs().amax(-1, keepdim=True)
    sf_ref = amax.squeeze(-1) / 2.25
    out_ref = (rows / amax * 2.25).to(torch.float8_e4m3fn)     # the reference test's formula
    assert torch.equal(sf.reshape(B, Rp)[:, :R], sf_ref) and torch.all(sf.reshape(B, Rp)[:, R:] == 0)
    assert torch.equal(out.reshape(B, R, Kp), out_ref.view(torch.uint8))


def test_fp8_int8_closed_forms_on_gaussian():
    x = make_input((40, 100), seed=11, outliers=True)
    xf = torch.nn.functional.pad(x.float(), [0, 12])
    amax = xf.abs().amax(-1, keepdim=True)
    out, sf = T.quantize_fp8(x, 0, 1)
    assert torch.equal(sf[:40], (amax / 448.0).squeeze(-1)) and torch.all(sf[40:] == 0)
    ref = torch.clamp(xf * (torch.tensor(448.0) / amax), -448, 448)  # NB python_scalar / tensor is reciprocal*scalar in torch: not IEEE division
    ref = ref.to(torch.float8_e4m3fn).view(torch.uint8)
    assert torch.equal(out, ref)
    out, sf = T.quantize_int8(x, 0, 1)
    assert torch.equal(sf[:40], (amax / 127.0).squeeze(-1))
    assert torch.equal(out, torch.round(xf * (torch.tensor(127.0) / amax)).clamp(-128, 127).to(torch.int8))
    assert out.abs().max() == 127 and out.dtype == torch.int8
    out, sf = T.quantize_int8(x, 0, 1, max_scale=7)
    assert out.abs().max() == 7


def test_rowwise_zero_row_edge():
    x = make_input((3, 32), seed=13)
    x[1] = 0
    for q8, qi in ((T.quantize_fp8, T.quantize_int8), (C.quantize_fp8, C.quantize_int8)):
        out, sf = q8(x, 0, 1)
        assert sf[1] == 0 and torch.all(out[1] == 0x7F)   # 0 * inf = NaN -> 0x7F
        out, sf = qi(x, 0, 1)
        assert sf[1] == 0 and torch.all(out[1] == 0)      # NaN -> 0


# ---------------------------------------------------------------------------
# torch restatement vs C restatement on random shapes / dims / swizzle
# ---------------------------------------------------------------------------
def test_torch_vs_c_random():
    rnd = random.Random(4)
    for trial in range(40):
        nd = rnd.randint(2, 4)
        shape = [rnd.randint(1, 70) for _ in range(nd)]
        c, r = rnd.sample(range(nd), 2)
        sw = rnd.choice([False, True])
        x = make_input(shape, seed=trial, outliers=trial % 2 == 0)
        if trial % 5 == 0:
            x = x * (torch.rand(shape) < 0.5)
        a, b = T.quantize_nvfp4(x, c, r, sw), C.quantize_nvfp4(x, c, r, sw)
        assert all(torch.equal(p, q) for p, q in zip(a, b)), (shape, c, r, sw)
        a, b = T.quantize_fp8(x, c, r, None, sw), C.quantize_fp8(x, c, r, 448.0, sw)
        assert all(torch.equal(p, q) for p, q in zip(a, b)), (shape, c, r, sw)
        a, b = T.quantize_int8(x, c, r), C.quantize_int8(x, c, r)
        assert all(torch.equal(p, q) for p, q in zip(a, b)), (shape, c, r)


def test_negative_dims_and_asserts():
    x = make_input((6, 40, 20), seed=21)
    a, b = T.quantize_nvfp4(x, -2, -1), T.quantize_nvfp4(x, 1, 2)
    assert all(torch.equal(p, q) for p, q in zip(a, b))
    with pytest.raises(AssertionError):
        T.quantize_nvfp4(x, 1, 1)
    with pytest.raises(AssertionError):
        T.quantize_nvfp4(torch.zeros(8, dtype=torch.bfloat16), 0, 0)

"""Pins the oracle's scalar conversions against definitions that do not share its code:
brute-force nearest-grid-point search with explicit tie rules, torch's own casts, and the
C restatement against the torch restatement over every bf16 value times several scales."""
import math

import pytest
import torch

from oracle import c_oracle as C
from oracle import nvfp4_oracle as T

E2M1_GRID = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0]  # code = index (test/test_linear_bench.py:18-35)


def all_bf16_as_f32():
    return torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16).float()


def brute_e2m1(v: float) -> int:
    if math.isnan(v):
        return 0x7
    sign = 8 if math.copysign(1.0, v) < 0 else 0
    a = min(abs(v), 6.0)  # satfinite
    best, best_d = None, None
    for code, gv in enumerate(E2M1_GRID):
        d = abs(a - gv)
        if best is None or d < best_d or (d == best_d and code % 2 == 0):
            best, best_d = code, d
    return sign | best


def e4m3_grid():
    vals = []
    for code in range(0x7F):  # 0x7F is NaN
        e, m = code >> 3, code & 7
        vals.append(m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7))
    return vals


def brute_e4m3(v: float, grid) -> int:
    if math.isnan(v):
        return 0x7F
    sign = 0x80 if math.copysign(1.0, v) < 0 else 0
    a = min(abs(v), 448.0)
    best, best_d = None, None
    for code, gv in enumerate(grid):
        d = abs(a - gv)
        if best is None or d < best_d or (d == best_d and code % 2 == 0):
            best, best_d = code, d
    return sign | best


def test_e2m1_code_table():
    lut = T.E2M1_LUT.tolist()
    assert lut[:8] == E2M1_GRID and lut[8:] == [-v for v in E2M1_GRID]
    for c in range(16):
        assert C.lib().oracle_e2m1_to_f32(c) == lut[c] or (c == 8 and lut[c] == 0.0)


def test_e2m1_rounding_brute_force():
    # every tie point, every grid point, neighbours one ulp to either side, saturation, zeros, NaN
    pts = [0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5.0] + E2M1_GRID + [6.0001, 7.0, 100.0, 1e30, float("inf")]
    vals = []
    for p in pts:
        t = torch.tensor(p, dtype=torch.float32)
        vals += [p, float(torch.nextafter(t, torch.tensor(float("inf")))),
                 float(torch.nextafter(t, torch.tensor(-float("inf"))))]
    vals += [-v for v in vals] + [0.0, -0.0, float("nan"), 1e-30, -1e-30]
    x = torch.tensor(vals, dtype=torch.float32)
    got = T.f32_to_e2m1_bits(x).tolist()
    for v, g in zip(x.tolist(), got):
        assert g == brute_e2m1(v), (v, g)
        assert C.lib().oracle_f32_to_e2m1(v) == g, v
    assert T.f32_to_e2m1_bits(torch.tensor([-0.0]))[0] == 0x8  # sign of zero is kept
    assert T.f32_to_e2m1_bits(torch.tensor([2.5, 3.5, 5.0, 0.25, 0.75, 1.25, 1.75])).tolist() == [4, 6, 6, 0, 2, 2, 4]


def test_e2m1_random_brute_force():
    g = torch.Generator().manual_seed(1)
    x = (torch.rand(4000, generator=g) * 8 - 4) * torch.tensor([1.0, 0.1, 2.0, 0.01]).repeat(1000)
    got = T.f32_to_e2m1_bits(x).tolist()
    assert got == [brute_e2m1(v) for v in x.tolist()]


@pytest.mark.parametrize("scale", [1.0, 0.37, 3.3, 1.0 / 3.0, 448.0 / 6.0, 2.0 ** -12, 1e-3])
def test_c_vs_torch_all_bf16(scale):
    v = all_bf16_as_f32() * scale
    L = C.lib()
    vl = v.tolist()
    e2 = T.f32_to_e2m1_bits(v).tolist()
    e4 = T.f32_to_e4m3_bits(v).tolist()
    s8 = T.f32_to_s8_sat(v).tolist()
    for i, f in enumerate(vl):
        assert L.oracle_f32_to_e2m1(f) == e2[i], f
        assert L.oracle_f32_to_e4m3(f) == e4[i], f
        assert L.oracle_f32_to_s8(f) == s8[i], f


def test_e4m3_rounding_brute_force():
    grid = e4m3_grid()
    assert grid[0x7E] == 448.0 and grid[0x08] == 2.0 ** -6 and grid[0x01] == 2.0 ** -9
    g = torch.Generator().manual_seed(2)
    x = torch.cat([
        torch.tensor(grid, dtype=torch.float32),
        (torch.tensor(grid[:-1]) + torch.tensor(grid[1:])).float() / 2,  # every tie point
        torch.exp(torch.rand(3000, generator=g) * 14 - 8),               # log-uniform 3e-4 .. 400
        torch.tensor([448.0, 449.0, 463.9, 464.0, 480.0, 1e9, float("inf"), 2.0 ** -10, 2.0 ** -10 * 1.0001, 0.0]),
    ])
    x = torch.cat([x, -x, torch.tensor([float("nan")])])
    got = T.f32_to_e4m3_bits(x).tolist()
    for v, gcode in zip(x.tolist(), got):
        assert gcode == brute_e4m3(v, grid), (v, gcode)
        assert C.lib().oracle_f32_to_e4m3(v) == gcode, v


def test_e4m3_decode_matches_torch():
    codes = torch.arange(256, dtype=torch.uint8)
    ref = codes.view(torch.float8_e4m3fn).float()
    for c in range(256):
        got = C.lib().oracle_e4m3_to_f32(c)
        assert (math.isnan(got) and math.isnan(ref[c].item())) or got == ref[c].item()


def test_s8_round_half_even_and_saturation():
    x = torch.tensor([0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5, 127.5, 300.0, -128.5, -129.0, -1e9,
                      float("inf"), -float("inf"), float("nan")])
    assert T.f32_to_s8_sat(x).tolist() == [0, 2, 2, 0, -2, -2, 126, 127, 127, -128, -128, -128, 127, -128, 0]


def test_products_exact_in_fp16_and_bf16():
    # the GEMM decodes e2m1 * e4m3 to a 16-bit float: must be exact for all 8 x 127 products
    grid = torch.tensor(e4m3_grid(), dtype=torch.float64)
    vals = torch.tensor(E2M1_GRID, dtype=torch.float64)
    prod = (vals[:, None] * grid[None, :]).reshape(-1)
    assert torch.equal(prod.to(torch.float16).double(), prod)
    assert torch.equal(prod.to(torch.bfloat16).double(), prod)
    assert prod[prod > 0].min() == 2.0 ** -10 and prod.max() == 2688.0

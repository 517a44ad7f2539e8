"""Committed fixtures (tests/golden/*.npz, written by tests/golden/make_golden.py): both CPU
oracles must reproduce them (not gpu), and so must the HIP kernels (gpu)."""
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle as C
from oracle import nvfp4_oracle as T

G = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    z = np.load(os.path.join(G, name), allow_pickle=False)
    return {k: torch.from_numpy(z[k].copy()) for k in z.files}


def bf16(t):
    return t.view(torch.int16).view(torch.bfloat16)


def oracles():
    return [("torch", T), ("c", C)]


@pytest.mark.parametrize("name,impl", oracles())
def test_nvfp4_fixtures_cpu(name, impl):
    z = load("nvfp4_gauss_64x128.npz")
    out, sf, gs = impl.quantize_nvfp4(bf16(z["x"]), 0, 1)
    assert torch.equal(out, z["out"]) and torch.equal(sf, z["sf"]) and gs.item() == z["gs"].item()
    z = load("nvfp4_valueset_70x45_t_swz.npz")
    out, sf, gs = impl.quantize_nvfp4(bf16(z["x"]), 1, 0, True)
    assert torch.equal(out, z["out"]) and torch.equal(sf, z["sf"]) and gs.item() == z["gs"].item()


@pytest.mark.parametrize("name,impl", oracles())
def test_rowwise_fixture_cpu(name, impl):
    z = load("rowwise_outliers_37x200.npz")
    x = bf16(z["x"])
    out, sf = impl.quantize_fp8(x, 0, 1)
    assert torch.equal(out, z["fp8"]) and torch.equal(sf, z["fp8_sf"])
    out, sf = impl.quantize_int8(x, 0, 1)
    assert torch.equal(out, z["int8"]) and torch.equal(sf, z["int8_sf"])


def test_linear_fixture_cpu():
    z = load("linear_32x48x128_bias.npz")
    bias = bf16(z["bias"])
    for d in (T.linear_nvfp4(z["a"], z["a_sf"], z["a_gs"], z["b"], z["b_sf"], z["b_gs"], bias=bias,
                             out_dtype=torch.float32),
              C.linear_nvfp4(z["a"], z["a_sf"], z["a_gs"], z["b"], z["b_sf"], z["b_gs"], bias=bias)):
        torch.testing.assert_close(d, z["d"], atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
def test_fixtures_gpu():
    from ac4k_kernel_amd.ops import linear, quantize
    z = load("nvfp4_gauss_64x128.npz")
    out, sf, gs = quantize(bf16(z["x"]).cuda(), 0, 1)
    assert torch.equal(out.cpu(), z["out"]) and torch.equal(sf.cpu().view(torch.uint8), z["sf"])
    assert gs.item() == z["gs"].item()
    z = load("nvfp4_valueset_70x45_t_swz.npz")
    out, sf, gs = quantize(bf16(z["x"]).cuda(), 1, 0, swizzle=True)
    assert torch.equal(out.cpu(), z["out"]) and torch.equal(sf.cpu().view(torch.uint8), z["sf"])
    assert gs.item() == z["gs"].item()
    z = load("rowwise_outliers_37x200.npz")
    x = bf16(z["x"]).cuda()
    out, sf = quantize(x, 0, 1, precision="fp8e4m3")
    assert torch.equal(out.cpu().view(torch.uint8), z["fp8"]) and torch.equal(sf.cpu(), z["fp8_sf"])
    out, sf = quantize(x, 0, 1, precision="int8")
    assert torch.equal(out.cpu(), z["int8"]) and torch.equal(sf.cpu(), z["int8_sf"])
    z = load("linear_32x48x128_bias.npz")
    d = linear(z["a"].cuda(), z["a_sf"].cuda().view(torch.float8_e4m3fn), z["a_gs"].cuda(), z["b"].cuda(),
               z["b_sf"].cuda().view(torch.float8_e4m3fn), z["b_gs"].cuda(), bias=bf16(z["bias"]).cuda(),
               out=torch.empty((32, 48), dtype=torch.float32, device="cuda"))
    torch.testing.assert_close(d.cpu(), z["d"], atol=1e-2, rtol=1e-2)  # tolerance of test_linear_bench.py:152

"""Pins the linear oracle: brute-force dot products on tiny shapes, the C triple loop against
the torch dequantize-matmul (test/test_linear_bench.py:53-107), linearity in the global scales,
bias broadcast and zero contribution of padding."""
import pytest
import torch

from conftest import make_input
from oracle import c_oracle as C
from oracle import nvfp4_oracle as T

E2M1 = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def quantized_pair(m, n, k, seed=0, wstd=1.0):
    a = make_input((m, k), seed=seed)
    b = make_input((n, k), seed=seed + 100, std=wstd)
    return T.quantize_nvfp4(a, 0, 1), T.quantize_nvfp4(b, 0, 1)


def brute(aq, bq, bias, m, n):
    (a, a_sf, a_gs), (b, b_sf, b_gs) = aq, bq
    K = a.shape[1] * 2
    out = torch.zeros(m, n, dtype=torch.float64)
    for i in range(m):
        for j in range(n):
            acc = 0.0
            for k in range(K):
                av = E2M1[(int(a[i, k // 2]) >> (4 * (k % 2))) & 0xF]
                bv = E2M1[(int(b[j, k // 2]) >> (4 * (k % 2))) & 0xF]
                sa = a_sf[k // 64, i, (k % 64) // 16:(k % 64) // 16 + 1].view(torch.float8_e4m3fn).float().item()
                sb = b_sf[k // 64, j, (k % 64) // 16:(k % 64) // 16 + 1].view(torch.float8_e4m3fn).float().item()
                acc += av * sa * bv * sb
            out[i, j] = acc * float(a_gs) * float(b_gs) + (0.0 if bias is None else float(bias[j]))
    return out


@pytest.mark.parametrize("m,n,k", [(3, 5, 64), (2, 3, 50), (1, 4, 130)])
def test_tiny_brute_force(m, n, k):
    aq, bq = quantized_pair(m, n, k, seed=k)
    bias = make_input((n,), seed=5).float()
    ref = brute(aq, bq, bias, m, n)
    got = T.linear_nvfp4(*aq, *bq, bias=bias, out_dtype=torch.float32)
    got_c = C.linear_nvfp4(*aq, *bq, bias=bias)
    got_k = T.linear_nvfp4_contract(*aq, *bq, bias=bias, out_dtype=torch.float32)
    for g in (got, got_c, got_k):
        torch.testing.assert_close(g.double(), ref, atol=1e-4, rtol=1e-5)


@pytest.mark.parametrize("m,n,k", [(12, 23, 55), (33, 17, 256), (64, 64, 128), (10, 15, 512)])
def test_c_vs_torch(m, n, k):
    aq, bq = quantized_pair(m, n, k, seed=m)
    ref = T.linear_nvfp4(*aq, *bq, out_dtype=torch.float32)
    got = C.linear_nvfp4(*aq, *bq)
    torch.testing.assert_close(got, ref, atol=1e-3, rtol=1e-4)


def test_linearity_bias_and_padding():
    (a, a_sf, a_gs), (b, b_sf, b_gs) = quantized_pair(8, 9, 100, seed=3)
    base = T.linear_nvfp4(a, a_sf, a_gs, b, b_sf, b_gs, out_dtype=torch.float32)
    doubled = T.linear_nvfp4(a, a_sf, a_gs * 2, b, b_sf, b_gs * 4, out_dtype=torch.float32)
    torch.testing.assert_close(doubled, base * 8, atol=0, rtol=1e-6)
    bias = torch.arange(9, dtype=torch.float32)
    withb = T.linear_nvfp4(a, a_sf, a_gs, b, b_sf, b_gs, bias=bias, out_dtype=torch.float32)
    torch.testing.assert_close(withb - base, bias.expand(8, 9), atol=1e-5, rtol=0)
    # K = 100 is padded to 128: the 28 pad columns are zero nibbles with zero scales
    assert a.shape == (8, 64) and torch.all(a[:, 50:] == 0) and torch.all(a_sf[1, :, 3] == 0)
    # out dtype default and transposition convention: D = A @ B^T
    d = T.linear_nvfp4(a, a_sf, a_gs, b, b_sf, b_gs)
    assert d.dtype == torch.bfloat16 and d.shape == (8, 9)
    da, db = T.dequantize_nvfp4(a, a_sf, a_gs), T.dequantize_nvfp4(b, b_sf, b_gs)
    torch.testing.assert_close(base, da @ db.t(), atol=0, rtol=0)


def test_quantized_matmul_tracks_bf16_matmul():
    # sanity on magnitude: nvfp4 x nvfp4 stays within ~15 % relative Frobenius error of the bf16 product
    a, b = make_input((64, 512), seed=1), make_input((48, 512), seed=2)
    d = T.linear_nvfp4(*T.quantize_nvfp4(a, 0, 1), *T.quantize_nvfp4(b, 0, 1), out_dtype=torch.float32)
    ref = a.float() @ b.float().t()
    assert (d - ref).norm() / ref.norm() < 0.15

"""GPU tests of the pre-packed weight image: the image's byte layout against a numpy restatement of
its definition, and the linear on the image against the linear on the plain tensors (bit for bit
wherever both run the same kernel) and the fp32 dequantize-then-matmul oracle (atol = rtol = 1e-2,
test/test_linear_bench.py:152)."""
import numpy as np
import pytest
import torch

from conftest import make_input
from oracle import nvfp4_oracle as T

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2
BLOCK_ROWS, BLOCK_K, BLOCK_DATA, BLOCK_BYTES = 128, 128, 8192, 9216


def ops():
    from ac4k_kernel_amd import ops as o
    return o


def quant(shape, seed, std=1.0):
    return ops().quantize(make_input(shape, seed=seed, std=std).cuda(), 0, 1)


def cpu(q):
    return q[0].cpu(), q[1].cpu().view(torch.uint8), q[2].cpu()


def expected_image(b, b_sf):
    """The image of packed rows b [N, K/2] and scale bytes b_sf [K/64, Np, 4], from its definition."""
    n, kb = b.shape
    bands, nkt = -(-n // BLOCK_ROWS), kb * 2 // BLOCK_K
    img = np.zeros((bands, nkt, BLOCK_BYTES), dtype=np.uint8)
    for band in range(bands):
        for kt in range(nkt):
            blk = img[band, kt]
            for r in range(BLOCK_ROWS):
                row = band * BLOCK_ROWS + r
                if row >= n:
                    continue
                for p in range(4):
                    pos = p ^ ((r >> 1) & 3)
                    blk[r * 64 + pos * 16:r * 64 + pos * 16 + 16] = b[row, kt * 64 + p * 16:kt * 64 + p * 16 + 16]
                for c in range(2):
                    o = BLOCK_DATA + (c * BLOCK_ROWS + r) * 4
                    blk[o:o + 4] = b_sf[kt * 2 + c, row]
    return img.reshape(-1)


@pytest.mark.parametrize("n,k", [(130, 256), (128, 128), (5, 384)])
def test_image_layout(n, k):
    wq = quant((n, k), seed=n)
    img = ops().prepack_weight(wq[0], wq[1])
    assert img.dtype == torch.uint8 and img.numel() == -(-n // 128) * (k // 128) * BLOCK_BYTES
    exp = expected_image(wq[0].cpu().numpy(), wq[1].cpu().view(torch.uint8).numpy())
    assert np.array_equal(img.cpu().numpy(), exp)


def both(m, n, k, seed=0, wstd=0.02, bias_dtype=None, o_dtype=torch.bfloat16):
    aq, wq = quant((m, k), seed), quant((n, k), seed + 1, wstd)
    bias = None if bias_dtype is None else make_input((1, n), seed=seed + 2).to(bias_dtype).cuda()
    img = ops().prepack_weight(wq[0], wq[1])
    d_img = ops().linear_prepacked(*aq, img, wq[2], bias=bias, out=torch.full((m, n), 7.0, dtype=o_dtype, device="cuda"))
    d_plain = ops().linear(*aq, *wq, bias=bias, out=torch.full((m, n), 9.0, dtype=o_dtype, device="cuda"))
    return aq, wq, bias, d_img, d_plain


def check_oracle(aq, wq, bias, d, o_dtype):
    ref = T.linear_nvfp4(*cpu(aq), *cpu(wq), bias=None if bias is None else bias.cpu(), out_dtype=o_dtype)
    torch.testing.assert_close(d.cpu(), ref, atol=ATOL, rtol=RTOL)


# M > 32 and N >= 128: both entry points run the same kernel with the same plan (the K-split-waves kernel for
# M <= 128 with K % 256 == 0, the packed-operand tile kernel otherwise)
@pytest.mark.parametrize("m,n,k", [(33, 128, 128), (130, 257, 384), (64, 130, 1280), (300, 384, 256), (129, 1000, 512),
                                   (100, 128, 4096), (128, 1000, 768), (96, 200, 2048)])
def test_tile_kernel_bit_identical(m, n, k):
    aq, wq, bias, d_img, d_plain = both(m, n, k, seed=m, bias_dtype=torch.float32, o_dtype=torch.float32)
    assert torch.equal(d_img, d_plain)
    check_oracle(aq, wq, bias, d_img, torch.float32)


# decode-sized M with K % 256 == 0: the LDS-ring kernel on both sides when the plain side is told so
@pytest.mark.parametrize("m", [1, 5, 12, 16, 32])
@pytest.mark.parametrize("n,k", [(1024, 2048), (130, 256), (384, 14336)])
def test_lds_ring_kernel_bit_identical(m, n, k, linear_tuning):
    linear_tuning(decode_kernel=2)
    aq, wq, bias, d_img, d_plain = both(m, n, k, seed=m + n, bias_dtype=torch.bfloat16)
    assert torch.equal(d_img, d_plain)
    check_oracle(aq, wq, bias, d_img, torch.bfloat16)


# shapes whose plain layout runs another kernel (N < 128, or M <= 32 with K % 256 == 128): oracle only
@pytest.mark.parametrize("m,n,k", [(40, 64, 256), (7, 33, 384), (32, 300, 128), (200, 5, 640)])
@pytest.mark.parametrize("o", [torch.bfloat16, torch.float16, torch.float32])
def test_other_shapes_against_oracle(m, n, k, o):
    aq, wq, bias, d_img, _ = both(m, n, k, seed=k, bias_dtype=torch.float16, o_dtype=o)
    check_oracle(aq, wq, bias, d_img, o)


# configuration 3, configuration 4 at M = 128 / 2048 / 8192, the headline 8192^3, and the decode-sized
# configuration 5 (LDS-ring kernel on both sides)
LARGE = [(4096, 4096, 4096, 1.0), (8192, 8192, 8192, 1.0)]
LARGE += [(m, n, k, 0.02) for (n, k) in ((14336, 4096), (4096, 14336)) for m in (128, 2048, 8192)]
LARGE += [(m, 28672, 8192, 0.02) for m in (1, 8, 32)]


@pytest.mark.parametrize("m,n,k,wstd", LARGE)
def test_large_shapes_bit_identical(m, n, k, wstd, linear_tuning):
    if m <= 32:
        linear_tuning(decode_kernel=2)
    aq, wq, _, d_img, d_plain = both(m, n, k, wstd=wstd)
    assert torch.equal(d_img, d_plain)
    rows = torch.tensor(sorted({0, min(1, m - 1), m // 2, m - 1}))
    cols = torch.arange(0, n, max(1, n // 64))
    ca, cb = cpu(aq), cpu(wq)
    fa = T.dequantize_nvfp4(ca[0][rows], ca[1][:, rows].contiguous(), ca[2])
    fb = T.dequantize_nvfp4(cb[0][cols], cb[1][:, cols].contiguous(), cb[2])
    ref = (fa @ fb.t()).to(torch.bfloat16)
    torch.testing.assert_close(d_img[rows.cuda()][:, cols.cuda()].cpu(), ref, atol=ATOL, rtol=RTOL)
    del d_img, d_plain
    torch.cuda.empty_cache()


def test_rejections():
    wq = quant((64, 192), seed=1)  # K % 128 != 0: no image
    with pytest.raises(RuntimeError, match="multiple of 128"):
        ops().prepack_weight(wq[0], wq[1])
    aq, wq = quant((8, 256), seed=2), quant((64, 256), seed=3)
    img = ops().prepack_weight(wq[0], wq[1])
    with pytest.raises(RuntimeError, match="not the weight image"):
        ops().linear_prepacked(*aq, img[:-16], wq[2], n=64)
    with pytest.raises(RuntimeError, match="not the weight image"):
        ops().linear_prepacked(*aq, img, wq[2], n=200)

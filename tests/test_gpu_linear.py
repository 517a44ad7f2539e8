"""GPU parity of the NVFP4 linear: HIP kernel (through the C ABI) against the fp32
dequantize-then-matmul oracle at atol = rtol = 1e-2 (test/test_linear_bench.py:152)."""
import random

import pytest
import torch

from conftest import make_input
from oracle import c_oracle as C
from oracle import nvfp4_oracle as T

pytestmark = pytest.mark.gpu
ATOL = RTOL = 1e-2


def ops():
    from ac4k_kernel_amd import ops as o
    return o


def gpu_quant(x):
    out, sf, gs = ops().quantize(x.cuda(), 0, 1)
    return out, sf, gs


def cpu(q):
    return q[0].cpu(), q[1].cpu().view(torch.uint8), q[2].cpu()


def run_case(m, n, k, bias_dtype=None, o_dtype=None, seed=0, wstd=1.0):
    a, b = make_input((m, k), seed=seed), make_input((n, k), seed=seed + 1, std=wstd)
    aq, bq = gpu_quant(a), gpu_quant(b)
    bias = None if bias_dtype is None else make_input((1, n), seed=seed + 2).to(bias_dtype)
    out = None if o_dtype is None else torch.full((m, n), 7.0, dtype=o_dtype, device="cuda")
    d = ops().linear(*aq, *bq, bias=None if bias is None else bias.cuda(), out=out)
    assert d.shape == (m, n) and d.dtype == (o_dtype or torch.bfloat16)
    ref = T.linear_nvfp4(*cpu(aq), *cpu(bq), bias=bias, out_dtype=o_dtype or torch.bfloat16)
    torch.testing.assert_close(d.cpu(), ref, atol=ATOL, rtol=RTOL)
    return d


REF_SHAPES = [(128, 128, 128), (10, 512, 512), (1024, 1024, 384), (130, 384, 256), (666, 768, 512), (123, 321, 256),
              (10, 15, 512), (1, 4, 256), (64, 64, 128), (12, 23, 55), (12, 23, 5), (256, 256, 2048), (129, 257, 192)]


@pytest.mark.parametrize("m,n,k", REF_SHAPES)
def test_reference_shapes(m, n, k):
    run_case(m, n, k, seed=m + n)


DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


@pytest.mark.parametrize("o", ["bf16", "fp16", "fp32"])
@pytest.mark.parametrize("b", ["bf16", "fp16", "fp32"])
def test_dtype_matrix(o, b):
    run_case(5, 33, 51, bias_dtype=DT[b], o_dtype=DT[o], seed=5)
    run_case(130, 140, 128, bias_dtype=DT[b], o_dtype=DT[o], seed=6)


def test_bias_1d_and_out_default():
    a, b = make_input((7, 128), seed=1), make_input((9, 128), seed=2)
    aq, bq = gpu_quant(a), gpu_quant(b)
    bias = make_input((9,), seed=3)
    d = ops().linear(*aq, *bq, bias=bias.cuda())
    ref = T.linear_nvfp4(*cpu(aq), *cpu(bq), bias=bias)
    torch.testing.assert_close(d.cpu(), ref, atol=ATOL, rtol=RTOL)


def test_random_shapes():
    rnd = random.Random(9567)
    for t in range(20):
        run_case(rnd.randint(2, 555), rnd.randint(2, 555), rnd.randint(2, 555), seed=t)


def test_c_oracle_and_contract():
    a, b = make_input((96, 320), seed=11), make_input((80, 320), seed=12, std=0.02)
    aq, bq = gpu_quant(a), gpu_quant(b)
    d = ops().linear(*aq, *bq, out=torch.empty((96, 80), dtype=torch.float32, device="cuda")).cpu()
    torch.testing.assert_close(d, C.linear_nvfp4(*cpu(aq), *cpu(bq)), atol=1e-5, rtol=1e-4)
    torch.testing.assert_close(d, T.linear_nvfp4_contract(*cpu(aq), *cpu(bq), out_dtype=torch.float32), atol=1e-5,
                               rtol=1e-4)


def gpu_dequant(q, rows):
    """fp32 dequantize on the GPU with torch ops (for sizes the CPU oracle would take minutes on)."""
    packed, sf, gs = q
    lut = T.E2M1_LUT.cuda()
    v = torch.stack((lut[(packed & 0xF).long()], lut[(packed >> 4).long()]), dim=-1).reshape(rows, -1, 16)
    s = sf.permute(1, 0, 2).reshape(sf.shape[1], -1)[:rows].float() * gs
    return (v * s.unsqueeze(-1)).reshape(rows, -1)


# configuration 3, all eight LLM shapes of configuration 4, the headline 8192^3, and two of the
# reference's own timed shapes (test/test_linear_tflops.py:190-203: M = 75600 leaves a ragged last
# tile row and an output of more than 2^30 elements)
LARGE_SHAPES = [(4096, 4096, 4096, 1.0), (8192, 8192, 8192, 1.0)]
LARGE_SHAPES += [(m, n, k, 0.02) for (n, k) in ((14336, 4096), (4096, 14336)) for m in (16, 128, 2048, 8192)]
LARGE_SHAPES += [(75600, 5120, 5120, 0.02), (75600, 13824, 5120, 0.02)]


@pytest.mark.parametrize("m,n,k,wstd", LARGE_SHAPES)
def test_large_shapes(m, n, k, wstd):
    a, b = make_input((m, k), seed=0), make_input((n, k), seed=1, std=wstd)
    aq, bq = gpu_quant(a), gpu_quant(b)
    d = ops().linear(*aq, *bq)
    # (1) CPU oracle on a sample of rows and columns
    rows = torch.tensor([0, 1, m // 2, m - 1] if m >= 4 else list(range(m)))
    cols = torch.arange(0, n, max(1, n // 64))
    ca, cb = cpu(aq), cpu(bq)
    fa = T.dequantize_nvfp4(ca[0][rows], ca[1][:, rows].contiguous(), ca[2])
    fb = T.dequantize_nvfp4(cb[0][cols], cb[1][:, cols].contiguous(), cb[2])
    ref = (fa @ fb.t()).to(torch.bfloat16)
    torch.testing.assert_close(d[rows.cuda()][:, cols.cuda()].cpu(), ref, atol=ATOL, rtol=RTOL)
    # (2) the whole matrix against a torch fp32 dequantize-matmul on the GPU
    full = (gpu_dequant(aq, m) @ gpu_dequant(bq, n).t()).to(torch.bfloat16)
    torch.testing.assert_close(d, full, atol=ATOL, rtol=RTOL)
    del full, d
    torch.cuda.empty_cache()


@pytest.mark.parametrize("m,n,k", [(4096, 4096, 4096), (128, 4096, 14336), (8, 28672, 8192), (2048, 4096, 14336)])
def test_size_independent_properties(m, n, k):
    """At full BASELINE sizes, with fp32 output so that nothing is rounded after the accumulation:
    (1) the result is linear in the global scale, bit for bit for a power of two;
    (2) an output row depends only on its own activation row: permuting the rows of the packed
        activation (and of its scales) permutes the output rows, bit for bit, wherever the rows land
        in the tiling."""
    aq = gpu_quant(make_input((m, k), seed=4))
    bq = gpu_quant(make_input((n, k), seed=5, std=0.02))
    d1 = ops().linear(*aq, *bq, out=torch.empty((m, n), dtype=torch.float32, device="cuda"))
    d2 = ops().linear(aq[0], aq[1], aq[2] * 4.0, *bq, out=torch.empty((m, n), dtype=torch.float32, device="cuda"))
    assert torch.equal(d2, d1 * 4.0)
    perm = torch.randperm(m, generator=torch.Generator().manual_seed(m)).cuda()
    mp = aq[1].shape[1]
    sf_perm = aq[1].clone()
    sf_perm[:, :m] = aq[1][:, perm]
    assert mp >= m
    d3 = ops().linear(aq[0][perm].contiguous(), sf_perm, aq[2], *bq,
                      out=torch.empty((m, n), dtype=torch.float32, device="cuda"))
    assert torch.equal(d3, d1[perm])


# K = 256 is one K slice (no reduce kernel), 14336 is 28 of them; N = 130 leaves a ragged row group.
@pytest.mark.parametrize("m", [1, 2, 3, 4, 5, 8, 32])
@pytest.mark.parametrize("n,k", [(1024, 2048), (130, 256), (384, 14336)])
def test_fused_skinny_equals_composition(m, n, k):
    x = make_input((m, k), seed=m, outliers=True).cuda()
    wq = gpu_quant(make_input((n, k), seed=50, std=0.02))
    bias = make_input((1, n), seed=7).to(torch.float32).cuda()
    d, (xq, xsf, xgs) = ops().fused_linear(x, *wq, bias=bias, return_quantized=True)
    eq, esf, egs = T.quantize_nvfp4(x.cpu(), 0, 1)
    assert torch.equal(xq.cpu(), eq) and torch.equal(xsf.cpu().view(torch.uint8), esf) and xgs.item() == egs.item()
    ref = T.linear_nvfp4(eq, esf, egs, *cpu(wq), bias=bias.cpu())
    torch.testing.assert_close(d.cpu(), ref, atol=ATOL, rtol=RTOL)
    comp = ops().linear(*ops().quantize(x, 0, 1), *wq, bias=bias)
    assert torch.equal(d, comp)  # same packed activation, same kernel arithmetic, same slice order


def test_more_than_2_to_31_outputs():
    """An output of 2.15e9 elements: element offsets past 32 bits in the epilogue.  Sampled rows and a
    band of the last columns against the fp32 dequantize-matmul (on the GPU: the oracle would take
    minutes), for the 2-byte and the 4-byte epilogue."""
    m, n, k = 65536 + 16, 32768 + 8, 128
    g = torch.Generator(device="cuda").manual_seed(11)
    aq = ops().quantize(torch.empty((m, k), dtype=torch.bfloat16, device="cuda").normal_(generator=g), 0, 1)
    bq = ops().quantize(torch.empty((n, k), dtype=torch.bfloat16, device="cuda").normal_(generator=g), 0, 1)
    bias = torch.empty((1, n), dtype=torch.float32, device="cuda").normal_(generator=g)
    da, db = gpu_dequant(aq, m), gpu_dequant(bq, n)
    rows = torch.tensor([0, 1, 255, 256, m // 2, m - 17, m - 1], device="cuda")
    for dt in (torch.bfloat16, torch.float32):
        d = torch.full((m, n), 7.0, dtype=dt, device="cuda")
        ops().linear(*aq, *bq, bias=bias, out=d)
        ref = (da[rows] @ db.t() + bias).to(dt)
        torch.testing.assert_close(d[rows], ref, atol=ATOL, rtol=RTOL)
        refc = (da @ db[n - 40:].t() + bias[:, n - 40:]).to(dt)
        torch.testing.assert_close(d[:, n - 40:], refc, atol=ATOL, rtol=RTOL)
        del d, ref, refc
    torch.cuda.empty_cache()


def test_fused_skinny_edge_activations():
    """Blocks of zeros, a negative zero, one huge outlier and a whole row of zeros through the fused
    entry point: bytes, scales and global scale equal the oracle's."""
    n, k = 256, 1024
    x = make_input((3, k), seed=9)
    x[0, 64:96] = 0.0
    x[0, 70] = -0.0
    x[1, :] = 0.0
    x[2, 5] = 3000.0
    wq = gpu_quant(make_input((n, k), seed=52, std=0.02))
    d, (xq, xsf, xgs) = ops().fused_linear(x.cuda(), *wq, return_quantized=True)
    eq, esf, egs = T.quantize_nvfp4(x, 0, 1)
    assert torch.equal(xq.cpu(), eq) and torch.equal(xsf.cpu().view(torch.uint8), esf) and xgs.item() == egs.item()
    torch.testing.assert_close(d.cpu(), T.linear_nvfp4(eq, esf, egs, *cpu(wq)), atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("m,n,k", [(1, 256, 256), (7, 300, 512), (16, 130, 768), (32, 1000, 1024), (32, 64, 4096),
                                   (5, 33, 2304)])
def test_decode_sized_shapes(m, n, k):
    # the weight-streaming split-K path (M <= 32, K % 256 == 0), ragged N, all output / bias dtypes
    run_case(m, n, k, seed=m + k, wstd=0.02)
    run_case(m, n, k, bias_dtype=torch.float32, o_dtype=torch.float32, seed=m, wstd=0.02)
    run_case(m, n, k, bias_dtype=torch.bfloat16, o_dtype=torch.float16, seed=n, wstd=0.02)


# the decode-sized kernels at every M class (the library picks by M and N; here each is forced: 1 registers,
# 2 LDS ring with 128-row tiles, 3 LDS ring with 64-row tiles): ragged N, one K range and several, every
# output / bias type
@pytest.mark.parametrize("kind", [1, 2, 3])
@pytest.mark.parametrize("m", [1, 5, 8, 11, 12, 16, 17, 31, 32])
def test_decode_kernels_forced(kind, m, linear_tuning):
    linear_tuning(decode_kernel=kind)
    for (n, k) in [(1000, 1024), (130, 256), (384, 3584), (4096, 2048)]:
        run_case(m, n, k, seed=m + k + kind, wstd=0.02)
    run_case(m, 520, 1536, bias_dtype=torch.float32, o_dtype=torch.float32, seed=m, wstd=0.02)
    run_case(m, 200, 768, bias_dtype=torch.bfloat16, o_dtype=torch.float16, seed=m + 1, wstd=0.02)
    linear_tuning(skinny_ks=256, decode_kernel=kind)  # as many K ranges as K allows
    run_case(m, 333, 1280, bias_dtype=torch.float16, seed=m + 2, wstd=0.02)


@pytest.mark.parametrize("m", [1, 8, 32])
def test_fused_decode_config5(m):
    n, k = 28672, 8192
    x = make_input((m, k), seed=m, outliers=True).cuda()
    wq = gpu_quant(make_input((n, k), seed=51, std=0.02))
    d1, (xq, xsf, xgs) = ops().fused_linear(x, *wq, return_quantized=True)
    d2 = ops().fused_linear(x, *wq)                       # second call: the ticket counters reset themselves
    assert torch.equal(d1, d2)
    eq, esf, egs = T.quantize_nvfp4(x.cpu(), 0, 1)
    assert torch.equal(xq.cpu(), eq) and torch.equal(xsf.cpu().view(torch.uint8), esf) and xgs.item() == egs.item()
    cols = torch.arange(0, n, 97)
    cw = cpu(wq)
    fb = T.dequantize_nvfp4(cw[0][cols], cw[1][:, cols].contiguous(), cw[2])
    ref = (T.dequantize_nvfp4(eq, esf, egs) @ fb.t()).to(torch.bfloat16)
    torch.testing.assert_close(d1.cpu()[:, cols], ref, atol=ATOL, rtol=RTOL)
    full = (gpu_dequant((xq, xsf, xgs), m) @ gpu_dequant(wq, n).t()).to(torch.bfloat16)
    torch.testing.assert_close(d1, full, atol=ATOL, rtol=RTOL)


# 32 < M with few output tiles: the 128-row packed tile, with split-K through a workspace when K is
# long enough, and without (short K, or N too small for the packed kernel)
MID_SHAPES = [(33, 512, 1024), (64, 256, 4096), (100, 300, 2048), (128, 1024, 4096), (128, 4096, 1024),
              (129, 512, 2048), (200, 333, 1536), (256, 512, 8192), (128, 520, 512), (48, 128, 256),
              (96, 2050, 1152), (128, 14336, 4096)]


@pytest.mark.parametrize("m,n,k", MID_SHAPES)
def test_mid_m_shapes(m, n, k):
    from ac4k_kernel_amd import _lib
    run_case(m, n, k, seed=m + k, wstd=0.02)
    if _lib.load().ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k) > 0:
        # the split-K reduction applies bias and output type in its own kernel
        run_case(m, n, k, bias_dtype=torch.float32, o_dtype=torch.float16, seed=m + k + 1, wstd=0.02)
        run_case(m, n, k, bias_dtype=torch.bfloat16, o_dtype=torch.float32, seed=m + k + 2, wstd=0.02)


# the K-split-waves kernel (32 < M <= 128, K % 256 == 0: all of M in one tile, the four waves split every
# 256-k stage): its three tiles (128 x 64 above 64 rows, 64 x 64 below, 64 x 128 for very wide weights), ragged
# M and N, K shorter and longer than the stage ring, one K range and forced ranges of one and two stages
# (partial sums through the workspace), every output / bias type
KSPLIT_SHAPES = [(33, 64, 256), (64, 200, 512), (65, 64, 1280), (100, 333, 2048), (128, 130, 3072), (127, 1000, 768),
                 (40, 24600, 256), (128, 2048, 2560)]


@pytest.mark.parametrize("m,n,k", KSPLIT_SHAPES)
@pytest.mark.parametrize("ks", [0, 256, 512])
def test_ksplit_kernel(m, n, k, ks, linear_tuning):
    linear_tuning(skinny_ks=ks)
    run_case(m, n, k, seed=m + k + ks, wstd=0.02)
    run_case(m, n, k, bias_dtype=torch.float32, o_dtype=torch.float16, seed=m + k + 1, wstd=0.02)
    run_case(m, n, k, bias_dtype=torch.bfloat16, o_dtype=torch.float32, seed=m + k + 2, wstd=0.02)


def test_ksplit_kernel_against_c_oracle():
    """fp32 output of the K-split-waves kernel against the C oracle's double sum: 1e-5, far inside the
    1e-2 contract, so a dropped chunk, a swapped scale or a wrong k part would show."""
    for (m, n, k) in [(128, 192, 1024), (50, 70, 512)]:
        aq, bq = gpu_quant(make_input((m, k), seed=21)), gpu_quant(make_input((n, k), seed=22, std=0.02))
        d = ops().linear(*aq, *bq, out=torch.empty((m, n), dtype=torch.float32, device="cuda")).cpu()
        torch.testing.assert_close(d, C.linear_nvfp4(*cpu(aq), *cpu(bq)), atol=1e-5, rtol=1e-4)


# every tile shape of the packed-LDS kernel (64*mi rows x 64*nj columns, its own LDS stage depth),
# alone and split along K, forced through ac4k_set_linear_tuning; ragged M and N included
TILE_PLANS = [(2, 1, 1), (2, 2, 1), (2, 4, 1), (4, 2, 1), (4, 4, 1), (2, 1, 3), (2, 2, 2), (2, 4, 5), (4, 2, 2), (4, 4, 4)]


@pytest.mark.parametrize("mi,nj,splits", TILE_PLANS)
def test_tile_plans(mi, nj, splits, linear_tuning):
    linear_tuning(mi, nj, splits)
    for (m, n, k) in [(64 * mi, 128 * nj, 1280), (64 * mi + 37, 64 * nj * 3 - 10, 1536), (33, 136, 2048)]:
        run_case(m, n, k, seed=mi * 100 + nj * 10 + splits, wstd=0.02)
        run_case(m, n, k, bias_dtype=torch.bfloat16, o_dtype=torch.float32, seed=m + n, wstd=0.02)
        run_case(m, n, k, bias_dtype=torch.float32, o_dtype=torch.float16, seed=m + n + 1, wstd=0.02)
    # K of one and of two stages: shorter than the stage ring
    run_case(96, 256, 128, seed=3)
    run_case(96, 256, 256, bias_dtype=torch.float16, seed=4)


def test_mid_m_workspace_entry_matches_plain_entry():
    """The workspace-assisted entry point and ac4k_linear_nvfp4 compute the same contract; with fp32
    output they agree to accumulation-order noise."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    m, n, k = 128, 1024, 4096
    aq, bq = gpu_quant(make_input((m, k), seed=1)), gpu_quant(make_input((n, k), seed=2, std=0.02))
    nbytes = L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k)
    assert nbytes > 0
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    d1 = torch.empty((m, n), dtype=torch.float32, device="cuda")
    d2 = torch.empty_like(d1)
    st = torch.cuda.current_stream().cuda_stream
    args = (aq[0].data_ptr(), aq[1].data_ptr(), aq[2].data_ptr(), bq[0].data_ptr(), bq[1].data_ptr(), bq[2].data_ptr(),
            None, 0, m, n, k)
    _lib.check(L.ac4k_linear_nvfp4(d1.data_ptr(), 2, *args, st))
    _lib.check(L.ac4k_linear_nvfp4_skinny(d2.data_ptr(), 2, *args, ws.data_ptr(), nbytes, st))
    torch.testing.assert_close(d1.cpu(), d2.cpu(), atol=1e-5, rtol=1e-4)
    assert L.ac4k_linear_nvfp4_skinny(d2.data_ptr(), 2, *args, ws.data_ptr(), nbytes - 1, st) != 0
    assert b"workspace too small" in L.ac4k_last_error()


@pytest.mark.parametrize("m,n,k", [(8, 28672, 8192), (32, 28672, 8192), (16, 14336, 4096), (1, 256, 256), (40, 14336, 4096)])
def test_reference_shaped_entry_runs_the_fast_kernels(m, n, k):
    """ac4k_linear_nvfp4 has the reference's signature (no workspace).  Where the plan of the workspace entry
    point needs no scratch (one K range per tile) both entry points run the same kernel: equal outputs,
    bit for bit, through the C ABI."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    assert L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k) == 0
    aq, bq = gpu_quant(make_input((m, k), seed=m)), gpu_quant(make_input((n, k), seed=n, std=0.02))
    bias = make_input((1, n), seed=9).float().cuda()
    d1 = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    d2 = torch.full((m, n), -7.0, dtype=torch.bfloat16, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (aq[0].data_ptr(), aq[1].data_ptr(), aq[2].data_ptr(), bq[0].data_ptr(), bq[1].data_ptr(), bq[2].data_ptr(),
            bias.data_ptr(), 2, m, n, k)
    _lib.check(L.ac4k_linear_nvfp4(d1.data_ptr(), 0, *args, st))
    if m <= 32:
        _lib.check(L.ac4k_linear_nvfp4_skinny(d2.data_ptr(), 0, *args, None, 0, st))
        assert torch.equal(d1, d2)
    full = (gpu_dequant(aq, m) @ gpu_dequant(bq, n).t() + bias).to(torch.bfloat16)
    torch.testing.assert_close(d1, full, atol=ATOL, rtol=RTOL)


@pytest.mark.parametrize("m,n,k", [(16, 4096, 14336), (4, 1024, 4096), (1, 4096, 2048), (32, 384, 3584)])
def test_reference_shaped_entry_without_scratch_on_split_shapes(m, n, k):
    """Shapes whose best plan splits K: ac4k_linear_nvfp4 streams the weights with one K range per tile
    instead (no scratch), within the contract; the workspace entry point gives the split result."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    assert L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k) > 0
    aq, bq = gpu_quant(make_input((m, k), seed=m)), gpu_quant(make_input((n, k), seed=n, std=0.02))
    d1 = torch.full((m, n), 7.0, dtype=torch.float32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    _lib.check(L.ac4k_linear_nvfp4(d1.data_ptr(), 2, aq[0].data_ptr(), aq[1].data_ptr(), aq[2].data_ptr(),
                                   bq[0].data_ptr(), bq[1].data_ptr(), bq[2].data_ptr(), None, 0, m, n, k, st))
    d2 = ops().linear(*aq, *bq, out=torch.empty((m, n), dtype=torch.float32, device="cuda"))
    torch.testing.assert_close(d1, d2, atol=1e-5, rtol=1e-4)
    full = gpu_dequant(aq, m) @ gpu_dequant(bq, n).t()
    torch.testing.assert_close(d1, full, atol=ATOL, rtol=RTOL)


def test_graph_replay_of_linear_paths():
    """Captured calls of the tile kernel, the split-K path and the fused decode path replay correctly
    with eager work in between (no host-side state is baked into a launch)."""
    k, n = 2048, 512
    wq = gpu_quant(make_input((n, k), seed=3, std=0.02))
    cases = []
    for m, fused in ((1, True), (16, True), (128, False), (300, False)):
        x = make_input((m, k), seed=m).cuda()
        xs = x.clone()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):  # warm-up outside the capture
            if fused:
                ops().fused_linear(xs, *wq)
            else:
                ops().linear(*ops().quantize(xs, 0, 1), *wq)
        torch.cuda.current_stream().wait_stream(side)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            d = ops().fused_linear(xs, *wq) if fused else ops().linear(*ops().quantize(xs, 0, 1), *wq)
        cases.append((m, xs, g, d))
    for rep in range(3):
        for m, xs, g, d in cases:
            x = make_input((m, k), seed=100 * rep + m)
            xs.copy_(x.cuda())
            g.replay()
            torch.cuda.synchronize()
            aq = T.quantize_nvfp4(x, 0, 1, False)
            ref = T.linear_nvfp4(*aq, *cpu(wq))
            torch.testing.assert_close(d.cpu(), ref, atol=ATOL, rtol=RTOL)
        run_case(40, 96, 256, seed=rep)  # eager work between the replays


def test_error_behaviour():
    o = ops()
    aq, bq = gpu_quant(make_input((8, 128), seed=1)), gpu_quant(make_input((16, 128), seed=2))
    with pytest.raises(RuntimeError):
        o.linear(*aq, *bq, out=torch.empty((8, 16), dtype=torch.float64, device="cuda"))
    with pytest.raises(RuntimeError):
        o.linear(*aq, *bq, bias=torch.zeros((1, 15), device="cuda"))
    with pytest.raises(RuntimeError):
        o.linear(aq[0], aq[1][:, :8], aq[2], *bq)        # scale tensor with the wrong row padding
    with pytest.raises(RuntimeError):
        o.linear(aq[0][:, :60], aq[1], aq[2], *bq)       # non-contiguous / K mismatch
    with pytest.raises(RuntimeError):
        o.linear(aq[0], aq[1], aq[2].reshape(1), *bq)    # global scale must be 0-dim


@pytest.mark.parametrize("m,n,k", [(5, 7, 48), (70, 130, 80), (3, 4, 16), (33, 140, 208)])
def test_k_not_a_multiple_of_64(m, n, k):
    """The quantizer pads K to 64, so operands with a K % 64 tail are built by hand: random nibbles, random
    finite block scales for the K/16 blocks that exist and 0x7E (448) in the unused slots of the last
    scale dword, which the kernel must not read into the sum.  Checked against the C oracle (fp64 sum)
    and against a dequantize-matmul written out here."""
    g = torch.Generator().manual_seed(k * 1000 + m)
    nb, nc = k // 16, (k + 63) // 64

    def operand(rows):
        packed = torch.randint(0, 256, (rows, k // 2), generator=g, dtype=torch.uint8)
        rp = (rows + 15) // 16 * 16
        sf = torch.full((nc, rp, 4), 0x7E, dtype=torch.uint8)
        codes = torch.randint(0x20, 0x48, (rows, nb), generator=g, dtype=torch.uint8)  # 2^-3 .. 3.5
        for j in range(nb):
            sf[j // 4, :rows, j % 4] = codes[:, j]
        return packed, sf, torch.tensor(0.5 + rows / 256.0, dtype=torch.float32)

    a, b = operand(m), operand(n)
    d = torch.empty((m, n), dtype=torch.float32, device="cuda")
    ops().linear(a[0].cuda(), a[1].cuda().view(torch.float8_e4m3fn), a[2].cuda(),
                 b[0].cuda(), b[1].cuda().view(torch.float8_e4m3fn), b[2].cuda(), out=d)
    ref_c = C.linear_nvfp4(*a, *b)

    def dequant(q, rows):
        v = T.e2m1_unpack(q[0]).float().reshape(rows, nb, 16)
        s = T.sf_to_linear(q[1], rows)[:, :nb] * q[2]
        return (v * s.unsqueeze(-1)).reshape(rows, k).double()

    ref_t = (dequant(a, m) @ dequant(b, n).t()).float()
    torch.testing.assert_close(ref_c, ref_t, atol=1e-4, rtol=1e-5)
    torch.testing.assert_close(d.cpu(), ref_c, atol=1e-4, rtol=1e-5)

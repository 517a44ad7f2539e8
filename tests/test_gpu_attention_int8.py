"""GPU parity of the INT8 (QK) x FP8 (PV) attention forward (head dims up to 128) and of the per-token-block int8
quantizer in front of it: the HIP kernels, through the C ABI, against the CPU oracle on the same operands, and
the whole `attention(..., precision="int8+fp8e4m3")` call against an fp32 attention at the tolerance of the
reference's test (test/test_attention_bench.py:69-177: atol 0.2, rtol 1e-2, cosine similarity > 0.99)."""
import math

import pytest
import torch

from conftest import make_input
from oracle import attention_oracle as A
from oracle import nvfp4_oracle as T

pytestmark = pytest.mark.gpu

# The kernel and the oracle evaluate the same contract on the same operands; they differ in the order of the fp32
# sums and in the last bit of exp2, which now and then moves a probability across an e4m3 rounding boundary.
ATOL = RTOL = 2e-2


def ops():
    from ac4k_kernel_amd import ops as o
    return o


def binding():
    from ac4k_kernel_amd import _rocm_ops
    return _rocm_ops


def sdpa_fp32(q, k, v, layout):
    q, k, v = (t.float() for t in (q, k, v))
    if layout == "BNHD":
        q, k, v = (t.transpose(1, 2) for t in (q, k, v))
    o = torch.softmax(q @ k.transpose(-1, -2) / math.sqrt(q.shape[-1]), dim=-1) @ v
    return o.transpose(1, 2).contiguous() if layout == "BNHD" else o


@pytest.mark.parametrize("shape,layout,block", [((1, 100, 1, 128), "BNHD", 64), ((2, 3, 333, 128), "BHND", 128),
                                                 ((1, 64, 2, 100), "BNHD", 32), ((2, 2, 17, 12), "BHND", 16),
                                                 ((1, 200, 3, 88), "BNHD", 64)])
def test_token_block_quantizer_bit_exact(shape, layout, block):
    """Scales and int8 values equal the oracle's bit for bit, over ragged last blocks, head dims that are padded
    to 16, both layouts, an all-zero block and an outlier."""
    x = make_input(shape, seed=11, outliers=True)
    if layout == "BHND":
        x[0, 0, :block] = 0  # one block whose scale is 0
    ey, es = A.int8_block_token_quantize(x, layout, block)
    n_dim = 1 if layout == "BNHD" else 2
    import importlib
    front = importlib.import_module("ac4k_kernel_amd.ops.attention")  # the module (`ops.attention` is the function)
    y, s = front._int8_quantize(x.cuda(), layout, n_dim, BLOCK_SIZE=block)
    assert y.dtype == torch.int8 and list(y.shape) == list(ey.shape) and list(s.shape) == list(es.shape)
    assert torch.equal(s.cpu(), es) and torch.equal(y.cpu(), ey)


# the first rows are the reference's own test shapes (test/test_attention_bench.py:69-177), head dims 12 to 128
CASES = [(1, 256, 1, 128, "BNHD"), (1, 100, 1, 128, "BNHD"), (2, 111, 2, 100, "BHND"), (1, 444, 1, 88, "BNHD"),
         (11, 100, 12, 12, "BNHD"), (11, 100, 12, 65, "BNHD"), (2, 330, 3, 100, "BNHD"), (2, 111, 2, 128, "BHND"),
         (1, 129, 2, 128, "BHND"), (2, 1, 1, 128, "BNHD"), (1, 1000, 4, 128, "BNHD"),
         # enough (query block, head) pairs that the kernel takes 256 query rows per workgroup, ragged last block
         (1, 300, 200, 128, "BHND")]


@pytest.mark.parametrize("B,N,H,D,layout", CASES)
def test_attention_against_oracle_and_fp32(B, N, H, D, layout):
    shape = (B, N, H, D) if layout == "BNHD" else (B, H, N, D)
    q, k, v = (make_input(shape, seed=s + N) for s in (1, 2, 3))
    o = ops().attention(q.cuda(), k.cuda(), v.cuda(), layout=layout, precision="int8+fp8e4m3")
    assert o.shape == shape and o.dtype == torch.bfloat16
    ref = A.attention_int8_x_fp8(q, k, v, layout)
    torch.testing.assert_close(o.cpu().float(), ref.float(), atol=ATOL, rtol=RTOL)
    if N < 32:  # a single kv position returns the quantized V row itself: nothing averages its rounding
        return
    full = sdpa_fp32(q, k, v, layout)
    cos = torch.nn.functional.cosine_similarity(o.cpu().float().flatten(), full.flatten(), dim=0).item()
    assert cos > 0.99, cos
    torch.testing.assert_close(o.cpu().float(), full, atol=2e-1, rtol=1e-2)


def test_entry_point_on_given_operands():
    """The C entry point on hand-made operands: different lengths of q and kv, q blocks of 32, scales that are not
    those of a quantizer (a zero scale among them), an output with odd strides; against the oracle."""
    B, H, Nq, Nkv = 2, 3, 77, 200
    g = torch.Generator().manual_seed(5)
    q = torch.randint(-127, 128, (B, H, Nq, 128), generator=g, dtype=torch.int8)
    k = torch.randint(-127, 128, (B, H, Nkv, 128), generator=g, dtype=torch.int8)
    q_sf = torch.rand((B, H, 3), generator=g) * 0.01
    k_sf = torch.rand((B, H, 2), generator=g) * 0.01
    k_sf[0, 0, 1] = 0.0
    v = make_input((B, H, Nkv, 128), seed=6)
    v8, v_sf = T.quantize_fp8(v, 3, 2, 2.25, True)
    ref = A.mha_int8_x_fp8_fwd(q, q_sf, 32, k, k_sf, 128, v8, v_sf, 0.09)
    store = torch.zeros((B, H, Nq, 130), dtype=torch.bfloat16, device="cuda")
    o = store[..., 1:129]
    binding().mha_int8_x_fp8_fwd(o, q.cuda(), q_sf.cuda(), 32, k.cuda(), k_sf.cuda(), 128,
                                 v8.cuda().view(torch.float8_e4m3fn), v_sf.cuda(), 0.09)
    torch.testing.assert_close(o.cpu().float(), ref.float(), atol=ATOL, rtol=RTOL)
    assert (store[..., 0] == 0).all() and (store[..., 129] == 0).all()


def test_error_behaviour():
    b = binding()
    q = torch.zeros((1, 1, 16, 128), dtype=torch.int8, device="cuda")
    sf = torch.ones((1, 1, 1), device="cuda")
    v = torch.zeros((1, 1, 128, 16), dtype=torch.float8_e4m3fn, device="cuda")
    v_sf = torch.ones((1, 1, 128), device="cuda")
    o = torch.empty((1, 1, 16, 128), dtype=torch.bfloat16, device="cuda")
    b.mha_int8_x_fp8_fwd(o, q, sf, 64, q, sf, 128, v, v_sf, 1.0)
    with pytest.raises(RuntimeError, match="Q must be"):
        b.mha_int8_x_fp8_fwd(o, q.float(), sf, 64, q, sf, 128, v, v_sf, 1.0)
    with pytest.raises(RuntimeError, match="k_quantize_block_size"):
        b.mha_int8_x_fp8_fwd(o, q, sf, 64, q, torch.ones((1, 1, 1), device="cuda"), 64, v, v_sf, 1.0)
    with pytest.raises(RuntimeError, match="multiple of 16"):
        q24 = torch.zeros((1, 1, 16, 24), dtype=torch.int8, device="cuda")
        b.mha_int8_x_fp8_fwd(o, q24, sf, 64, q24, sf, 128, v, v_sf, 1.0)


@pytest.mark.parametrize("precision", ["int8+fp8e4m3", "nvfp4"])
def test_reference_long_sequence_shape(precision):
    """The long shape of the reference's test list, (1, 75600, 1, 128) BNHD (test/test_attention_bench.py:69-77), for
    both precisions, against an fp32 attention evaluated on the GPU in blocks of query rows, at the reference's
    tolerance."""
    B, N, H, D = 1, 75600, 1, 128
    g = torch.Generator(device="cuda").manual_seed(9567)
    q, k, v = (torch.empty((B, N, H, D), dtype=torch.float32, device="cuda").normal_(generator=g).to(torch.bfloat16)
               for _ in range(3))
    o = ops().attention(q, k, v, layout="BNHD", precision=precision)
    kf, vf = k[0, :, 0].float(), v[0, :, 0].float()
    ref = torch.empty((N, D), dtype=torch.float32, device="cuda")
    for m0 in range(0, N, 4096):
        s = (q[0, m0:m0 + 4096, 0].float() @ kf.t()) / math.sqrt(D)
        ref[m0:m0 + 4096] = torch.softmax(s, dim=-1) @ vf
    got = o[0, :, 0].float()
    cos = torch.nn.functional.cosine_similarity(got.flatten(), ref.flatten(), dim=0).item()
    rtol, stol = (1e-2, 0.99) if precision == "int8+fp8e4m3" else (1e-1, 0.98)
    assert cos > stol, cos
    torch.testing.assert_close(got, ref, atol=2e-1, rtol=rtol)


@pytest.mark.parametrize("precision", ["int8+fp8e4m3", "nvfp4"])
def test_random_shapes(precision):
    """Seeded random batch sizes, head counts, lengths around the tile and block boundaries, head dims and layouts,
    some with outliers: the whole `attention()` call against the oracle."""
    import random
    rnd = random.Random(2024 if precision == "nvfp4" else 4202)
    for t in range(14):
        B, H = rnd.choice([1, 1, 2, 3]), rnd.choice([1, 2, 3, 5, 40])
        N = rnd.choice([1, 15, 16, 17, 63, 64, 65, 127, 128, 129, 255, 256, 257, 300, 511, 777])
        if H == 40:
            N = min(N, 300)
        D = rnd.choice([128, 128, 64, 100, 40, 88, 96, 16, 120])
        layout = rnd.choice(["BNHD", "BHND"])
        shape = (B, N, H, D) if layout == "BNHD" else (B, H, N, D)
        q, k, v = (make_input(shape, seed=s * 1000 + t, outliers=rnd.random() < 0.3) for s in (1, 2, 3))
        o = ops().attention(q.cuda(), k.cuda(), v.cuda(), layout=layout, precision=precision)
        ref = A.attention_nvfp4(q, k, v, layout) if precision == "nvfp4" else A.attention_int8_x_fp8(q, k, v, layout)
        torch.testing.assert_close(o.cpu().float(), ref.float(), atol=ATOL, rtol=RTOL, msg=lambda m: f"{shape} {layout}: {m}")

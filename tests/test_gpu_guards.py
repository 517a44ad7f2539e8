"""No entry point writes outside the buffers it is given (GPU, through the C ABI).

Every output (and the workspace of the scratch-assisted linears) is a window inside a larger
allocation whose margins hold a byte pattern; after the call the margins must be untouched and the
window must hold what the same call writes into an ordinary tensor.  The shapes are chosen to reach
every quantize kernel and every linear kernel family, with edge tiles and unaligned windows.
"""
import pytest
import torch

from conftest import make_input

pytestmark = pytest.mark.gpu

MARGIN = 4096
PATTERN = 0xA5


class Window:
    """`shape`/`dtype` tensor placed `shift` bytes after a 256-byte boundary inside a padded buffer."""

    def __init__(self, shape, dtype, shift=0):
        n = 1
        for s in shape:
            n *= s
        self.nbytes = n * torch.empty((), dtype=dtype).element_size()
        self.buf = torch.full((MARGIN + shift + self.nbytes + MARGIN,), PATTERN, dtype=torch.uint8, device="cuda")
        self.lo = MARGIN + shift
        assert self.buf.data_ptr() % 256 == 0
        self.t = self.buf[self.lo:self.lo + self.nbytes].view(dtype).reshape(tuple(shape))

    def intact(self):
        b = self.buf
        return bool((b[:self.lo] == PATTERN).all().item()) and bool((b[self.lo + self.nbytes:] == PATTERN).all().item())


def ops():
    from ac4k_kernel_amd import ops as o
    return o


def same_bytes(a, b):
    return torch.equal(a.contiguous().view(torch.uint8), b.contiguous().view(torch.uint8))


# (shape, cross, reduce, swizzle): small single launch, single launch with the grid wait, two-kernel row-major
# (K % 64 != 0), leading dims, reduce dim strided (cross contiguous), everything else
NVFP4_CASES = [
    ((16, 4096), 0, 1, False), ((5, 64), 0, 1, True), ((1024, 4096), 0, 1, False), ((300, 1088), 0, 1, True),
    ((257, 1000), 0, 1, False), ((33, 48), 0, 1, True), ((3, 5, 40, 128), 2, 3, False), ((2, 300, 5, 128), 3, 1, True),
    ((2, 77, 3, 136), 3, 1, False), ((130, 70), 1, 0, False), ((3, 50, 70), 1, 0, True), ((2, 3, 9, 40), 1, 3, False),
]


@pytest.mark.parametrize("shape,c,r,swz", NVFP4_CASES)
def test_nvfp4_quantize_stays_inside_its_outputs(shape, c, r, swz):
    x = make_input(shape, seed=sum(shape), outliers=True).cuda()
    eo, es, eg = ops().quantize(x, c, r, swizzle=swz)
    wo, ws = Window(eo.shape, torch.uint8, shift=0), Window(es.shape, torch.float8_e4m3fn, shift=0)
    o, s, g = ops().quantize(x, c, r, swizzle=swz, output=wo.t, sf=ws.t)
    torch.cuda.synchronize()
    assert wo.intact() and ws.intact()
    assert same_bytes(o, eo) and same_bytes(s, es) and g.item() == eg.item()


# row in registers (several widths), long rows, reduce dim strided, everything else
ROWWISE_CASES = [
    ((64, 48), 0, 1), ((70, 100), 0, 1), ((33, 1000), 0, 1), ((40, 4096), 0, 1), ((9, 16384), 0, 1), ((6, 20000), 0, 1),
    ((2, 300, 5, 128), 3, 1), ((2, 77, 3, 136), 3, 1), ((130, 70), 1, 0), ((2, 3, 9, 40), 1, 3), ((3, 5, 40, 128), 2, 3),
]


@pytest.mark.parametrize("precision", ["fp8e4m3", "int8"])
@pytest.mark.parametrize("shape,c,r", ROWWISE_CASES)
def test_rowwise_quantize_stays_inside_its_outputs(shape, c, r, precision):
    x = make_input(shape, seed=sum(shape) + 1, outliers=True).cuda()
    for swz in ((False, True) if precision == "fp8e4m3" else (False,)):
        eo, es = ops().quantize(x, c, r, precision=precision, swizzle=swz)
        wo, ws = Window(eo.shape, eo.dtype), Window(es.shape, torch.float32)
        o, s = ops().quantize(x, c, r, precision=precision, swizzle=swz, output=wo.t, sf=ws.t)
        torch.cuda.synchronize()
        assert wo.intact() and ws.intact()
        assert same_bytes(o, eo) and same_bytes(s, es)


def test_global_scale_writes_four_bytes():
    from ac4k_kernel_amd import _rocm_ops
    x = make_input((1000, 1001), seed=3).cuda()
    w = Window((), torch.float32)
    _rocm_ops.global_scale(w.t, x, 2688.0)
    torch.cuda.synchronize()
    assert w.intact()
    assert w.t.item() == (x.abs().max().float().cpu() / 2688.0).item()  # IEEE division, as on the CPU


# (M, N, K, tile plan or None): generic kernel (K % 64 != 0), fp16-tile kernel (K % 128 == 64), packed-LDS kernel
# with interior and edge tiles of every shape, row lengths that rule the 16-byte stores out, K ranges
LINEAR_CASES = [
    (5, 33, 48, None), (130, 140, 48, None), (200, 300, 192, None), (300, 330, 256, None), (300, 333, 256, None),
    (256, 256, 512, None), (520, 777, 384, "4,4,1"), (300, 328, 1024, "4,2,1"), (300, 135, 1024, "2,4,2"),
    (129, 200, 1536, "2,2,3"), (100, 70, 1024, "2,1,4"), (64, 1000, 4096, None),
]


@pytest.mark.parametrize("odt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m,n,k,plan", LINEAR_CASES)
def test_linear_stays_inside_its_output(m, n, k, plan, odt, linear_tuning):
    if plan:
        linear_tuning(*[int(v) for v in plan.split(",")])
    aq = ops().quantize(make_input((m, k), seed=m).cuda(), 0, 1)
    bq = ops().quantize(make_input((n, k), seed=n, std=0.02).cuda(), 0, 1)
    bias = make_input((1, n), seed=7).float().cuda()
    ref = ops().linear(*aq, *bq, bias=bias, out=torch.empty((m, n), dtype=odt, device="cuda"))
    esize = torch.empty((), dtype=odt).element_size()
    for shift in (0, esize):  # 256-byte aligned, and aligned to the element only
        w = Window((m, n), odt, shift=shift)
        ops().linear(*aq, *bq, bias=bias, out=w.t)
        torch.cuda.synchronize()
        assert w.intact(), (m, n, k, plan, shift)
        assert same_bytes(w.t, ref), (m, n, k, plan, shift)


@pytest.mark.parametrize("kind", [0, 1, 2, 3])  # decode-sized shapes: the library's choice, register kernel, LDS ring (128, 64 rows)
@pytest.mark.parametrize("m,n,k", [(1, 1000, 1024), (5, 136, 2048), (32, 520, 512), (16, 130, 3584), (128, 1024, 4096),
                                   (96, 300, 2048)])
def test_workspace_linear_stays_inside_workspace_and_output(m, n, k, kind, linear_tuning):
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    if kind and m > 32:
        pytest.skip("the kernel choice only exists for decode-sized shapes")
    linear_tuning(decode_kernel=kind)
    aq = ops().quantize(make_input((m, k), seed=m).cuda(), 0, 1)
    bq = ops().quantize(make_input((n, k), seed=n, std=0.02).cuda(), 0, 1)
    nbytes = L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k)  # 0: one K range per tile, nothing to write there
    ref = ops().linear(*aq, *bq)
    d, ws = Window((m, n), torch.bfloat16), Window((max(nbytes, 256),), torch.uint8)
    _lib.check(L.ac4k_linear_nvfp4_skinny(d.t.data_ptr(), 0, aq[0].data_ptr(), aq[1].data_ptr(), aq[2].data_ptr(),
                                          bq[0].data_ptr(), bq[1].data_ptr(), bq[2].data_ptr(), None, 0, m, n, k,
                                          ws.t.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert d.intact() and ws.intact()
    assert same_bytes(d.t, ref)


@pytest.mark.parametrize("m,n,k", [(1, 1000, 1024), (7, 136, 2048), (32, 520, 512)])
def test_fused_linear_stays_inside_every_buffer(m, n, k):
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    x = make_input((m, k), seed=m + 50, outliers=True).cuda()
    bq = ops().quantize(make_input((n, k), seed=n, std=0.02).cuda(), 0, 1)
    ref, (rq, rs, rg) = ops().fused_linear(x, *bq, return_quantized=True)
    nbytes = L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k)
    d, ws = Window((m, n), torch.bfloat16), Window((max(nbytes, 256),), torch.uint8)
    xq, xs, xg = Window(rq.shape, torch.uint8), Window(rs.shape, torch.float8_e4m3fn), Window((), torch.float32)
    _lib.check(L.ac4k_linear_nvfp4_fused_bf16(d.t.data_ptr(), 0, x.data_ptr(), xq.t.data_ptr(), xs.t.data_ptr(),
                                              xg.t.data_ptr(), bq[0].data_ptr(), bq[1].data_ptr(), bq[2].data_ptr(),
                                              None, 0, m, n, k, ws.t.data_ptr(), nbytes,
                                              torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert all(w.intact() for w in (d, ws, xq, xs, xg))
    assert same_bytes(d.t, ref) and same_bytes(xq.t, rq) and same_bytes(xs.t, rs) and xg.t.item() == rg.item()


# the weight image and the linear that reads it: tile kernel (edge tiles, split along K), LDS-ring kernel (one and
# several K ranges, 16- and 32-row activation stages), ragged N inside the last 128-row band
@pytest.mark.parametrize("m,n,k", [(1, 1000, 1024), (12, 136, 2048), (32, 520, 512), (128, 1024, 4096), (96, 300, 2048),
                                   (300, 130, 384), (20, 64, 128)])
def test_prepacked_linear_stays_inside_image_workspace_and_output(m, n, k):
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    aq = ops().quantize(make_input((m, k), seed=m + 3).cuda(), 0, 1)
    bq = ops().quantize(make_input((n, k), seed=n + 3, std=0.02).cuda(), 0, 1)
    st = torch.cuda.current_stream().cuda_stream
    nimg = L.ac4k_prepack_weight_nvfp4_bytes(n, k)
    assert nimg == -(-n // 128) * (k // 128) * 9216
    img = Window((nimg,), torch.uint8)
    _lib.check(L.ac4k_prepack_weight_nvfp4(img.t.data_ptr(), bq[0].data_ptr(), bq[1].data_ptr(), n, k, st))
    torch.cuda.synchronize()
    assert img.intact()
    assert same_bytes(img.t, ops().prepack_weight(bq[0], bq[1]))
    nws = L.ac4k_linear_nvfp4_prepacked_workspace_bytes(m, n, k)
    ref = ops().linear_prepacked(*aq, img.t, bq[2], n=n)
    for shift in (0, 2):  # 256-byte aligned, and aligned to the element only
        d, ws = Window((m, n), torch.bfloat16, shift=shift), Window((max(nws, 16),), torch.uint8)
        _lib.check(L.ac4k_linear_nvfp4_prepacked(d.t.data_ptr(), 0, aq[0].data_ptr(), aq[1].data_ptr(), aq[2].data_ptr(),
                                                 img.t.data_ptr(), bq[2].data_ptr(), None, 0, m, n, k,
                                                 ws.t.data_ptr() if nws else None, nws, st))
        torch.cuda.synchronize()
        assert d.intact() and ws.intact() and img.intact(), (m, n, k, shift)
        assert same_bytes(d.t, ref), (m, n, k, shift)


def test_attention_stays_inside_its_output():
    """The attention kernel writes O through its strides: a BNHD output that is a window inside a pattern-filled
    allocation keeps its surroundings, for query lengths that leave a ragged last tile."""
    import math
    for (B, Nq, Nkv, H) in ((1, 33, 70, 2), (2, 130, 130, 1), (1, 260, 200, 192)):  # the last: 256-row workgroups
        q = make_input((B, Nq, H, 128), seed=3).cuda()
        k, v = make_input((B, Nkv, H, 128), seed=4).cuda(), make_input((B, Nkv, H, 128), seed=5).cuda()
        qq, kq, vq = ops().quantize(q, 1, 3), ops().quantize(k, 1, 3), ops().quantize(v, 3, 1, swizzle=True)
        ref = torch.empty((B, Nq, H, 128), dtype=torch.bfloat16, device="cuda")
        ops().mha_nvfp4_fwd(ref.permute(0, 2, 1, 3), *qq, *kq, *vq, 1 / math.sqrt(128))
        w = Window((B, Nq, H, 128), torch.bfloat16)
        ops().mha_nvfp4_fwd(w.t.permute(0, 2, 1, 3), *qq, *kq, *vq, 1 / math.sqrt(128))
        torch.cuda.synchronize()
        assert w.intact() and same_bytes(w.t, ref)
        # the int8 x fp8 attention on the same shapes, and its quantizer's outputs
        import importlib
        front = importlib.import_module("ac4k_kernel_amd.ops.attention")
        q8, q_sf = front._int8_quantize(q, "BNHD", 1, BLOCK_SIZE=64)
        k8, k_sf = front._int8_quantize(k, "BNHD", 1, BLOCK_SIZE=128)
        v8, v_sf = ops().quantize(v, 3, 1, swizzle=True, max_scale=2.25, precision="fp8e4m3")
        ops().mha_int8_x_fp8_fwd(ref.permute(0, 2, 1, 3), q8, q_sf, 64, k8, k_sf, 128, v8, v_sf, 1 / math.sqrt(128))
        w = Window((B, Nq, H, 128), torch.bfloat16)
        ops().mha_int8_x_fp8_fwd(w.t.permute(0, 2, 1, 3), q8, q_sf, 64, k8, k_sf, 128, v8, v_sf, 1 / math.sqrt(128))
        wy, ws = Window(tuple(q8.shape), torch.int8), Window(tuple(q_sf.shape), torch.float32)
        from ac4k_kernel_amd import _rocm_ops
        _rocm_ops.quantize_int8_token_block(wy.t, ws.t, q.permute(0, 2, 1, 3), 64)
        torch.cuda.synchronize()
        assert w.intact() and same_bytes(w.t, ref)
        assert wy.intact() and ws.intact() and same_bytes(wy.t, q8) and same_bytes(ws.t, q_sf)

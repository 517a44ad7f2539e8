"""GPU parity of the quantizers: HIP kernels (through the C ABI) against the CPU oracle,
bit for bit, on the same seeded inputs."""
import random

import pytest
import torch

from conftest import make_input
from oracle import c_oracle as C
from oracle import nvfp4_oracle as T

pytestmark = pytest.mark.gpu


def ops():
    from ac4k_kernel_amd import ops as o
    return o


def check_nvfp4(x, cross, red, swz=False, oracle=T, **kw):
    out, sf, gs = ops().quantize(x.cuda(), cross, red, swizzle=swz, **kw)
    eo, es, eg = oracle.quantize_nvfp4(x, cross, red, swz, **({"max_scale": kw["max_scale"]} if "max_scale" in kw else {}))
    same_gs = gs.item() == eg.item() or (gs.item() != gs.item() and eg.item() != eg.item())  # NaN equals NaN here
    assert gs.dtype == torch.float32 and gs.dim() == 0 and same_gs, (gs.item(), eg.item())
    assert out.dtype == torch.uint8 and sf.dtype == torch.float8_e4m3fn
    assert list(out.shape) == list(eo.shape) and list(sf.shape) == list(es.shape)
    sfb = sf.cpu().view(torch.uint8)
    nb = (out.cpu() != eo).sum().item()
    ns = (sfb != es).sum().item()
    assert nb == 0 and ns == 0, f"shape {tuple(x.shape)} cross {cross} reduce {red} swz {swz}: {nb} bytes, {ns} scales differ"


NVFP4_SHAPES = [((128, 512), 0, 1), ((4096, 4096), 0, 1), ((1024, 1024), 1, 0), ((777, 879), 0, 1),
                ((12, 5), 0, 1), ((1, 64), 0, 1), ((17, 8), 0, 1), ((33, 200), 0, 1), ((100, 1000), 0, 1),
                ((3, 50, 72), 1, 2), ((3, 50, 72), 2, 1), ((2, 3, 40, 128), 2, 3), ((2, 300, 5, 128), 1, 3),
                ((2, 300, 5, 128), 3, 1), ((5, 7, 96), 0, 2), ((257, 520), 0, 1), ((64, 136), 0, 1)]


@pytest.mark.parametrize("shape,cross,red", NVFP4_SHAPES)
@pytest.mark.parametrize("swz", [False, True])
def test_nvfp4_gaussian(shape, cross, red, swz):
    check_nvfp4(make_input(shape, seed=len(shape) + shape[-1], outliers=True), cross, red, swz)


def test_nvfp4_value_set_and_c_oracle():
    g = torch.Generator().manual_seed(9567)
    vals = torch.tensor([1, 2, 4, 6, -1, -2, -4, -6], dtype=torch.bfloat16)
    for shape, c, r, s in [((1024, 1024), 1, 0, False), ((128, 512), 0, 1, False), ((300, 77), 0, 1, True)]:
        x = vals[torch.randint(0, 8, shape, generator=g)]
        check_nvfp4(x, c, r, s, oracle=C)


def test_nvfp4_random_shapes():
    rnd = random.Random(9527)
    for t in range(25):
        shape = [rnd.randint(1, 512) for _ in range(2)]
        c = rnd.randint(0, 1)
        check_nvfp4(make_input(shape, seed=t), c, 1 - c, rnd.choice([False, True]))


def test_nvfp4_config2_outliers_and_max_scale():
    x = make_input((8192, 4096), seed=0, outliers=True)
    check_nvfp4(x, 0, 1)
    check_nvfp4(make_input((64, 256), seed=1), 0, 1, max_scale=1000.0)


def test_nvfp4_edges():
    x = torch.zeros((20, 100), dtype=torch.bfloat16)
    x[3, 5], x[7, 70], x[9, 20] = 3.0, -0.5, -0.0
    check_nvfp4(x, 0, 1)
    check_nvfp4(torch.zeros((16, 64), dtype=torch.bfloat16), 0, 1)           # all-zero tensor: gs = 0
    tiny = torch.full((4, 64), 1.0, dtype=torch.bfloat16)
    tiny[:, 16:32] = 1e-6                                                    # block scale underflow
    check_nvfp4(tiny, 0, 1)
    big = make_input((32, 128), seed=2).float() * 1e30                       # large magnitudes
    check_nvfp4(big.to(torch.bfloat16), 0, 1)


def test_nvfp4_all_scale_codes():
    # global scale 1 (one element is 6 * 448), then a block whose maximum is 6 * e4m3(c) for every
    # code c: the kernel's reciprocal table is exercised entry by entry, plus in-between maxima
    codes = torch.arange(1, 127, dtype=torch.uint8)
    sv = codes.view(torch.float8_e4m3fn).float()
    g = torch.Generator().manual_seed(5)
    x = (torch.rand((126 * 4, 16), generator=g) * 2 - 1)
    mx = torch.cat([sv * 6.0, sv * 6.0 * 1.03, sv * 6.0 * 0.97, sv * 6.0 * 1.06]).clamp(max=2688.0)
    x = x * mx[:, None]
    x[:, 3] = mx * torch.where(torch.rand(126 * 4, generator=g) < 0.5, -1.0, 1.0)
    x = x.reshape(-1, 64).contiguous()
    x = torch.cat([x, torch.zeros((1, 64))])
    x[-1, 0] = 2688.0
    xb = x.to(torch.bfloat16)
    check_nvfp4(xb, 0, 1)
    _, sf, gs = T.quantize_nvfp4(xb, 0, 1)
    assert gs.item() == 1.0 and len(set(sf.flatten().tolist())) >= 126


# Dense shapes with the reduce dim a multiple of 64 take the single-launch quantizer; its three ways
# through (grid wait passes; the wait runs out and every workgroup recomputes the missing maxima from
# memory itself; fill + maxima + quantize) must agree with the oracle bit for bit.  (96, 1024) is 192 KB:
# above the 128 KB of the one-launch kernel without a grid wait, below the 256 KB that kernel takes under
# graph capture.
ONEPASS_SHAPES = [((64, 128), 0, 1), ((8192, 4096), 0, 1), ((4096, 4096), 0, 1), ((1000, 2048), 0, 1),
                  ((33, 14336), 0, 1), ((2049, 192), 0, 1), ((3, 37, 256), 1, 2), ((2, 3, 40, 128), 2, 3),
                  ((5000, 64), 0, 1), ((1, 8192), 0, 1), ((32, 8192), 0, 1), ((6100, 5120), 0, 1), ((96, 1024), 0, 1),
                  ((64, 1024), 0, 1)]


# which path ac4k_quantize_nvfp4_bf16 took: ac4k_debug_last_quantize_path()
PATH_SMALL, PATH_ONEPASS, PATH_TWO_KERNEL = 1, 2, 3


@pytest.mark.parametrize("timeout_us", [200, 0, -1])
def test_nvfp4_single_launch_paths(timeout_us):
    """200: the grid wait as shipped; 0: every workgroup looks once at the others' words and recomputes
    the maxima that are missing from memory (the path of a wait that ran out); -1: single-launch
    kernel off (fill + maxima + quantize)."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    L.ac4k_set_quantize_sync_timeout_us(timeout_us)
    try:
        for i, (shape, c, r) in enumerate(ONEPASS_SHAPES):
            check_nvfp4(make_input(shape, seed=40 + i, outliers=True), c, r)
            numel = 1
            for d in shape:
                numel *= d
            expect = PATH_SMALL if numel * 2 <= 128 * 1024 and timeout_us >= 0 else (PATH_ONEPASS if timeout_us >= 0 else PATH_TWO_KERNEL)
            assert L.ac4k_debug_last_quantize_path() == expect, (shape, L.ac4k_debug_last_quantize_path())
            check_nvfp4(make_input(shape, seed=80 + i, outliers=True), c, r, swz=True)
        # repeated calls on one stream reuse the synchronisation words with a new launch number
        x = make_input((512, 1024), seed=3)
        for _ in range(5):
            check_nvfp4(x, 0, 1)
        # scales that are not positive finite numbers take the full-range arithmetic
        check_nvfp4(torch.zeros(128, 256, dtype=torch.bfloat16), 0, 1)
        check_nvfp4(torch.zeros(1024, 256, dtype=torch.bfloat16), 0, 1)
        for rows in (128, 2048):
            z = make_input((rows, 256), seed=5)
            z[5, 7] = float("inf")
            check_nvfp4(z, 0, 1)
            z[5, 7] = float("nan")
            check_nvfp4(z, 0, 1)
    finally:
        L.ac4k_set_quantize_sync_timeout_us(200)


def test_nvfp4_single_launch_two_streams():
    """Two streams quantize at once: whichever way the workgroups get scheduled (waits may time out),
    both results are exact."""
    xs = [make_input((4096, 2048), seed=70 + i, outliers=True) for i in range(2)]
    exp = [T.quantize_nvfp4(x, 0, 1, False) for x in xs]
    dev = [x.cuda() for x in xs]
    streams = [torch.cuda.Stream() for _ in xs]
    torch.cuda.synchronize()
    res = [[], []]
    for _ in range(4):
        for i, st in enumerate(streams):
            with torch.cuda.stream(st):
                res[i].append(ops().quantize(dev[i], 0, 1))
    torch.cuda.synchronize()
    for i in range(2):
        for out, sf, gs in res[i]:
            assert gs.item() == exp[i][2].item()
            assert torch.equal(out.cpu(), exp[i][0]) and torch.equal(sf.cpu().view(torch.uint8), exp[i][1])


# cross dim contiguous, reduce dim strided (the layout of V in the reference's attention wrappers,
# python/ac4k_kernel/ops/attention.py:116,169; its bandwidth test uses (1, 75600, 40, 128))
CROSSMAJOR_SHAPES = [((1, 756, 40, 128), 3, 1), ((2, 100, 3, 40), 3, 1), ((200, 128), 1, 0), ((77, 8), 1, 0),
                     ((5, 1000, 24), 2, 1), ((3, 2, 4100, 16), 3, 2), ((2100, 136), 1, 0)]


@pytest.mark.parametrize("shape,cross,red", CROSSMAJOR_SHAPES)
@pytest.mark.parametrize("swz", [False, True])
def test_crossmajor_layouts(shape, cross, red, swz):
    x = make_input(shape, seed=shape[-1] + red, outliers=True)
    check_nvfp4(x, cross, red, swz)
    out, sf = ops().quantize(x.cuda(), cross, red, precision="fp8e4m3", swizzle=swz)
    eo, es = T.quantize_fp8(x, cross, red, None, swz)
    assert torch.equal(out.cpu().view(torch.uint8), eo) and torch.equal(sf.cpu(), es)
    if not swz:
        out, sf = ops().quantize(x.cuda(), cross, red, precision="int8")
        eo, es = T.quantize_int8(x, cross, red)
        assert torch.equal(out.cpu(), eo) and torch.equal(sf.cpu(), es)


def test_nvfp4_graph_replay():
    """A captured quantize call replays correctly: under capture the library takes the path whose whole
    state is in the caller's buffers, so nothing in it depends on host-side state that changes from
    launch to launch, and eager calls in between do not disturb it."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    shape = (2048, 1024)
    static = make_input(shape, seed=1).cuda()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        ops().quantize(static, 0, 1)
        assert L.ac4k_debug_last_quantize_path() == PATH_ONEPASS
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out, sf, gs = ops().quantize(static, 0, 1)
        assert L.ac4k_debug_last_quantize_path() == PATH_TWO_KERNEL
    for seed in (11, 12, 13, 14):
        x = make_input(shape, seed=seed, outliers=True)
        static.copy_(x.cuda())
        graph.replay()
        torch.cuda.synchronize()
        eo, es, eg = T.quantize_nvfp4(x, 0, 1, False)
        assert gs.item() == eg.item()
        assert torch.equal(out.cpu(), eo) and torch.equal(sf.cpu().view(torch.uint8), es)
        check_nvfp4(make_input((300, 640), seed=seed), 0, 1)  # eager work between the replays


def test_nvfp4_graph_replay_next_to_eager_calls():
    """Two captured quantizes replay on a second stream while the capture stream and a third stream run
    eager single-launch quantizes: captured calls share no state with anything, every result is exact."""
    shapes = [(2048, 1024), (1024, 4096)]
    xs = [make_input(sh, seed=30 + i, outliers=True) for i, sh in enumerate(shapes)]
    exp = [T.quantize_nvfp4(x, 0, 1, False) for x in xs]
    statics = [x.cuda() for x in xs]
    graphs, outs = [], []
    for st in statics:
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            outs.append(ops().quantize(st, 0, 1))
        graphs.append(g)
    replay_stream, eager_stream = torch.cuda.Stream(), torch.cuda.Stream()
    eager_in = make_input((4096, 2048), seed=77, outliers=True)
    eager_exp = T.quantize_nvfp4(eager_in, 0, 1, False)
    eager_dev = eager_in.cuda()
    torch.cuda.synchronize()
    eager_res = []
    for rep in range(3):
        with torch.cuda.stream(replay_stream):
            for g in graphs:
                g.replay()
        eager_res.append(ops().quantize(eager_dev, 0, 1))          # on the stream the graphs were captured from
        with torch.cuda.stream(eager_stream):
            eager_res.append(ops().quantize(eager_dev, 0, 1))
        torch.cuda.synchronize()
        for (out, sf, gs), (eo, es, eg) in zip(outs, exp):
            assert gs.item() == eg.item()
            assert torch.equal(out.cpu(), eo) and torch.equal(sf.cpu().view(torch.uint8), es)
    for out, sf, gs in eager_res:
        assert gs.item() == eager_exp[2].item()
        assert torch.equal(out.cpu(), eager_exp[0]) and torch.equal(sf.cpu().view(torch.uint8), eager_exp[1])


def test_nvfp4_slots_are_recycled():
    """A process that keeps creating and destroying streams keeps the single-launch path: the 100th
    stream gets synchronisation words like the first."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    x = make_input((1024, 2048), seed=55, outliers=True)
    exp = T.quantize_nvfp4(x, 0, 1, False)
    dx = x.cuda()
    torch.cuda.synchronize()
    for i in range(100):
        st = torch.cuda.Stream()
        with torch.cuda.stream(st):
            out, sf, gs = ops().quantize(dx, 0, 1)
            assert L.ac4k_debug_last_quantize_path() == PATH_ONEPASS, i
        st.synchronize()
        if i % 33 == 0 or i == 99:
            assert gs.item() == exp[2].item()
            assert torch.equal(out.cpu(), exp[0]) and torch.equal(sf.cpu().view(torch.uint8), exp[1])
        del st


def test_nvfp4_many_streams():
    """More streams at once than the library has sets of synchronisation words: late streams evict the
    least recently used ones, whose kernels may still be waiting on those words - such a kernel stops
    waiting after its timeout and finishes through its slow path.  Every result is still exact."""
    x = make_input((300, 640), seed=21, outliers=True)
    big = make_input((2048, 2048), seed=22)
    ex, eb = T.quantize_nvfp4(x, 0, 1, False), T.quantize_nvfp4(big, 0, 1, False)
    dx, db = x.cuda(), big.cuda()
    streams = [torch.cuda.Stream() for _ in range(40)]
    torch.cuda.synchronize()
    results = []
    for st in streams:
        with torch.cuda.stream(st):
            results.append((ops().quantize(dx, 0, 1), ops().quantize(db, 0, 1)))
    torch.cuda.synchronize()
    for rx, rb in results:
        for (out, sf, gs), (eo, es, eg) in ((rx, ex), (rb, eb)):
            assert gs.item() == eg.item()
            assert torch.equal(out.cpu(), eo) and torch.equal(sf.cpu().view(torch.uint8), es)


def test_nvfp4_host_threads_share_a_stream():
    """Several host threads quantize on the same stream at once (the C calls run without the GIL):
    the launches of one call stay together, so every result is exact."""
    import threading
    shapes = [(1024, 2048), (300, 640), (4096, 1024), (8192, 8192 // 8)]
    xs = [make_input(sh, seed=90 + i, outliers=True) for i, sh in enumerate(shapes)]
    exp = [T.quantize_nvfp4(x, 0, 1, False) for x in xs]
    dev = [x.cuda() for x in xs]
    stream = torch.cuda.current_stream()
    results = [[] for _ in xs]

    def work(i):
        with torch.cuda.stream(stream):
            for _ in range(25):
                results[i].append(ops().quantize(dev[i], 0, 1))

    threads = [threading.Thread(target=work, args=(i,)) for i in range(len(xs))]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    torch.cuda.synchronize()
    for i, res in enumerate(results):
        for out, sf, gs in res:
            assert gs.item() == exp[i][2].item()
            assert torch.equal(out.cpu(), exp[i][0]) and torch.equal(sf.cpu().view(torch.uint8), exp[i][1])


def test_many_leading_indices():
    """More than 65535 (batch-like) leading indices: the launches are issued in slices."""
    x = make_input((300, 256, 2, 8), seed=8, outliers=True)
    check_nvfp4(x, 2, 3)
    check_nvfp4(x, 3, 2, True)
    for cross, red in ((2, 3), (3, 2)):
        out, sf = ops().quantize(x.cuda(), cross, red, precision="fp8e4m3")
        eo, es = T.quantize_fp8(x, cross, red, None, False)
        assert torch.equal(out.cpu().view(torch.uint8), eo) and torch.equal(sf.cpu(), es)
        out, sf = ops().quantize(x.cuda(), cross, red, precision="int8")
        eo, es = T.quantize_int8(x, cross, red)
        assert torch.equal(out.cpu(), eo) and torch.equal(sf.cpu(), es)


def test_nvfp4_caller_buffers_and_negative_dims():
    x = make_input((40, 192), seed=3).cuda()
    out = torch.full((40, 96), 0xAA, dtype=torch.uint8, device="cuda")
    sf = torch.full((3, 48, 4), 0.5, device="cuda").to(torch.float8_e4m3fn)
    o2, s2, gs = ops().quantize(x, -2, -1, output=out, sf=sf)
    assert o2 is out and s2 is sf
    eo, es, eg = T.quantize_nvfp4(x.cpu(), 0, 1)
    assert torch.equal(out.cpu(), eo) and torch.equal(sf.cpu().view(torch.uint8), es)


def test_global_scale_unaligned_and_sizes():
    from ac4k_kernel_amd import _rocm_ops
    base = make_input((1 << 20) + 37, seed=4).cuda()
    for off, n in [(0, 1), (1, 7), (3, 1000), (5, 65536 + 3), (0, (1 << 20) + 37), (7, 1 << 20)]:
        x = base[off:off + n]
        gs = torch.full((), 123.0, device="cuda")
        _rocm_ops.global_scale(gs, x, 2688.0)
        assert gs.item() == T.global_scale(x.cpu()).item(), (off, n)


ROW_SHAPES = [((1024, 1024), 0, 1), ((8192, 4096), 0, 1), ((1024, 10), 0, 1), ((16, 16), 0, 1), ((777, 879), 0, 1),
              ((2, 300, 5, 128), 3, 1), ((2, 300, 5, 128), 1, 3), ((50, 70), 1, 0), ((33, 8200), 0, 1),
              ((9, 20000), 0, 1), ((65, 264), 0, 1), ((3, 50, 72), 1, 2), ((100, 2056), 0, 1)]


@pytest.mark.parametrize("shape,cross,red", ROW_SHAPES)
def test_fp8_gaussian(shape, cross, red):
    x = make_input(shape, seed=shape[0], outliers=True)
    for swz in (False, True):
        out, sf = ops().quantize(x.cuda(), cross, red, precision="fp8e4m3", swizzle=swz)
        eo, es = T.quantize_fp8(x, cross, red, None, swz)
        assert out.dtype == torch.float8_e4m3fn and list(out.shape) == list(eo.shape)
        assert torch.equal(sf.cpu(), es), (shape, swz)
        n = (out.cpu().view(torch.uint8) != eo).sum().item()
        assert n == 0, f"{shape} swz={swz}: {n} bytes differ"


@pytest.mark.parametrize("shape,cross,red", ROW_SHAPES)
def test_int8_gaussian(shape, cross, red):
    x = make_input(shape, seed=shape[0] + 1, outliers=True)
    out, sf = ops().quantize(x.cuda(), cross, red, precision="int8")
    eo, es = T.quantize_int8(x, cross, red)
    assert out.dtype == torch.int8 and list(out.shape) == list(eo.shape)
    assert torch.equal(sf.cpu(), es)
    n = (out.cpu() != eo).sum().item()
    assert n == 0, f"{shape}: {n} bytes differ"


def test_fp8_value_set_bit_exact():
    g = torch.Generator().manual_seed(9567)
    vals = torch.tensor([-8, -6, -5, -4, 1, 2, 3, 4, 5, 6, 8, 9], dtype=torch.bfloat16)
    for shape, c, r, s in [((1024, 1024), 0, 1, False), ((1, 500, 40, 128), 3, 1, True), ((1024, 10), 0, 1, False),
                           ((16, 16), 0, 1, True), ((777, 879), 0, 1, True)]:
        x = vals[torch.randint(0, len(vals), shape, generator=g)]
        out, sf = ops().quantize(x.cuda(), c, r, max_scale=2.25, swizzle=s, precision="fp8e4m3")
        eo, es = C.quantize_fp8(x, c, r, 2.25, s)
        assert torch.equal(sf.cpu(), es) and torch.equal(out.cpu().view(torch.uint8), eo), shape


def test_rowwise_edges_and_max_scale():
    x = make_input((40, 96), seed=6)
    x[5] = 0                                   # zero row: fp8 bytes 0x7F, int8 bytes 0, scale 0
    x[6, :] = 1e-38                            # amax so small that scale_max / amax overflows
    for prec, orc, kw in [("fp8e4m3", T.quantize_fp8, {}), ("int8", T.quantize_int8, {}),
                          ("fp8e4m3", T.quantize_fp8, {"max_scale": 1000.0}), ("int8", T.quantize_int8, {"max_scale": 7})]:
        out, sf = ops().quantize(x.cuda(), 0, 1, precision=prec, **kw)
        eo, es = orc(x, 0, 1, *( [kw["max_scale"]] if kw else []))
        raw = out.cpu().view(torch.uint8) if prec == "fp8e4m3" else out.cpu()
        assert torch.equal(sf.cpu(), es), (prec, kw)
        assert torch.equal(raw, eo), (prec, kw, (raw != eo).nonzero()[:4])


def test_more_than_2_to_31_elements():
    """A tensor of 2.15e9 elements (4.3 GB): offsets past 32 bits.  The oracle would take minutes at
    this size, so the check is by parts: with the global scale of the whole tensor given, quantizing
    the two halves separately must give the bytes and scales of the one big call, the global scale
    must be the maximum / 2688, and two sampled row bands must equal the oracle."""
    from ac4k_kernel_amd import _rocm_ops
    R, K = 65536 + 16, 32768
    x = torch.empty((R, K), dtype=torch.bfloat16, device="cuda")
    x.normal_(generator=torch.Generator(device="cuda").manual_seed(5))
    x[R - 3, K - 5] = 37.0  # the maximum sits past the 2^31-th element
    out, sf, gs = ops().quantize(x, 0, 1)
    assert gs.item() == (torch.tensor(37.0, dtype=torch.float32) / 2688.0).item()
    for r0, r1 in ((0, 32768), (32768, R)):
        xo, xs = torch.empty_like(out[r0:r1]), torch.empty_like(sf[:, r0:r1])
        _rocm_ops.quantize_nvfp4(xo, xs, x[r0:r1], gs, 0, 1, False)
        assert torch.equal(xo, out[r0:r1])
        assert torch.equal(xs.view(torch.uint8), sf[:, r0:r1].contiguous().view(torch.uint8))
    for r0 in (0, R - 64):  # 64-row bands against the oracle, global scale of the whole tensor
        band = x[r0:r0 + 64].cpu()
        eo, es, _ = T.quantize_nvfp4(band, 0, 1, False, gs=gs.cpu())
        assert torch.equal(out[r0:r0 + 64].cpu(), eo)
        assert torch.equal(sf[:, r0:r0 + 64].cpu().contiguous().view(torch.uint8), es)
    o8, s8 = ops().quantize(x, 0, 1, precision="fp8e4m3")
    e8, es8 = T.quantize_fp8(x[R - 64:].cpu(), 0, 1)
    assert torch.equal(o8[R - 64:].cpu().view(torch.uint8), e8) and torch.equal(s8[R - 64:].cpu(), es8)
    del x, out, sf, o8, s8
    torch.cuda.empty_cache()


def test_error_behaviour():
    o = ops()
    x = make_input((8, 64), seed=7).cuda()
    with pytest.raises(AssertionError):
        o.quantize(x, 1, 1)
    with pytest.raises(RuntimeError):
        o.quantize(x.float(), 0, 1)                      # not bf16
    with pytest.raises(RuntimeError):
        o.quantize(x.t(), 0, 1)                          # not contiguous
    with pytest.raises(RuntimeError):
        o.quantize(x, 0, 1, output=torch.empty((8, 16), dtype=torch.uint8, device="cuda"))
    with pytest.raises(RuntimeError):
        o.quantize(x, 0, 1, sf=torch.empty((1, 8, 4), dtype=torch.float8_e4m3fn, device="cuda"))
    gs = torch.ones((1,), device="cuda")
    with pytest.raises(RuntimeError):                    # global scale must be 0-dim
        o.quantize_nvfp4(torch.empty((8, 32), dtype=torch.uint8, device="cuda"),
                         torch.empty((1, 16, 4), dtype=torch.float8_e4m3fn, device="cuda"), x, gs, 0, 1, False)


def test_reference_bandwidth_shape_at_full_size():
    """The reference's own quantize shape (test/test_quantize_bandwidth.py:37-38: (1, 75600, 40, 128), nvfp4 with
    cross 1 / reduce 3 and with cross 3 / reduce 1 swizzled) and the fp8 call of its attention wrapper
    (python/ac4k_kernel/ops/attention.py:169-174: cross 3, reduce the token dim, swizzled, max_scale 2.25), at full
    size: 387 M elements.  The global scale must equal the oracle's formula on the tensor's maximum (taken with
    a torch reduction), and bands of the outputs - the first, a middle one and the last, which holds the padding -
    must equal the oracle's bytes; the oracle quantizes the band with the global scale given, which is exact
    because blocks, chunks and swizzle groups do not reach across a band that starts on a multiple of 64."""
    shape = (1, 75600, 40, 128)
    g = torch.Generator(device="cuda").manual_seed(20)
    x = torch.empty(shape, dtype=torch.float32, device="cuda").normal_(generator=g)
    x = torch.where(torch.rand(shape, device="cuda", generator=g) < 0.001, x * 20.0, x).to(torch.bfloat16)
    amax = x.abs().max().reshape(1).cpu()
    gs_ref = T.global_scale(amax)

    # cross 1 (tokens), reduce 3 (head dim): bands of 64 tokens
    out, sf, gs = ops().quantize(x, 1, 3)
    assert gs.item() == gs_ref.item()
    assert list(out.shape) == [1, 40, 75600, 64] and list(sf.shape) == [1, 40, 2, 75600, 4]
    for t0 in (0, 37792, 75600 - 64):
        eo, es, _ = T.quantize_nvfp4(x[:, t0:t0 + 64].cpu(), 1, 3, False, gs=gs_ref)
        assert torch.equal(out[:, :, t0:t0 + 64].cpu(), eo), f"nvfp4 cross 1: bytes of tokens {t0}.. differ"
        assert torch.equal(sf[:, :, :, t0:t0 + 64].cpu().view(torch.uint8), es), f"nvfp4 cross 1: scales of tokens {t0}.. differ"
    del out, sf

    # cross 3 (head dim), reduce 1 (tokens), swizzled: bands of 256 tokens along the reduce dim; the last band
    # ends in the 48 padding positions (75600 -> 75648)
    out, sf, gs = ops().quantize(x, 3, 1, swizzle=True)
    assert gs.item() == gs_ref.item()
    assert list(out.shape) == [1, 40, 128, 75648 // 2] and list(sf.shape) == [1, 40, 1182, 128, 4]
    for k0 in (0, 37760, 75648 - 256):
        eo, es, _ = T.quantize_nvfp4(x[:, k0:k0 + 256].cpu(), 3, 1, True, gs=gs_ref)
        assert torch.equal(out[..., k0 // 2:(k0 + 256) // 2].cpu(), eo), f"nvfp4 cross 3: bytes of tokens {k0}.. differ"
        assert torch.equal(sf[:, :, k0 // 64:(k0 + 256) // 64].cpu().view(torch.uint8), es), f"nvfp4 cross 3: scales of tokens {k0}.. differ"
    del out, sf

    # fp8, cross 3, reduce 1, swizzled, max_scale 2.25: a row is (head, d) over all 75600 tokens, so whole heads are compared
    out, sf = ops().quantize(x, 3, 1, max_scale=2.25, precision="fp8e4m3", swizzle=True)
    assert list(out.shape) == [1, 40, 128, 75600] and list(sf.shape) == [1, 40, 128]
    for h in (0, 17, 39):
        eo, es = T.quantize_fp8(x[:, :, h:h + 1].cpu(), 3, 1, 2.25, True)
        assert torch.equal(out[:, h:h + 1].cpu().view(torch.uint8), eo), f"fp8 cross 3: bytes of head {h} differ"
        assert torch.equal(sf[:, h:h + 1].cpu(), es), f"fp8 cross 3: scales of head {h} differ"
    del out, sf

    # fp8 and int8, cross 1, reduce 3: rows are tokens, bands of 64 tokens
    for prec, orc in (("fp8e4m3", T.quantize_fp8), ("int8", T.quantize_int8)):
        out, sf = ops().quantize(x, 1, 3, precision=prec)
        for t0 in (0, 37792, 75600 - 64):
            eo, es = orc(x[:, t0:t0 + 64].cpu(), 1, 3)
            got = out[:, :, t0:t0 + 64].cpu()
            assert torch.equal(got.view(torch.uint8) if prec == "fp8e4m3" else got, eo), f"{prec} cross 1: tokens {t0}.. differ"
            assert torch.equal(sf[:, :, t0:t0 + 64].cpu(), es)
        del out, sf
    torch.cuda.empty_cache()


def test_single_launch_timeout_is_reported_and_backs_off():
    """A grid wait that runs out is reported to the host through mapped memory; the next calls on that stream
    take the three-launch path (64 of them), then the single launch is tried again.  The condition is forced
    from the host with a bound of 1 us: with it a workgroup looks at the clock on its first poll, more than 1 us
    after its entry, and the first workgroup to get there finds peers missing (the launch stagger alone is longer
    than a poll).  Every kernel still exits normally, and every output equals the oracle's."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    x = make_input((4096, 2048), seed=77, outliers=True)
    exp = T.quantize_nvfp4(x, 0, 1, False)
    xg = x.cuda()

    def run():
        out, sf, gs = ops().quantize(xg, 0, 1)
        path = L.ac4k_debug_last_quantize_path()
        torch.cuda.synchronize()  # the report of this launch has reached host memory before the next call looks
        assert torch.equal(out.cpu(), exp[0]) and torch.equal(sf.cpu().view(torch.uint8), exp[1]) and gs.item() == exp[2].item()
        return path

    try:
        L.ac4k_set_quantize_sync_timeout_us(1)
        seen0 = L.ac4k_debug_quantize_timeouts_seen()
        assert run() == PATH_ONEPASS          # the wait runs out inside this launch: same bits, slower
        paths = [run() for _ in range(64)]    # the report is read before the first of these
        assert L.ac4k_debug_quantize_timeouts_seen() == seen0 + 1
        assert paths == [PATH_TWO_KERNEL] * 64
        assert run() == PATH_ONEPASS          # back-off over: the single launch is tried again
        L.ac4k_set_quantize_sync_timeout_us(200)  # ends the back-off that the last launch caused
        assert run() == PATH_ONEPASS
        assert run() == PATH_ONEPASS          # an idle GPU: nothing to report
    finally:
        L.ac4k_set_quantize_sync_timeout_us(200)


def test_quantize_next_to_a_long_gemm_on_another_stream():
    """The GPU shared with the 8192^3 linear running back to back on a second stream: the quantizer's workgroups
    are not all resident at once, waits may run out, calls may back off to the three-launch path - whatever
    happens, every call returns the oracle's bytes."""
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    L.ac4k_set_quantize_sync_timeout_us(200)
    aq = ops().quantize(make_input((8192, 8192), seed=1).cuda(), 0, 1)
    bq = ops().quantize(make_input((8192, 8192), seed=2).cuda(), 0, 1)
    d = torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda")
    x = make_input((8192, 4096), seed=78, outliers=True)
    exp = T.quantize_nvfp4(x, 0, 1, False)
    xg = x.cuda()
    torch.cuda.synchronize()
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    results, paths = [], []
    with torch.cuda.stream(s1):
        for _ in range(12):
            ops().linear(*aq, *bq, out=d)
    with torch.cuda.stream(s2):
        for _ in range(12):
            results.append(ops().quantize(xg, 0, 1))
            paths.append(L.ac4k_debug_last_quantize_path())
    torch.cuda.synchronize()
    for out, sf, gs in results:
        assert torch.equal(out.cpu(), exp[0]) and torch.equal(sf.cpu().view(torch.uint8), exp[1]) and gs.item() == exp[2].item()
    assert set(paths) <= {PATH_ONEPASS, PATH_TWO_KERNEL}
    L.ac4k_set_quantize_sync_timeout_us(200)

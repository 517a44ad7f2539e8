"""The entry point that allocates nothing (ac4k_linear_nvfp4_skinny_static): through the C ABI, its
output equals ac4k_linear_nvfp4_skinny's bit for bit on the same operands, on calls in a row that
share the library's scratch array (large, then smaller, then another kernel family), and a shape
beyond the array is rejected."""
import pytest
import torch

from conftest import make_input

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 << 20  # AC4K_STATIC_SCRATCH_BYTES of include/ac4k_nvfp4.h


def _operands(m, n, k, seed):
    from ac4k_kernel_amd import ops
    aq = ops.quantize(make_input((m, k), seed=seed, outliers=True).cuda(), 0, 1)
    bq = ops.quantize(make_input((n, k), seed=seed + 1, std=0.02).cuda(), 0, 1)
    return aq, bq


def _both(L, lib, m, n, k, seed, d_tag, dtype, bias_dtype=None):
    aq, bq = _operands(m, n, k, seed)
    bias = None if bias_dtype is None else make_input((1, n), seed=seed + 2).to(bias_dtype).cuda()
    btag = {None: 0, torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}[bias_dtype]
    need = L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k)
    assert 0 < need <= STATIC_BYTES, (m, n, k, need)
    ws = torch.empty(need, dtype=torch.uint8, device="cuda")
    ref = torch.full((m, n), 7.0, dtype=dtype, device="cuda")
    got = torch.full((m, n), -7.0, dtype=dtype, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    args = (aq[0].data_ptr(), aq[1].data_ptr(), aq[2].data_ptr(), bq[0].data_ptr(), bq[1].data_ptr(), bq[2].data_ptr(),
            None if bias is None else bias.data_ptr(), btag, m, n, k)
    lib.check(L.ac4k_linear_nvfp4_skinny(ref.data_ptr(), d_tag, *args, ws.data_ptr(), need, st))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    lib.check(L.ac4k_linear_nvfp4_skinny_static(got.data_ptr(), d_tag, *args, st))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(got, ref), f"M={m} N={n} K={k}: {(got != ref).sum().item()} outputs differ"
    return got


def test_static_scratch_entry_equals_workspace_entry(linear_tuning):
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    # decode-sized through the register kernel (forced: it splits K eight ways here), nearly the whole
    # array (29.4 MB of partial sums), then a smaller input right behind it
    linear_tuning(decode_kernel=1)
    _both(L, _lib, 32, 28672, 8192, 1, 0, torch.bfloat16)
    linear_tuning()
    _both(L, _lib, 8, 1024, 2048, 4, 0, torch.bfloat16, torch.float32)
    # the LDS-ring kernel with a K split (few tiles)
    _both(L, _lib, 20, 1024, 4096, 5, 0, torch.bfloat16, torch.float32)
    # the split-K tile family through the same array, then decode-sized again, fp32 output
    _both(L, _lib, 128, 1024, 4096, 7, 2, torch.float32, torch.bfloat16)
    _both(L, _lib, 1, 4096, 14336, 10, 1, torch.float16)
    _both(L, _lib, 8, 1024, 2048, 4, 0, torch.bfloat16, torch.float32)


def test_static_scratch_entry_rejects_what_does_not_fit():
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    m, n, k = 7, 8 * 28672, 8192  # the register kernel's eight K slices: 51.4 MB of partial sums
    assert L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k) > STATIC_BYTES
    one = torch.zeros(64, dtype=torch.uint8, device="cuda").data_ptr()  # never reached: the size check comes first
    rc = L.ac4k_linear_nvfp4_skinny_static(one, 0, one, one, one, one, one, one, None, 0, m, n, k, None)
    assert rc != 0 and b"static scratch holds" in L.ac4k_last_error()
    # shapes that take no scratch are refused like ac4k_linear_nvfp4_skinny refuses them
    rc = L.ac4k_linear_nvfp4_skinny_static(one, 0, one, one, one, one, one, one, None, 0, 8192, 8192, 8192, None)
    assert rc != 0 and b"no workspace-assisted path" in L.ac4k_last_error()


def test_static_scratch_entry_under_graph_capture(linear_tuning):
    """The callers the entry point is for: a decode step captured into a HIP graph (quantize, then the
    linear on the library's own scratch; no allocation inside the capture), replayed on fresh activations
    with eager work in between, equals the eager result every time.  A shape that splits K is used, so
    the replays really go through the scratch array."""
    from ac4k_kernel_amd import _lib, _rocm_ops, ops
    L = _lib.load()
    m, n, k = 4, 1024, 4096
    need = L.ac4k_linear_nvfp4_skinny_workspace_bytes(m, n, k)
    assert 256 < need <= STATIC_BYTES  # more than the marker value: partial sums go through the scratch
    wq = ops.quantize(make_input((n, k), seed=91, std=0.02).cuda(), 0, 1)
    x_static = make_input((m, k), seed=92).cuda()
    xq = ops.quantize(x_static, 0, 1)  # output buffers of the captured quantize
    d_static = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda")
    d_eager = torch.zeros_like(d_static)
    st = lambda: torch.cuda.current_stream().cuda_stream  # noqa: E731

    def linear_static(dst):
        _lib.check(L.ac4k_linear_nvfp4_skinny_static(dst.data_ptr(), 0, xq[0].data_ptr(), xq[1].data_ptr(),
                                                     xq[2].data_ptr(), wq[0].data_ptr(), wq[1].data_ptr(),
                                                     wq[2].data_ptr(), None, 0, m, n, k, st()))

    linear_static(d_eager)  # first call on this GPU outside capture: it looks up the array's address
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _rocm_ops.quantize_nvfp4_with_global_scale(xq[0], xq[1], xq[2], x_static, 0, 1, False, 2688.0)
        linear_static(d_static)
    for seed in (101, 102, 103):
        x = make_input((m, k), seed=seed, outliers=True).cuda()
        x_static.copy_(x)
        graph.replay()
        torch.cuda.synchronize()
        got = d_static.clone()
        ref = ops.linear(*ops.quantize(x, 0, 1), *wq)  # eager work between the replays, and the expected value
        assert torch.equal(got, ref), f"replay with seed {seed}: {(got != ref).sum().item()} outputs differ"

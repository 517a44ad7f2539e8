#!/usr/bin/env python3
"""Benchmark of the NVFP4 path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload all|linear|quantize|traffic|quantize-timeline|linear-timeline]
                    [--no-cpu-baseline] [--no-check]

Prints ONE JSON line.  The headline `value` is the NVFP4 linear at M=N=K=8192 (the
north-star GEMM, also the first shape of the reference's test/test_linear_tflops.py:189)
in TFLOP/s = 2*M*N*K / t, with the operands already quantized and resident in HBM.  The
same line carries, under "quantize", the BF16->NVFP4 / FP8 / INT8 quantizers on the
8192x4096 outlier activations and the 4096x4096 case (GB/s = (in + out + sf bytes) / t as
in test/test_quantize_bandwidth.py:32-33, whole quantize() call, three rotating input
buffers), under "linear_shapes" the other GEMM configurations and under "decode" the fused
decode-sized linear.

oracle/ is used by the CPU leg of the run only: the oracle is timed on the host cores as
`cpu_baseline`, and the same oracle checks the quantizers' GPU output of the same inputs bit
for bit (`bit_exact_vs_oracle`); --no-cpu-baseline skips both.  The GEMM check compares with an
fp32 dequantize-matmul made of torch ops on the GPU.  Nothing that is timed on the GPU calls the
oracle.

A "step" is one pass of the timed op over one batch of synthetic input.  Timing uses
events recorded on the stream the kernels are launched on (torch's current stream, which
is the stream handed to the C ABI).  `roofline.traffic` is not measured live: it is the HBM
byte count per launch taken from the rocprofv3 --pmc summaries in profiles/traffic.json
(made with `--workload traffic`, see profiles/).
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HOST = {}                   # host core counts of the CPU leg, filled in main()
HBM_PEAK_GBS = 8000.0       # MI355X HBM3E
MFMA_PEAK_TFLOPS = 2500.0   # MI355X dense fp16 / bf16 MFMA (identical rates)


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def make_input(shape, seed=0, outliers=False, std=1.0):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32) * std
    if outliers:
        x = torch.where(torch.rand(shape, generator=g) < 0.001, x * 20.0, x)
    return x.to(torch.bfloat16)


SETTLE_MS = 150.0  # see time_gpu; --settle-ms


def time_gpu(fn, steps, warmup):
    """-> (total ms over `steps` calls, ms per call); events on the launch stream.

    `warmup` untimed calls come first.  Then the untimed calls go on until the GPU has been under
    this load for SETTLE_MS of wall time: the clock governor of the box ramps up over the first
    40 ms or so of sustained work (the 8192^3 linear goes from 1.2 ms for the first calls to a steady
    0.77 ms), and a run of a few dozen steps would time the ramp, not the kernel."""
    import time
    t0 = time.perf_counter()
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    while (time.perf_counter() - t0) * 1e3 < SETTLE_MS:
        for _ in range(max(1, warmup)):
            fn()
        torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    end.record()
    torch.cuda.synchronize()
    total = start.elapsed_time(end)
    return total, total / steps


def measured_traffic(key):
    try:
        with open(os.path.join(ROOT, "profiles", "traffic.json")) as f:
            return json.load(f).get(key)
    except (OSError, ValueError):
        return None


def roofline(bound, achieved, traffic_key=None):
    peak, unit = (HBM_PEAK_GBS, "GB/s") if bound == "hbm" else (MFMA_PEAK_TFLOPS, "TFLOP/s")
    return {"bound": bound, "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
            "traffic": measured_traffic(traffic_key) if traffic_key else None}


# --------------------------------------------------------------------------- quantize
def quant_bytes(shape_rk, precision):
    R, K = shape_rk
    if precision == "nvfp4":
        Kp, Rp = (K + 63) // 64 * 64, (R + 15) // 16 * 16
        return 2 * R * K + R * Kp // 2 + (Kp // 64) * Rp * 4 + 4
    Kp, Rp = (K + 15) // 16 * 16, (R + 15) // 16 * 16
    return 2 * R * K + R * Kp + 4 * Rp


MALL_BYTES = 256 << 20  # memory-side cache of the MI355X


def bench_quantize(ops, shape, precision, steps, warmup, outliers, check=True, nbuf=None, key=None):
    """`check`: the CPU leg of the run compares the GPU output of the first input with the oracle's, bit for bit.
    The headline rotates over enough (input, output) buffer sets that a set is evicted from the 256 MB
    memory-side cache before its turn comes again (their bytes together exceed twice the cache): every call
    reads its input from HBM.  The same call over three sets, which fit the cache, is reported beside it."""
    nbytes = quant_bytes(shape, precision)
    if nbuf is None:
        nbuf = max(3, -(-2 * MALL_BYTES // nbytes) + 1)
    xs_cpu = [make_input(shape, seed=s, outliers=outliers) for s in range(min(nbuf, 3))]
    xs = [x.cuda() for x in xs_cpu]
    xs += [xs[i % 3].clone() for i in range(nbuf - len(xs))]  # distinct memory, same values as the first three
    res = ops.quantize(xs[0], 0, 1, precision=precision)
    outs = [[torch.empty_like(t) for t in res[:2]] for _ in range(nbuf)]
    ok = None
    if check:
        from oracle import nvfp4_oracle as T
        if precision == "nvfp4":
            e = T.quantize_nvfp4(xs_cpu[0], 0, 1)
            ok = (torch.equal(res[0].cpu(), e[0]) and torch.equal(res[1].cpu().view(torch.uint8), e[1])
                  and res[2].item() == e[2].item())
        elif precision == "fp8e4m3":
            e = T.quantize_fp8(xs_cpu[0], 0, 1)
            ok = torch.equal(res[0].cpu().view(torch.uint8), e[0]) and torch.equal(res[1].cpu(), e[1])
        else:
            e = T.quantize_int8(xs_cpu[0], 0, 1)
            ok = torch.equal(res[0].cpu(), e[0]) and torch.equal(res[1].cpu(), e[1])
    i = [0]
    rot = [nbuf]

    def step():
        j = i[0] % rot[0]
        i[0] += 1
        ops.quantize(xs[j], 0, 1, precision=precision, output=outs[j][0], sf=outs[j][1])

    _, ms = time_gpu(step, steps, warmup)
    gbs = nbytes / (ms * 1e-3) / 1e9
    rot[0] = 3
    _, ms3 = time_gpu(step, steps, warmup)
    rot[0] = nbuf
    r = {"workload": f"quantize {precision} {shape[0]}x{shape[1]} bf16" + (" outliers" if outliers else ""),
         "ms": ms, "bytes": nbytes, "GB/s": gbs, "bit_exact_vs_oracle": ok,
         "roofline": roofline("hbm", gbs, key), "rotating_buffers": nbuf, "rotating_bytes": nbuf * nbytes,
         "input_from": "HBM (the rotation exceeds twice the 256 MB memory-side cache)",
         "three_buffers_cache_assisted": {"ms": ms3, "GB/s": nbytes / (ms3 * 1e-3) / 1e9,
                                          "frac_of_hbm_peak": nbytes / (ms3 * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                          "rotating_bytes": 3 * nbytes}}
    if precision == "nvfp4":  # the quantize kernel alone, its global scale already on the device
        from ac4k_kernel_amd import _rocm_ops
        gss = [ops.quantize(x, 0, 1)[2] for x in xs]

        def kernel_only():
            j = i[0] % nbuf
            i[0] += 1
            _rocm_ops.quantize_nvfp4(outs[j][0], outs[j][1], xs[j], gss[j], 0, 1, False)

        i[0] = 0
        kernel_only()
        same = torch.equal(outs[0][0], res[0]) and torch.equal(outs[0][1].view(torch.uint8), res[1].view(torch.uint8))
        i[0] = 0
        _, kms = time_gpu(kernel_only, steps, warmup)
        r["global_scale_given"] = {"ms": kms, "GB/s": (nbytes - 4) / (kms * 1e-3) / 1e9,
                                   "frac_of_hbm_peak": (nbytes - 4) / (kms * 1e-3) / 1e9 / HBM_PEAK_GBS,
                                   "equals_whole_op_output": same}
    return r


def cpu_quantize_baseline(shape, outliers, budget_s=10.0):
    """The torch oracle on the host cores: whole quantizes of one tensor, repeated for about
    `budget_s` seconds (at least three), median time."""
    from oracle import nvfp4_oracle as T
    x = make_input(shape, seed=0, outliers=outliers)
    T.quantize_nvfp4(x[:256], 0, 1)
    ts, t_begin = [], time.perf_counter()
    while len(ts) < 3 or time.perf_counter() - t_begin < budget_s:
        t0 = time.perf_counter()
        T.quantize_nvfp4(x, 0, 1)
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[len(ts) // 2]
    return {"value": quant_bytes(shape, "nvfp4") / t / 1e9, "unit": "GB/s", "cores": torch.get_num_threads(),
            "host": dict(HOST), "kind": "port",
            "sample": f"full nvfp4 quantize of one {shape[0]}x{shape[1]} bf16 tensor, median of {len(ts)} runs "
                      f"({time.perf_counter() - t_begin:.0f} s)"}


# --------------------------------------------------------------------------- linear
# the sixteen E2M1 codes (test/test_linear_bench.py:18-35 of the reference holds the same table)
E2M1_VALUES = [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0]


def gpu_dequant(q, rows):
    """fp32 dequantization of a packed operand with torch ops on the GPU (the GEMM check's reference)."""
    packed, sf, gs = q
    lut = torch.tensor(E2M1_VALUES, dtype=torch.float32, device="cuda")
    v = torch.stack((lut[(packed & 0xF).long()], lut[(packed >> 4).long()]), dim=-1).reshape(rows, -1, 16)
    s = sf.permute(1, 0, 2).reshape(sf.shape[1], -1)[:rows].float() * gs
    return (v * s.unsqueeze(-1)).reshape(rows, -1)


def linear_bytes(m, n, k):
    return (m + n) * k // 2 + ((m + 15) // 16 * 16 + (n + 15) // 16 * 16) * k // 16 + m * n * 2 + 8


def bench_linear(ops, m, n, k, steps, warmup, wstd=1.0, check=True, key=None, with_quantize=False, gen_on_gpu=False,
                 with_image=False):
    if gen_on_gpu:  # very large operands: the host generator would take longer than the measurement
        g = torch.Generator(device="cuda").manual_seed(0)
        a = torch.empty((m, k), dtype=torch.float32, device="cuda").normal_(generator=g).to(torch.bfloat16)
        b = (torch.empty((n, k), dtype=torch.float32, device="cuda").normal_(generator=g) * wstd).to(torch.bfloat16)
    else:
        a, b = make_input((m, k), seed=0), make_input((n, k), seed=1, std=wstd)
    aq, bq = ops.quantize(a.cuda(), 0, 1), ops.quantize(b.cuda(), 0, 1)
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    ops.linear(*aq, *bq, out=out)
    ok = None
    if check:  # fp32 dequantize-matmul on a row sample, atol = rtol = 1e-2
        rows = torch.arange(0, m, max(1, m // 128), device="cuda")
        ref = (gpu_dequant(aq, m)[rows] @ gpu_dequant(bq, n).t()).to(torch.bfloat16)
        got = out[rows]
        ok = bool(torch.all((got.float() - ref.float()).abs() <= 1e-2 + 1e-2 * ref.float().abs()).item())
        del ref
    # memory-bound shapes rotate over enough copies of the weight operand to exceed the 256 MB
    # memory-side cache, so that the weights really come from HBM (as distinct layers' weights would)
    t_flops0, t_bytes0 = 2.0 * m * n * k / (MFMA_PEAK_TFLOPS * 1e12), linear_bytes(m, n, k) / (HBM_PEAK_GBS * 1e9)
    wbytes = bq[0].nbytes + bq[1].nbytes
    ncopy = 1 if t_flops0 >= t_bytes0 else max(2, min(12, -(-320_000_000 // wbytes)))
    bqs = [bq] + [tuple(t.clone() for t in bq) for _ in range(ncopy - 1)]
    turn = [0]

    def weights():
        turn[0] += 1
        return bqs[turn[0] % ncopy]

    total, ms = time_gpu(lambda: ops.linear(*aq, *weights(), out=out), steps, warmup)
    ms_with_quantize = None
    if with_quantize:  # the activation quantized inside the timed region, the weights not
        xa = a.cuda()
        if m <= 32 and k % 64 == 0:  # decode-sized: the fused entry point (one C call) is the product's path
            _, ms_with_quantize = time_gpu(lambda: ops.fused_linear(xa, *weights(), out=out), steps, warmup)
        else:
            _, ms_with_quantize = time_gpu(lambda: ops.linear(*ops.quantize(xa, 0, 1), *weights(), out=out), steps, warmup)
        del xa
    image = None
    if with_image and k % 128 == 0:  # the same linear on pre-packed weight images of the same weights
        imgs = [ops.prepack_weight(w[0], w[1]) for w in bqs]
        out_i = torch.empty_like(out)
        ops.linear_prepacked(*aq, imgs[0], bq[2], out=out_i)
        ops.linear(*aq, *bq, out=out)
        same = bool(torch.equal(out, out_i))
        _, ms_i = time_gpu(lambda: (turn.__setitem__(0, turn[0] + 1),
                                    ops.linear_prepacked(*aq, imgs[turn[0] % ncopy], bq[2], out=out_i)), steps, warmup)
        _, ms_p = time_gpu(lambda: ops.linear(*aq, *weights(), out=out), steps, warmup)  # plain layout again, after it
        image = {"ms": ms_i, "plain_layout_ms_before": ms, "plain_layout_ms_after": ms_p,
                 "bit_identical_to_plain_layout": same,
                 "TFLOP/s": 2.0 * m * n * k / (ms_i * 1e-3) / 1e12, "GB/s": linear_bytes(m, n, k) / (ms_i * 1e-3) / 1e9}
        del imgs, out_i
    del bqs
    tflops = 2.0 * m * n * k / (ms * 1e-3) / 1e12
    gbs = linear_bytes(m, n, k) / (ms * 1e-3) / 1e9
    t_flops, t_bytes = 2.0 * m * n * k / (MFMA_PEAK_TFLOPS * 1e12), linear_bytes(m, n, k) / (HBM_PEAK_GBS * 1e9)
    rl = roofline("mfma", tflops, key) if t_flops >= t_bytes else roofline("hbm", gbs, key)
    return {"workload": f"NVFP4 linear M={m} N={n} K={k}, bf16 out, operands pre-quantized", "ms": ms,
            "total_ms": total, "TFLOP/s": tflops, "GB/s": gbs, "within_1e-2_of_fp32_dequant_matmul": ok,
            "roofline": rl, "ms_with_activation_quantize": ms_with_quantize, "rotating_weight_copies": ncopy,
            "weight_image": image}


def _read_sclk_mhz():
    """Current shader clock in MHz as the driver reports it: the starred line of pp_dpm_sclk in sysfs,
    else what `rocm-smi --showclocks` prints (run as a child process); None when neither is readable."""
    import glob
    import re
    import subprocess
    for path in sorted(glob.glob("/sys/class/drm/card*/device/pp_dpm_sclk")):
        try:
            for ln in open(path).read().splitlines():
                m = re.search(r"(\d+)\s*Mhz\s*\*", ln, re.I)
                if m:
                    return float(m.group(1)), "sysfs pp_dpm_sclk"
        except OSError:
            pass
    try:
        r = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20)
        for ln in r.stdout.splitlines():
            m = re.search(r"sclk clock level.*\((\d+)\s*Mhz\)", ln, re.I)
            if m:
                return float(m.group(1)), "rocm-smi --showclocks"
    except (OSError, subprocess.SubprocessError):
        pass
    return None, None


def shader_clock_under_load(ops, n=8192, seconds=1.5):
    """Shader clock while the n^3 NVFP4 linear runs back to back (outside every timed region): a host
    thread keeps the queue full, the main thread samples the driver's clock read-out.  The roofline
    peak assumes 2.4 GHz; this is the clock the power limit leaves the kernel."""
    import threading
    idle, src = _read_sclk_mhz()
    if src is None:
        return {"under_load_mhz": None, "before_mhz": None, "source": None, "assumed_by_peak_mhz": 2400}
    aq = ops.quantize(make_input((n, n), seed=0).cuda(), 0, 1)
    bq = ops.quantize(make_input((n, n), seed=1).cuda(), 0, 1)
    out = torch.empty((n, n), dtype=torch.bfloat16, device="cuda")
    stop = [False]

    def work():
        while not stop[0]:
            for _ in range(50):
                ops.linear(*aq, *bq, out=out)
            torch.cuda.synchronize()

    th = threading.Thread(target=work)
    th.start()
    samples = []
    try:
        time.sleep(0.6 * seconds)
        for _ in range(3):
            samples.append(_read_sclk_mhz()[0])
            time.sleep(0.13 * seconds)
    finally:
        stop[0] = True
        th.join()
    samples = sorted(x for x in samples if x is not None)
    return {"under_load_mhz": samples[len(samples) // 2] if samples else None, "before_mhz": idle, "source": src,
            "assumed_by_peak_mhz": 2400, "workload": f"NVFP4 linear M=N=K={n} back to back"}


def vendor_gemm_yardstick(steps, warmup, n=8192):
    """What the vendor library's dense 16-bit GEMM (torch.matmul) sustains on this box at n^3: not part
    of the product and not a baseline of the metric (its operands are dense fp16/bf16, nothing is
    decoded), only a measure of how far the 2.5 PFLOP/s peak is reachable at this box's clocks."""
    res = {"workload": f"torch.matmul M=N=K={n}, dense operands"}
    for name, dt in (("bf16", torch.bfloat16), ("fp16", torch.float16)):
        a = torch.randn((n, n), device="cuda", dtype=dt)
        b = torch.randn((n, n), device="cuda", dtype=dt)
        _, ms = time_gpu(lambda: torch.matmul(a, b.t()), steps, warmup)
        res[f"{name}_TFLOP/s"] = 2.0 * n ** 3 / (ms * 1e-3) / 1e12
        del a, b
    return res


def bench_decode(ops, m, n, k, steps, warmup, check=True, ncopy=3, key=None):
    """Fused decode-sized linear: bf16 activation in, on-the-fly NVFP4 quantize + GEMM.  The calls
    rotate over `ncopy` copies of the weights (3 x 132 MB: more than the 256 MB memory-side cache holds),
    so that the weights are streamed from HBM."""
    x = make_input((m, k), seed=2, outliers=True).cuda()
    wq = ops.quantize(make_input((n, k), seed=3, std=0.02).cuda(), 0, 1)
    wqs = [wq] + [tuple(t.clone() for t in wq) for _ in range(ncopy - 1)]
    out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
    ops.fused_linear(x, *wq, out=out)
    ok = None
    if check:
        ref = ops.linear(*ops.quantize(x, 0, 1), *wq)
        ok = bool(torch.all((out.float() - ref.float()).abs() <= 1e-2 + 1e-2 * ref.float().abs()).item())
    turn = [0]

    def step():
        turn[0] += 1
        ops.fused_linear(x, *wqs[turn[0] % ncopy], out=out)

    _, ms = time_gpu(step, steps, warmup)
    nbytes = n * k // 2 + n * k // 16 + 2 * m * k + 2 * m * n
    gbs = nbytes / (ms * 1e-3) / 1e9
    return {"workload": f"fused decode linear M={m} N={n} K={k} (bf16 activation quantized on the fly)", "ms": ms,
            "bytes": nbytes, "GB/s": gbs, "equals_quantize_then_linear_within_1e-2": ok,
            "roofline": roofline("hbm", gbs, key), "rotating_weight_copies": ncopy}


def bench_quantize_layouts(ops, steps, warmup):
    """Quantizer layouts beyond (cross 0, reduce 1): the two calls of the reference's bandwidth test
    (test/test_quantize_bandwidth.py:37-38, shape (1, 75600, 40, 128)) for nvfp4 and fp8, and the
    swizzled row-major case.  Bytes = input + output + scales, the input counted once."""
    res = {}
    g = torch.Generator(device="cpu").manual_seed(4)
    x = torch.randn((1, 75600, 40, 128), generator=g, dtype=torch.float32).to(torch.bfloat16).cuda()
    y = make_input((8192, 4096), seed=0, outliers=True).cuda()
    cases = (("attn_cross1_reduce3", x, 1, 3, False), ("attn_cross3_reduce1_swizzle", x, 3, 1, True),
             ("rowmajor_8192x4096_swizzle", y, 0, 1, True))
    for name, t, cross, red, swz in cases:
        for prec in ("nvfp4", "fp8e4m3"):
            r = ops.quantize(t, cross, red, precision=prec, swizzle=swz)
            o, sf = r[0], r[1]
            _, ms = time_gpu(lambda: ops.quantize(t, cross, red, precision=prec, swizzle=swz, output=o, sf=sf),
                             steps, warmup)
            nbytes = t.nbytes + o.nbytes + sf.nbytes
            res[f"{name}_{prec}"] = {"shape": list(t.shape), "cross_dim": cross, "reduce_dim": red, "swizzle": swz,
                                     "ms": ms, "GB/s": nbytes / (ms * 1e-3) / 1e9}
            del r, o, sf
    return res


def bench_attention(ops, B, N, H, D, steps, warmup, check=True, precision="nvfp4"):
    """Attention forward, precision "nvfp4" or "int8+fp8e4m3": flops = 4 B H N^2 D as in
    the reference's test/test_attention_tflops.py:31-33; the kernel alone on pre-quantized operands and the whole
    attention() call (its quantizers + kernel).  Check: cosine similarity and elementwise distance to torch's
    scaled_dot_product_attention on the GPU, at the tolerance of test/test_attention_bench.py:19-66 (nvfp4: cosine
    0.98, atol 0.2, rtol 0.1; int8+fp8e4m3: cosine 0.99, atol 0.2, rtol 0.01)."""
    import importlib
    import math
    g = torch.Generator(device="cuda").manual_seed(7)
    q, k, v = (torch.empty((B, N, H, D), dtype=torch.float32, device="cuda").normal_(generator=g).to(torch.bfloat16)
               for _ in range(3))
    out = torch.empty((B, N, H, D), dtype=torch.bfloat16, device="cuda")
    ops.attention(q, k, v, layout="BNHD", precision=precision, out=out)
    ok = cos = None
    if check:
        ref = torch.nn.functional.scaled_dot_product_attention(q.transpose(1, 2).float(), k.transpose(1, 2).float(),
                                                               v.transpose(1, 2).float()).transpose(1, 2)
        cos = torch.nn.functional.cosine_similarity(out.float().flatten(), ref.flatten(), dim=0).item()
        rtol, stol = (1e-1, 0.98) if precision == "nvfp4" else (1e-2, 0.99)
        inside = ((out.float() - ref).abs() <= 2e-1 + rtol * ref.abs()).float().mean().item()
        ok = bool(cos > stol and inside > 0.999)
        del ref
    o_bhnd = out.permute(0, 2, 1, 3)
    if precision == "nvfp4":
        qq, kq, vq = ops.quantize(q, 1, 3), ops.quantize(k, 1, 3), ops.quantize(v, 3, 1, swizzle=True)
        kernel = lambda: ops.mha_nvfp4_fwd(o_bhnd, *qq, *kq, *vq, 1.0 / math.sqrt(D))  # noqa: E731
    else:
        front = importlib.import_module("ac4k_kernel_amd.ops.attention")
        q8, q_sf = front._int8_quantize(q, "BNHD", 1, BLOCK_SIZE=64)
        k8, k_sf = front._int8_quantize(k - k.mean(dim=1, keepdim=True), "BNHD", 1, BLOCK_SIZE=128)
        v8, v_sf = ops.quantize(v, 3, 1, swizzle=True, max_scale=2.25, precision="fp8e4m3")
        kernel = lambda: ops.mha_int8_x_fp8_fwd(o_bhnd, q8, q_sf, 64, k8, k_sf, 128, v8, v_sf, 1.0 / math.sqrt(D))  # noqa: E731
    _, ms_k = time_gpu(kernel, steps, warmup)
    _, ms_a = time_gpu(lambda: ops.attention(q, k, v, layout="BNHD", precision=precision, out=out), steps, warmup)
    flops = 4.0 * B * H * N * N * D
    name = "NVFP4" if precision == "nvfp4" else "INT8 x FP8"
    rl = roofline("mfma", flops / (ms_k * 1e-3) / 1e12)
    if precision != "nvfp4":  # both products on 8-bit MFMAs: int8 and fp8 dense peaks are 5.0 P(FL)OP/s
        rl.update(peak=5000.0, frac=rl["achieved"] / 5000.0)
    return {"workload": f"{name} attention forward B={B} N={N} H={H} D={D}, bf16 in / out", "kernel_ms": ms_k,
            "kernel_TFLOP/s": flops / (ms_k * 1e-3) / 1e12, "with_quantize_ms": ms_a,
            "with_quantize_TFLOP/s": flops / (ms_a * 1e-3) / 1e12, "cosine_vs_fp32_attention": cos,
            "within_reference_tolerance_of_fp32_attention": ok,
            "roofline": rl}


def bench_linear_epilogues(ops, steps, warmup, n=8192):
    """Output dtype x bias matrix of the linear (test/test_linear_bench.py:178-205) at n^3."""
    a, b = make_input((n, n), seed=0).cuda(), make_input((n, n), seed=1).cuda()
    aq, bq = ops.quantize(a, 0, 1), ops.quantize(b, 0, 1)
    del a, b
    res = {}
    for od in (torch.bfloat16, torch.float16, torch.float32):
        for bd in (None, torch.bfloat16, torch.float32):
            out = torch.empty((n, n), dtype=od, device="cuda")
            bias = None if bd is None else torch.randn((1, n), device="cuda").to(bd)
            _, ms = time_gpu(lambda: ops.linear(*aq, *bq, bias=bias, out=out), steps, warmup)
            name = f"out_{str(od).split('.')[-1]}_bias_{'none' if bd is None else str(bd).split('.')[-1]}"
            res[name] = {"ms": ms, "TFLOP/s": 2.0 * n ** 3 / (ms * 1e-3) / 1e12}
            del out
    return res


def cpu_linear_baseline(n, k, rows=8192, budget_s=10.0):
    """fp32 dequantize-then-matmul of the oracle on the whole 8192^3 problem, repeated for about
    `budget_s` seconds of host work (at least three runs), median time."""
    from oracle import nvfp4_oracle as T
    a, b = make_input((rows, k), seed=0), make_input((n, k), seed=1)
    aq, bq = T.quantize_nvfp4(a, 0, 1), T.quantize_nvfp4(b, 0, 1)
    del a, b
    ts, t_begin = [], time.perf_counter()
    while len(ts) < 3 or time.perf_counter() - t_begin < budget_s:
        t0 = time.perf_counter()
        T.linear_nvfp4(*aq, *bq)
        ts.append(time.perf_counter() - t0)
    t = sorted(ts)[len(ts) // 2]
    return {"value": 2.0 * rows * n * k / t / 1e12, "unit": "TFLOP/s", "cores": torch.get_num_threads(),
            "host": dict(HOST), "kind": "port",
            "sample": f"oracle fp32 dequantize + torch.matmul of the whole M={rows} N={n} K={k} problem, median of "
                      f"{len(ts)} runs ({time.perf_counter() - t_begin:.0f} s)"}


def run_traffic(ops):
    """A few launches of each hot kernel after a plain device copy of known size, for
    `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE` (the copy calibrates the counters)."""
    src = torch.empty((1 << 28,), dtype=torch.uint8, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(3):
        dst.copy_(src)  # 256 MiB read + 256 MiB written
    a = make_input((8192, 8192), seed=0).cuda()
    aq, bq = ops.quantize(a, 0, 1), ops.quantize(make_input((8192, 8192), seed=1).cuda(), 0, 1)
    out = torch.empty((8192, 8192), dtype=torch.bfloat16, device="cuda")
    for _ in range(3):
        ops.linear(*aq, *bq, out=out)
    img = ops.prepack_weight(bq[0], bq[1])
    for _ in range(3):
        ops.linear_prepacked(*aq, img, bq[2], out=out)
    del aq, bq, out, img, a
    # decode-sized kernels: configuration 5 at M = 1 / 8 / 32 and configuration 4 at M = 16, linear alone
    # (activation already quantized), then the same on weight images; the kernels are told apart by
    # their names and grids in the counter output
    for (n, k, ms_) in ((28672, 8192, (1, 8, 32)), (14336, 4096, (16,))):
        wq = ops.quantize(make_input((n, k), seed=3, std=0.02).cuda(), 0, 1)
        wimg = ops.prepack_weight(wq[0], wq[1])
        for m in ms_:
            xq = ops.quantize(make_input((m, k), seed=2).cuda(), 0, 1)
            o = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
            for _ in range(3):
                ops.linear(*xq, *wq, out=o)
            for _ in range(3):
                ops.linear_prepacked(*xq, wimg, wq[2], out=o)
        del wq, wimg
    # configuration 4 at M = 128: the K-split-waves kernel (one launch at N = 14336, K ranges + reduce at N = 4096)
    for (n, k) in ((14336, 4096), (4096, 14336)):
        wq = ops.quantize(make_input((n, k), seed=3, std=0.02).cuda(), 0, 1)
        xq = ops.quantize(make_input((128, k), seed=2).cuda(), 0, 1)
        o = torch.empty((128, n), dtype=torch.bfloat16, device="cuda")
        for _ in range(3):
            ops.linear(*xq, *wq, out=o)
        del wq, xq, o
    # attention kernel on pre-quantized operands, B = 1, N = 8192, H = 40, D = 128
    import math
    g = torch.Generator(device="cuda").manual_seed(7)
    q, k_, v = (torch.empty((1, 8192, 40, 128), dtype=torch.float32, device="cuda").normal_(generator=g).to(torch.bfloat16)
                for _ in range(3))
    qq, kq, vq = ops.quantize(q, 1, 3), ops.quantize(k_, 1, 3), ops.quantize(v, 3, 1, swizzle=True)
    o = torch.empty((1, 40, 8192, 128), dtype=torch.bfloat16, device="cuda")
    for _ in range(3):
        ops.mha_nvfp4_fwd(o, *qq, *kq, *vq, 1.0 / math.sqrt(128))
    # the int8 x fp8 attention kernel on the same tensors, with its quantizers in front
    import importlib
    front = importlib.import_module("ac4k_kernel_amd.ops.attention")
    q8, q_sf = front._int8_quantize(q, "BNHD", 1, BLOCK_SIZE=64)
    k8, k_sf = front._int8_quantize(k_, "BNHD", 1, BLOCK_SIZE=128)
    v8, v_sf = ops.quantize(v, 3, 1, swizzle=True, max_scale=2.25, precision="fp8e4m3")
    for _ in range(3):
        ops.mha_int8_x_fp8_fwd(o, q8, q_sf, 64, k8, k_sf, 128, v8, v_sf, 1.0 / math.sqrt(128))
    del q, k_, v, qq, kq, vq, o, q8, k8, v8
    x = make_input((8192, 4096), seed=0, outliers=True).cuda()
    for prec in ("nvfp4", "fp8e4m3", "int8"):
        for _ in range(3):
            ops.quantize(x, 0, 1, precision=prec)
    torch.cuda.synchronize()
    print(json.dumps({"traffic_run": "done"}))


def run_quantize_timeline(ops, reps=20):
    """Phase boundaries of the single-launch nvfp4 quantizer from clock stamps inside the kernel
    (needs the library built by `python ac4k_kernel_amd/build.py --timeline`, loaded through
    AC4K_NVFP4_LIB).  Per phase: microseconds after the first workgroup's entry, over all
    workgroups (min / mean / max), median over `reps` isolated launches."""
    import ctypes
    import statistics
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    fn = getattr(L, "ac4k_debug_onepass_timeline", None)
    if fn is None:
        sys.exit("bench.py: this library has no clock stamps; build with `python ac4k_kernel_amd/build.py --timeline` "
                 "and set AC4K_NVFP4_LIB to the library it prints")
    fn.restype, fn.argtypes = ctypes.c_int, [ctypes.c_void_p]
    names = ["entry", "loads_done_own_max", "global_max_known", "nibbles_stored", "scales_stored"]
    res = {}
    for tag, shape, outl in (("cfg1_4096x4096", (4096, 4096), False), ("cfg2_8192x4096", (8192, 4096), True)):
        # enough buffer sets that each one has left the memory-side cache before its next turn (see bench_quantize)
        nb = max(3, -(-2 * MALL_BYTES // quant_bytes(shape, "nvfp4")) + 1)
        xs = [make_input(shape, seed=s_, outliers=outl).cuda() for s_ in range(3)]
        xs += [xs[i_ % 3].clone() for i_ in range(nb - 3)]
        outs = [ops.quantize(x, 0, 1) for x in xs]
        buf = (ctypes.c_uint64 * (256 * 8))()
        rows = {n_: {"min": [], "mean": [], "max": []} for n_ in names}
        for r in range(reps + 3):
            j = r % nb
            ops.quantize(xs[j], 0, 1, output=outs[j][0], sf=outs[j][1])
            _lib.check(fn(buf))
            if r < 3:
                continue
            t = [[buf[w * 8 + i] for i in range(5)] for w in range(256)]
            t0 = min(x[0] for x in t)
            for i, n_ in enumerate(names):
                col = [(x[i] - t0) * 0.01 for x in t]
                rows[n_]["min"].append(min(col)); rows[n_]["mean"].append(sum(col) / len(col)); rows[n_]["max"].append(max(col))
        res[tag] = {n_: {k_: round(statistics.median(v), 2) for k_, v in d.items()} for n_, d in rows.items()}
        log(f"[timeline] {tag}: us after the first workgroup's entry, min / mean / max over 256 workgroups (median of {reps} launches)")
        for n_ in names:
            d = res[tag][n_]
            log(f"[timeline]   {n_:22s} {d['min']:7.2f} {d['mean']:7.2f} {d['max']:7.2f}")
    print(json.dumps({"quantize_timeline_us": res}))


def run_linear_timeline(ops, reps=12):
    """Per-workgroup phase boundaries of the linear kernels that carry clock stamps (the packed-operand tile
    kernel and the K-split-waves kernel; needs the library built by `python ac4k_kernel_amd/build.py --timeline`,
    loaded through AC4K_NVFP4_LIB): microseconds after the first workgroup's entry at loop entry, loop exit and
    kernel exit (min / mean / max over the workgroups of the last of `reps` launches), shader cycles in the loop."""
    import ctypes
    from ac4k_kernel_amd import _lib
    L = _lib.load()
    fn = getattr(L, "ac4k_debug_linear_timeline", None)
    if fn is None:
        sys.exit("bench.py: this library has no clock stamps; build with `python ac4k_kernel_amd/build.py --timeline` "
                 "and set AC4K_NVFP4_LIB to the library it prints")
    fn.restype, fn.argtypes = ctypes.c_int, [ctypes.c_void_p]
    res = {}
    for (m, n, k, nwg) in ((8192, 8192, 8192, 1024), (128, 14336, 4096, 224), (128, 4096, 14336, 256)):
        aq = ops.quantize(make_input((m, k), seed=0).cuda(), 0, 1)
        bqs = [ops.quantize(make_input((n, k), seed=1 + i, std=0.02).cuda(), 0, 1) for i in range(4)]
        out = torch.empty((m, n), dtype=torch.bfloat16, device="cuda")
        buf = (ctypes.c_uint64 * (8192 * 6))()
        for r in range(reps):
            ops.linear(*aq, *bqs[r % 4], out=out)
        _lib.check(fn(buf))
        rows = [[buf[w * 6 + i] for i in range(6)] for w in range(nwg)]
        t0 = min(x[0] for x in rows)
        tag = f"M{m}_N{n}_K{k}"
        res[tag] = {}
        for name, i in (("entry", 0), ("loop_entry", 1), ("loop_exit", 2), ("exit", 3)):
            col = [(x[i] - t0) * 0.01 for x in rows]
            res[tag][name] = {"min": round(min(col), 2), "mean": round(sum(col) / len(col), 2), "max": round(max(col), 2)}
        loop_us = sum((x[2] - x[1]) * 0.01 for x in rows) / len(rows)
        cyc = sum(x[4] for x in rows) / len(rows)
        res[tag]["loop"] = {"us": round(loop_us, 2), "cycles": round(cyc), "GHz": round(cyc / loop_us / 1e3, 3)}
        log(f"[timeline] {tag}: " + "  ".join(f"{k_} {v}" for k_, v in res[tag].items()))
    print(json.dumps({"linear_timeline_us": res}))


def main():
    global SETTLE_MS
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="all", choices=["all", "linear", "quantize", "traffic", "quantize-timeline", "linear-timeline"])
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS,
                    help="keep the untimed warm-up going for this long (clock ramp); 0 = exactly --warmup calls")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus must be 1")
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    # CPU leg: every host core the process may run on (a container's share can be smaller than
    # os.cpu_count(); both are reported next to the thread count torch actually uses)
    try:
        usable = len(os.sched_getaffinity(0))
    except (AttributeError, OSError):
        usable = os.cpu_count() or 1
    env_cap = os.environ.get("OMP_NUM_THREADS")
    threads = min(usable, int(env_cap)) if env_cap and env_cap.isdigit() and int(env_cap) > 0 else usable
    torch.set_num_threads(max(1, threads))
    HOST.update({"cpu_count": os.cpu_count(), "usable_cores": usable, "omp_num_threads_env": env_cap,
                 "threads": torch.get_num_threads()})
    from ac4k_kernel_amd import ops

    if args.workload == "traffic":
        return run_traffic(ops)
    if args.workload == "quantize-timeline":
        return run_quantize_timeline(ops)
    if args.workload == "linear-timeline":
        return run_linear_timeline(ops)
    check = not args.no_check  # the GEMM checks: fp32 dequantize-matmul with torch ops on the GPU
    # The CPU leg (the only user of oracle/): the oracle timed on the host cores as `cpu_baseline`, and the
    # same oracle as the checker of the quantizers' GPU output.  --no-cpu-baseline skips all of it.
    check_cpu = check and not args.no_cpu_baseline
    S, W = args.steps, args.warmup
    SETTLE_MS = args.settle_ms
    line = {"n_gpus": 1, "steps": S, "warmup": W, "warmup_settle_ms": SETTLE_MS, "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None, "data": "synthetic (seed 0, generated on CPU, cast to bf16)"}
    quant = None
    if args.workload in ("all", "quantize"):
        quant = {
            "cfg2_nvfp4": bench_quantize(ops, (8192, 4096), "nvfp4", S, W, True, check_cpu, key="quantize_nvfp4_8192x4096"),
            "cfg2_fp8e4m3": bench_quantize(ops, (8192, 4096), "fp8e4m3", S, W, True, check_cpu, key="quantize_fp8_8192x4096"),
            "cfg2_int8": bench_quantize(ops, (8192, 4096), "int8", S, W, True, check_cpu, key="quantize_int8_8192x4096"),
            "cfg1_nvfp4": bench_quantize(ops, (4096, 4096), "nvfp4", S, W, False, check_cpu),
        }
        for k_, v in quant.items():
            log(f"[bench] {k_}: {v['ms'] * 1e3:.1f} us  {v['GB/s']:.0f} GB/s  "
                f"({100 * v['roofline']['frac']:.1f}% of HBM peak, {v['rotating_buffers']} buffer sets from HBM; "
                f"{100 * v['three_buffers_cache_assisted']['frac_of_hbm_peak']:.1f}% over three sets that fit the "
                f"memory-side cache)  bit-exact={v['bit_exact_vs_oracle']}"
                + (f"  kernel alone with the global scale given: {v['global_scale_given']['ms'] * 1e3:.1f} us "
                   f"({100 * v['global_scale_given']['frac_of_hbm_peak']:.1f}%)" if "global_scale_given" in v else ""))
        if not args.no_cpu_baseline:
            quant["cpu_baseline"] = cpu_quantize_baseline((8192, 4096), True)
            log(f"[bench] cpu quantize oracle: {quant['cpu_baseline']['value']:.2f} GB/s on "
                f"{quant['cpu_baseline']['cores']} threads")
    if args.workload in ("all", "linear"):
        lin = bench_linear(ops, 8192, 8192, 8192, S, W, check=check, key="linear_8192", with_image=True)
        log(f"[bench] {lin['workload']}: {lin['ms']:.3f} ms  {lin['TFLOP/s']:.1f} TFLOP/s "
            f"({100 * lin['roofline']['frac']:.1f}% of MFMA peak)  ok={lin['within_1e-2_of_fp32_dequant_matmul']}")
        wi = lin["weight_image"]
        log(f"[bench]   same linear on a pre-packed weight image: {wi['ms']:.3f} ms  {wi['TFLOP/s']:.1f} TFLOP/s "
            f"({100 * wi['TFLOP/s'] / MFMA_PEAK_TFLOPS:.1f}% of MFMA peak; plain layout re-timed after it: "
            f"{wi['plain_layout_ms_after']:.3f} ms)  bit-identical={wi['bit_identical_to_plain_layout']}")
        line["linear_8192_weight_image_tflops"] = wi["TFLOP/s"]
        line["linear_8192_weight_image_frac"] = wi["TFLOP/s"] / MFMA_PEAK_TFLOPS
        line["linear_8192_weight_image_bit_identical"] = wi["bit_identical_to_plain_layout"]
        line.update({"metric": "nvfp4_linear_tflops", "value": lin["TFLOP/s"], "unit": "TFLOP/s",
                     "ms_per_step": lin["ms"], "dtype": "fp4 x e4m3 decoded exactly to fp16, fp32 accumulate",
                     "config": {"workload": lin["workload"]}, "roofline": lin["roofline"],
                     "parity": lin["within_1e-2_of_fp32_dequant_matmul"]})
        if not args.no_cpu_baseline:
            line["cpu_baseline"] = cpu_linear_baseline(8192, 8192)
            log(f"[bench] cpu linear oracle: {line['cpu_baseline']['value']:.3f} TFLOP/s")
        if args.workload == "all":
            line["shader_clock"] = shader_clock_under_load(ops)
            mhz = line["shader_clock"]["under_load_mhz"]
            if mhz:  # the same MFMA count per clock at the clock the power limit leaves
                line["shader_clock"]["peak_at_this_clock_TFLOP/s"] = MFMA_PEAK_TFLOPS * mhz / 2400.0
                line["shader_clock"]["frac_of_peak_at_this_clock"] = lin["TFLOP/s"] / (MFMA_PEAK_TFLOPS * mhz / 2400.0)
            log(f"[bench] shader clock: {mhz} MHz under the 8192^3 linear, "
                f"{line['shader_clock']['before_mhz']} MHz before it ({line['shader_clock']['source']}); "
                f"the {MFMA_PEAK_TFLOPS:.0f} TFLOP/s peak assumes 2400 MHz"
                + (f"; {100 * line['shader_clock']['frac_of_peak_at_this_clock']:.1f}% of the peak at this clock" if mhz else ""))
            line["vendor_dense_gemm"] = vendor_gemm_yardstick(S, W)
            log(f"[bench] yardstick, torch.matmul 8192^3 on already dense operands: "
                f"{line['vendor_dense_gemm']['bf16_TFLOP/s']:.0f} TFLOP/s bf16, "
                f"{line['vendor_dense_gemm']['fp16_TFLOP/s']:.0f} TFLOP/s fp16")
            shapes = {"cfg3_4096": bench_linear(ops, 4096, 4096, 4096, S, W, check=check, with_image=True)}
            for (n, k) in ((14336, 4096), (4096, 14336)):
                for m in (16, 128, 2048, 8192):
                    shapes[f"cfg4_M{m}_N{n}_K{k}"] = bench_linear(ops, m, n, k, S, W, wstd=0.02, check=check,
                                                                  with_quantize=True, with_image=True,
                                                                  key=f"decode_linear_M{m}_N{n}_K{k}" if m <= 128 else None)
            for m in (1, 8, 32):  # configuration 5 with the activation already quantized (linear alone)
                shapes[f"cfg5_M{m}_linear_alone"] = bench_linear(ops, m, 28672, 8192, S, W, wstd=0.02, check=check,
                                                                 with_image=True, key=f"decode_linear_M{m}")
            for k_, v in shapes.items():
                wq_ = v["ms_with_activation_quantize"]
                log(f"[bench] {k_}: {v['ms'] * 1e3:.1f} us  {v['TFLOP/s']:.1f} TFLOP/s  {v['GB/s']:.0f} GB/s  "
                    f"{100 * v['roofline']['frac']:.1f}% of {v['roofline']['bound']} peak  "
                    f"ok={v['within_1e-2_of_fp32_dequant_matmul']}"
                    + ("" if wq_ is None else f"  with activation quantize {wq_ * 1e3:.1f} us")
                    + ("" if v["weight_image"] is None else
                       f"  on a weight image {v['weight_image']['ms'] * 1e3:.1f} us "
                       f"(bit-identical={v['weight_image']['bit_identical_to_plain_layout']})"))
            line["linear_shapes"] = shapes
            dec = {f"cfg5_M{m}": bench_decode(ops, m, 28672, 8192, S, W, check, key=f"decode_fused_M{m}") for m in (1, 8, 32)}
            for k_, v in dec.items():
                log(f"[bench] {k_}: {v['ms'] * 1e3:.1f} us  {v['GB/s']:.0f} GB/s "
                    f"({100 * v['roofline']['frac']:.1f}% of HBM peak)  ok={v['equals_quantize_then_linear_within_1e-2']}")
            line["decode"] = dec
            lay = bench_quantize_layouts(ops, S, W)
            for k_, v in lay.items():
                log(f"[bench] quantize layout {k_}: {v['ms'] * 1e3:.1f} us  {v['GB/s']:.0f} GB/s")
            line["quantize_layouts"] = lay
            att = bench_attention(ops, 1, 16384, 40, 128, max(3, S // 10), 2, check=check)
            log(f"[bench] {att['workload']}: kernel {att['kernel_ms']:.2f} ms  {att['kernel_TFLOP/s']:.0f} TFLOP/s "
                f"({100 * att['roofline']['frac']:.1f}% of MFMA peak), with the three quantizes "
                f"{att['with_quantize_ms']:.2f} ms  ok={att['within_reference_tolerance_of_fp32_attention']}")
            line["attention"] = att
            att8 = bench_attention(ops, 1, 16384, 40, 128, max(3, S // 10), 2, check=check, precision="int8+fp8e4m3")
            log(f"[bench] {att8['workload']}: kernel {att8['kernel_ms']:.2f} ms  {att8['kernel_TFLOP/s']:.0f} TFLOP/s, "
                f"with its quantizers {att8['with_quantize_ms']:.2f} ms  ok={att8['within_reference_tolerance_of_fp32_attention']}")
            line["attention_int8_x_fp8"] = att8
            epi = bench_linear_epilogues(ops, S, W)
            log("[bench] linear 8192^3 by output/bias dtype, TFLOP/s: "
                + ", ".join(f"{k_} {v['TFLOP/s']:.0f}" for k_, v in epi.items()))
            line["linear_epilogues"] = epi
            # the shapes the reference itself times (test/test_linear_tflops.py:190-203), M x N x K
            refs = {}
            for (m, n, k) in ((75600, 5120, 5120), (75600, 13824, 5120), (75600, 5120, 6912), (75600, 5120, 13824)):
                refs[f"M{m}_N{n}_K{k}"] = bench_linear(ops, m, n, k, max(5, S // 3), W, wstd=0.02, check=check, gen_on_gpu=True)
                torch.cuda.empty_cache()
            for k_, v in refs.items():
                log(f"[bench] ref shape {k_}: {v['ms']:.3f} ms  {v['TFLOP/s']:.1f} TFLOP/s  "
                    f"{100 * v['roofline']['frac']:.1f}% of MFMA peak  ok={v['within_1e-2_of_fp32_dequant_matmul']}")
                line[f"linear_{k_}_tflops"] = v["TFLOP/s"]
                line[f"linear_{k_}_frac"] = v["roofline"]["frac"]
                line[f"linear_{k_}_ok"] = v["within_1e-2_of_fp32_dequant_matmul"]
            line["ref_shapes"] = refs
        if quant is not None:
            line["quantize"] = quant
    else:
        q = quant["cfg2_nvfp4"]
        line.update({"metric": "nvfp4_quantize_gbs", "value": q["GB/s"], "unit": "GB/s", "ms_per_step": q["ms"],
                     "dtype": "bf16 -> e2m1 + e4m3 scales (fp32 arithmetic)", "config": {"workload": q["workload"]},
                     "roofline": q["roofline"], "parity": q["bit_exact_vs_oracle"], "quantize": quant})
        if "cpu_baseline" in quant:
            line["cpu_baseline"] = quant["cpu_baseline"]
    # The quantize half of the metric as flat scalar keys of the line, and a short summary as the LAST
    # lines of stderr (what a captured tail keeps).
    summary = []
    if quant is not None:
        for key, tag in (("cfg1_nvfp4", "quantize_nvfp4_4096x4096"), ("cfg2_nvfp4", "quantize_nvfp4_8192x4096"),
                         ("cfg2_fp8e4m3", "quantize_fp8_8192x4096"), ("cfg2_int8", "quantize_int8_8192x4096")):
            q = quant[key]
            line[f"{tag}_gbs"] = q["GB/s"]
            line[f"{tag}_frac"] = q["roofline"]["frac"]
            line[f"{tag}_us"] = q["ms"] * 1e3
            line[f"{tag}_bit_exact"] = q["bit_exact_vs_oracle"]
            summary.append(f"{tag}: {q['ms'] * 1e3:.1f} us  {q['GB/s']:.0f} GB/s  frac {q['roofline']['frac']:.3f} of 8 TB/s  "
                           f"bit_exact={q['bit_exact_vs_oracle']}")
            if "global_scale_given" in q:
                g_ = q["global_scale_given"]
                line[f"{tag}_kernel_alone_frac"] = g_["frac_of_hbm_peak"]
                summary[-1] += f"  (kernel alone, scale given: {g_['ms'] * 1e3:.1f} us, frac {g_['frac_of_hbm_peak']:.3f})"
        if "cpu_baseline" in quant:
            c = quant["cpu_baseline"]
            line["quantize_cpu_baseline_gbs"] = c["value"]
            summary.append(f"quantize cpu oracle: {c['value']:.2f} GB/s on {c['cores']} threads "
                           f"(os.cpu_count {HOST.get('cpu_count')}, usable {HOST.get('usable_cores')}, "
                           f"OMP_NUM_THREADS {HOST.get('omp_num_threads_env')})")
    if "roofline" in line and line.get("unit") == "TFLOP/s":
        summary.append(f"linear 8192^3: {line['ms_per_step']:.3f} ms  {line['value']:.1f} TFLOP/s  "
                       f"frac {line['roofline']['frac']:.3f} of 2.5 PFLOP/s  ok={line.get('parity')}")
    for k_ in ("decode", "linear_shapes"):
        if k_ in line:
            summary.append(k_ + ": " + "  ".join(f"{n_.split('_', 1)[1]} {v['ms'] * 1e3:.1f}us/{v['roofline']['frac']:.2f}"
                                                 for n_, v in line[k_].items()))
    if "linear_shapes" in line:
        summary.append("weight image / plain layout, us: " + "  ".join(
            f"{n_.split('_', 1)[1]} {v['weight_image']['ms'] * 1e3:.1f}/{v['ms'] * 1e3:.1f}"
            for n_, v in line["linear_shapes"].items() if v.get("weight_image")))
    if "linear_8192_weight_image_tflops" in line:
        summary.append(f"linear 8192^3 on a weight image: {line['linear_8192_weight_image_tflops']:.1f} TFLOP/s  "
                       f"frac {line['linear_8192_weight_image_frac']:.3f}  "
                       f"bit_identical={line['linear_8192_weight_image_bit_identical']}")
    if "ref_shapes" in line:
        summary.append("ref shapes: " + "  ".join(f"{n_} {v['TFLOP/s']:.0f}TF/{v['roofline']['frac']:.2f}"
                                                  for n_, v in line["ref_shapes"].items()))
    line["host"] = dict(HOST)
    print(json.dumps(line), flush=True)
    log("[bench] ---- summary (time, throughput, fraction of the roofline) ----")
    for ln in summary:
        log("[bench] " + ln)


if __name__ == "__main__":
    main()

"""Builds libac4k_nvfp4.so (the C-ABI library) for gfx950 with hipcc, in-tree.

    python ac4k_kernel_amd/build.py            # build if sources are newer
    python ac4k_kernel_amd/build.py --force

(run it as a script: `python -m ac4k_kernel_amd.build` would import the package, which loads
the library that is about to be rebuilt)
"""
from __future__ import annotations

import os
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libac4k_nvfp4.so")
SOURCES = ["capi.hip", "quantize.hip", "linear.hip", "attention.hip"]
HEADERS = [os.path.join(CSRC, "ac4k_common.h"), os.path.join(ROOT, "include", "ac4k_nvfp4.h")]

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    # the quantizer spec has separate fp32 multiplies: never contract them into FMAs
    "-ffp-contract=off",
    # packed-fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-fvisibility=hidden", "-Wall", "-Wno-unused-command-line-argument",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def needs_build() -> bool:
    if not os.path.exists(LIB_PATH):
        return True
    t = os.path.getmtime(LIB_PATH)
    deps = [os.path.join(CSRC, s) for s in SOURCES] + HEADERS + [os.path.abspath(__file__)]
    return any(os.path.getmtime(d) > t for d in deps)


OBJ_DIR = os.path.join(PKG_DIR, "_obj")


def _run(cmd, verbose):
    if verbose:
        print("[ac4k build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)


def build(force: bool = False, verbose: bool = True, extra_flags=(), out: str = LIB_PATH) -> str:
    """One object per source file, compiled side by side, then one link.  An object is reused when it
    is newer than its source, the headers and this file (only for the default flags and output)."""
    if not force and out == LIB_PATH and not needs_build():
        return LIB_PATH
    from concurrent.futures import ThreadPoolExecutor
    reuse = not force and out == LIB_PATH and not extra_flags
    tag = "" if out == LIB_PATH else "." + os.path.splitext(os.path.basename(out))[0]
    os.makedirs(OBJ_DIR, exist_ok=True)
    compile_flags = [f for f in FLAGS if f != "-shared"] + list(extra_flags)
    common = HEADERS + [os.path.abspath(__file__)]
    jobs, objs = [], []
    for src_name in SOURCES:
        src = os.path.join(CSRC, src_name)
        obj = os.path.join(OBJ_DIR, src_name + tag + ".o")
        objs.append(obj)
        fresh = reuse and os.path.exists(obj) and all(os.path.getmtime(d) < os.path.getmtime(obj) for d in [src] + common)
        if not fresh:
            jobs.append([HIPCC] + compile_flags + ["-c", src, "-o", obj])
    with ThreadPoolExecutor(max_workers=max(1, len(jobs))) as pool:
        list(pool.map(lambda c: _run(c, verbose), jobs))
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-fvisibility=hidden"] + objs + ["-o", out], verbose)
    return out


TIMELINE_LIB_PATH = os.path.join(PKG_DIR, "libac4k_nvfp4_timeline.so")


def build_timeline(verbose: bool = True) -> str:
    """The same sources with the kernels' clock stamps compiled in (profiling aid, not the product):
    load it with AC4K_NVFP4_LIB=<path> for `bench.py --workload quantize-timeline` / `linear-timeline`."""
    return build(force=True, verbose=verbose, extra_flags=["-DAC4K_ONEPASS_TIMELINE", "-DAC4K_LINEAR_TIMELINE"], out=TIMELINE_LIB_PATH)


if __name__ == "__main__":
    if "--timeline" in sys.argv:
        print(build_timeline())
    else:
        print(build(force="--force" in sys.argv))

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
SOURCES = ["capi.hip", "quantize.hip", "linear.hip"]
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


def build(force: bool = False, verbose: bool = True, extra_flags=(), out: str = LIB_PATH) -> str:
    if not force and out == LIB_PATH and not needs_build():
        return LIB_PATH
    cmd = [HIPCC] + FLAGS + list(extra_flags) + [os.path.join(CSRC, s) for s in SOURCES] + ["-o", out]
    if verbose:
        print("[ac4k build]", " ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    log = "\n".join(l for l in res.stdout.splitlines() if "is not a recognized feature for this target" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + log)
    if verbose and log.strip():
        print(log)
    return out


if __name__ == "__main__":
    print(build(force="--force" in sys.argv))

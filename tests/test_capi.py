"""The C-ABI library: loads, exports every function include/ac4k_nvfp4.h declares, reports
attributes, and rejects bad arguments before touching the GPU (no compute calls here)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "ac4k_nvfp4.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(ac4k_[a-z0-9_]+)\s*\(", text)))


def test_header_and_loader_agree():
    from ac4k_kernel_amd import _lib
    names = declared_functions()
    assert len(names) >= 18
    assert sorted(_lib.SIGNATURES) == names
    lib = _lib.load()
    for n in names:
        assert hasattr(lib, n), n


def test_attributes():
    import ac4k_kernel_amd as pkg
    assert pkg.get_backend() == "rocm" and pkg.get_arch() == "gfx950"
    assert pkg.get_info() == {"version": "0.1.0", "backend": "rocm", "arch": "gfx950"}
    from ac4k_kernel_amd import ops
    for name in ["quantize", "linear", "quantize_nvfp4", "quantize_fp8", "quantize_int8", "linear_nvfp4"]:
        assert callable(getattr(ops, name))


def test_product_does_not_import_oracle():
    # the shipped package must not reach into oracle/ (it is the checker, not the product)
    pkg = os.path.join(ROOT, "ac4k_kernel_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                src = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in src, os.path.join(dirpath, f)


def test_argument_rejection_without_gpu():
    from ac4k_kernel_amd import _lib
    lib = _lib.load()
    one = ctypes.c_void_p(16)  # never dereferenced: every call below is rejected during validation
    rc = lib.ac4k_quantize_nvfp4(None, one, one, one, 1, 1, 4, 64, 0, 0, 64, 1, 0, None)
    assert rc != 0 and b"null" in lib.ac4k_last_error()
    rc = lib.ac4k_quantize_nvfp4(one, one, one, one, 1, 1, 0, 64, 0, 0, 64, 1, 0, None)
    assert rc != 0 and b"positive" in lib.ac4k_last_error()
    rc = lib.ac4k_linear_nvfp4(one, 0, one, one, one, one, one, one, None, 0, 4, 4, 24, None)
    assert rc != 0 and b"multiple of 16" in lib.ac4k_last_error()
    rc = lib.ac4k_linear_nvfp4(one, 7, one, one, one, one, one, one, None, 0, 4, 4, 64, None)
    assert rc != 0 and b"bfloat16, half or float" in lib.ac4k_last_error()
    # a sliced view (rows of 64 taken out of rows of 128) is not dense: the global scale would be taken
    # over the wrong elements, so the one-call quantizer refuses it; so it does a zero stride on a real dim
    rc = lib.ac4k_quantize_nvfp4_bf16(one, one, one, one, 1, 1, 4, 64, 0, 0, 128, 1, 0, 2688.0, None)
    assert rc != 0 and b"dense" in lib.ac4k_last_error()
    rc = lib.ac4k_quantize_nvfp4_bf16(one, one, one, one, 1, 3, 4, 64, 0, 0, 64, 1, 0, 2688.0, None)
    assert rc != 0 and b"strides must be positive" in lib.ac4k_last_error()
    # tuning values outside the instantiated kernels are refused, zeros are accepted
    assert lib.ac4k_set_linear_tuning(4, 1, 1, 0, 0) != 0 and b"tile plan" in lib.ac4k_last_error()
    assert lib.ac4k_set_linear_tuning(0, 0, 0, 100, 0) != 0 and b"skinny_ks" in lib.ac4k_last_error()
    assert lib.ac4k_set_linear_tuning(0, 0, 0, 0, 4) != 0 and b"decode_kernel" in lib.ac4k_last_error()
    # a rejected call leaves every earlier field alone: here the decode kernel choice is valid, skinny_ks is not,
    # and the plan of a decode-sized shape stays what the library picks on its own
    before = lib.ac4k_linear_nvfp4_skinny_workspace_bytes(4, 4096, 14336)
    assert lib.ac4k_set_linear_tuning(0, 0, 0, 100, 2) != 0
    assert lib.ac4k_linear_nvfp4_skinny_workspace_bytes(4, 4096, 14336) == before
    assert lib.ac4k_set_linear_tuning(0, 0, 0, 0, 0) == 0
    assert lib.ac4k_debug_last_quantize_path() in (0, 1, 2, 3)
    # K <= 0 never selects a weight-streaming plan, and the workspace entry points say what is wrong
    assert lib.ac4k_linear_nvfp4_skinny_workspace_bytes(8, 1024, 0) == 0
    assert lib.ac4k_linear_nvfp4_skinny_workspace_bytes(8, 1024, -256) == 0
    rc = lib.ac4k_linear_nvfp4_skinny(one, 0, one, one, one, one, one, one, None, 0, 8, 1024, 0, one, 256, None)
    assert rc != 0 and b"positive" in lib.ac4k_last_error()
    rc = lib.ac4k_linear_nvfp4_skinny_static(one, 0, one, one, one, one, one, one, None, 0, 8, 1024, -256, None)
    assert rc != 0 and b"positive" in lib.ac4k_last_error()
    rc = lib.ac4k_linear_nvfp4_fused_bf16(one, 0, one, one, one, one, one, one, one, None, 0, 8, 1024, 0, one, 256, None)
    assert rc != 0 and b"positive" in lib.ac4k_last_error()
    rc = lib.ac4k_linear_nvfp4_fused_bf16(one, 0, one, one, one, one, one, one, one, None, 0, 64, 4, 64, one, 0, None)
    assert rc != 0 and b"1 <= M <= 32" in lib.ac4k_last_error()
    with pytest.raises(RuntimeError):
        _lib.check(rc)


def test_python_checks_without_gpu():
    import torch
    from ac4k_kernel_amd import ops
    x = torch.zeros((4, 64), dtype=torch.bfloat16)
    with pytest.raises(AssertionError):
        ops.quantize(x, 0, 0)
    with pytest.raises(AssertionError):
        ops.quantize(x, 0, 1, precision="fp4")
    with pytest.raises(AssertionError):
        ops.quantize(torch.zeros(8, dtype=torch.bfloat16), 0, 1)
    with pytest.raises(RuntimeError):  # CPU tensor: "must be a CUDA tensor"
        ops.quantize_fp8(torch.empty((4, 64), dtype=torch.float8_e4m3fn), torch.empty(16), x,
                         torch.tensor(448.0), 0, 1, False)


def test_reference_import_lines_resolve():
    """The import lines of the reference's callers (test/test_quantize_bench.py:7,
    test/test_linear_bench.py:4) resolve to this library through the `ac4k_kernel` alias package."""
    import ac4k_kernel
    import ac4k_kernel_amd
    from ac4k_kernel.ops import attention, linear, quantize
    from ac4k_kernel.ops.attention import mha_int8_x_fp8_fwd, mha_nvfp4_fwd
    from ac4k_kernel.ops.linear import Ac4kLinearOp
    from ac4k_kernel.ops.quant import Ac4kQuantizeOp
    import ac4k_kernel._rocm_ops as binding
    assert ac4k_kernel.get_backend() == "rocm" and ac4k_kernel.get_arch() == "gfx950"
    assert ac4k_kernel.get_info() == ac4k_kernel_amd.get_info()
    assert quantize is ac4k_kernel_amd.ops.quantize and linear is ac4k_kernel_amd.ops.linear
    assert attention is ac4k_kernel_amd.ops.attention and mha_nvfp4_fwd is binding.mha_nvfp4_fwd
    assert mha_int8_x_fp8_fwd is binding.mha_int8_x_fp8_fwd
    assert binding is ac4k_kernel_amd._rocm_ops and binding.__backend__ == "rocm"
    assert issubclass(Ac4kLinearOp, __import__("torch").nn.Module) and Ac4kQuantizeOp is not None
    for name in ("quantize_nvfp4", "quantize_fp8", "quantize_int8", "linear_nvfp4"):
        assert getattr(ac4k_kernel, name) is getattr(ac4k_kernel_amd, name)
        assert getattr(ac4k_kernel.ops, name) is getattr(ac4k_kernel_amd.ops, name)
    # the alias must not pull in the checker either
    for f in ("__init__.py", os.path.join("ops", "__init__.py")):
        assert "oracle" not in open(os.path.join(ROOT, "ac4k_kernel", f)).read()

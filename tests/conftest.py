import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def make_input(shape, seed=0, outliers=False, dist="normal", std=1.0):
    """Synthetic bf16 input generated on the CPU so oracle and GPU see identical bits."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32) * std
    if outliers:
        mask = torch.rand(shape, generator=g) < 0.001
        x = torch.where(mask, x * 20.0, x)
    return x.to(torch.bfloat16)


@pytest.fixture
def linear_tuning():
    """Forces a tile plan / K slice of the linear kernels for one test (ac4k_set_linear_tuning) and gives
    the choice back to the library afterwards."""
    from ac4k_kernel_amd import _lib
    lib = _lib.load()

    def force(mi=0, nj=0, splits=0, skinny_ks=0, decode_kernel=0):
        _lib.check(lib.ac4k_set_linear_tuning(mi, nj, splits, skinny_ks, decode_kernel))

    yield force
    lib.ac4k_set_linear_tuning(0, 0, 0, 0, 0)

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

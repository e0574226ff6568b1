import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no HIP device visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def rand(shape, seed, dtype=torch.float32, scale=1.0):
    """Seeded N(0,1)*scale drawn in fp32 on the CPU, then cast — the input recipe of every config."""
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype)


def rand_qkv(shape, seed, dtype=torch.float32, scale=1.0, n=3):
    """q, k, v (and optionally more) drawn in that order from one generator."""
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(shape, generator=g, dtype=torch.float32) * scale).to(dtype) for _ in range(n)]
